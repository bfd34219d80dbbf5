"""GPU parity: every call goes through the C-ABI library and is compared with the CPU oracle on the
same seeded buffers.  Bounds: normwise max|Z - Zref| / max|Zref| <= 1e-5 (fp32), 1e-12 (fp64); integer-valued
inputs additionally use the reference harness's element-wise rule (reference tests/testBase.h:136-146)."""
import numpy as np
import pytest

from oracle import kron_oracle as ko
from tests.gpu_util import TOL, make_case, normwise, oracle_answer, run_gpu
from tests.kron_ref import eq_val

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fk():
    import fastkron_amd
    h = fastkron_amd.FastKron()
    yield h
    h.close()


def check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=0.0, seed=0, **kw):
    run_kw = {k: kw.pop(k) for k in ("use_temp2", "strided", "y_is_z") if k in kw}
    integer = kw.get("integer", False)
    X, Fs, Y = make_case(mm, M, Ps, Qs, dt, seed=seed, with_y=(beta != 0), **kw)
    kw.pop("integer", None)
    want = oracle_answer(mm, M, Ps, Qs, X, Fs, Y, alpha, beta, **kw)
    got, e = run_gpu(fk, mm, M, Ps, Qs, X, Fs, Y, alpha, beta, **kw, **run_kw)
    assert e == 0, f"fastKronError {e}"
    assert not np.isnan(got).any()
    err = normwise(got, want)
    assert err <= TOL[dt], f"normwise error {err:.3e}"
    if integer:
        assert eq_val(got, want)


# shape matrix of reference tests/src/general-tests-NN.cpp:52-100 (square, non-square, distinct), sized so
# that the oracle answers in seconds
SQUARE = [(16, [p] * n) for p, n in [(1, 4), (2, 8), (3, 5), (4, 6), (5, 4), (6, 3), (8, 4), (12, 3), (16, 3),
                                     (24, 2), (31, 2), (32, 3), (50, 2), (55, 2), (62, 2), (64, 2), (127, 2),
                                     (128, 2), (129, 1), (255, 1), (297, 1), (512, 1)]]
NONSQUARE = [(16, [1, 1, 1], [4, 4, 4]), (16, [5, 5, 5], [1, 1, 1]), (16, [2] * 5, [4] * 5),
             (16, [31, 31], [63, 63]), (16, [63, 63], [31, 31]), (8, [297], [127]), (8, [127], [297]),
             (16, [2, 5, 6], [3, 2, 4]), (16, [14, 19], [15, 13]), (4, [8, 8], [32, 32]), (4, [32, 32], [8, 8])]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M,Ps", SQUARE)
def test_mkm_square(fk, M, Ps, dt):
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=2.0, beta=1.0, integer=(max(Ps) ** len(Ps) < 4096))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M,Ps,Qs", NONSQUARE)
def test_mkm_nonsquare(fk, M, Ps, Qs, dt):
    check(fk, ko.MKM, M, Ps, Qs, dt, alpha=2.0, beta=1.0)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M", [1, 3, 16, 20])
@pytest.mark.parametrize("Ps,Qs", [([4] * 4, [4] * 4), ([8, 8, 8], [8, 8, 8]), ([2, 5, 6], [3, 2, 4]),
                                   ([32, 32], [16, 16]), ([31], [63])])
def test_kmm(fk, M, Ps, Qs, dt):
    check(fk, ko.KMM, M, Ps, Qs, dt, alpha=2.0, beta=1.0)


@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
@pytest.mark.parametrize("opX,opFs", [(ko.OP_T, ko.OP_T), (ko.OP_T, ko.OP_N), (ko.OP_N, ko.OP_T)])
@pytest.mark.parametrize("M,Ps,Qs", [(16, [8, 8, 8], [8, 8, 8]), (13, [2, 5, 6], [3, 2, 4]), (17, [31], [63]),
                                     (1, [4, 4, 4], [4, 4, 4])])
def test_transposed_operands(fk, mm, opX, opFs, M, Ps, Qs):
    """reference tests/src/general-tests-TT.cpp:36-83"""
    check(fk, mm, M, Ps, Qs, np.float32, alpha=2.0, beta=1.0, opX=opX, opFs=opFs)
    check(fk, mm, M, Ps, Qs, np.float64, alpha=2.0, beta=1.0, opX=opX, opFs=opFs)


@pytest.mark.parametrize("mm,M,Ps,dt", [(ko.MKM, 16, [8] * 5, np.float32), (ko.MKM, 4, [16] * 4, np.float32),
                                        (ko.MKM, 100, [32] * 3, np.float32), (ko.MKM, 600, [64] * 2, np.float64),
                                        (ko.MKM, 2, [16] * 5, np.float32), (ko.MKM, 5, [16] * 3, np.float64),
                                        (ko.KMM, 64, [4] * 6, np.float32), (ko.KMM, 40, [16] * 2, np.float64),
                                        (ko.MKM, 13, [12] * 3, np.float32), (ko.MKM, 7, [4] * 8, np.float32)])
def test_transposed_x_ahead_of_the_whole_row_kernels(fk, mm, M, Ps, dt):
    """op(X) = T on shapes whose fast kernels need contiguous rows: X is transposed into a temporary first
    (reference general-tests-TT.cpp:36-83 runs its whole shape list with transposed operands)."""
    check(fk, mm, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=71, opX=ko.OP_T, opFs=ko.OP_T)
    plan = fk.last_plan()
    if mm == ko.KMM and Ps[-1] >= 16:
        # KMM layout, a copy that saves no launch: the padded step reads the transposed X in the first launch instead
        assert not plan[0][2].startswith("transpose_"), plan
        return
    if mm == ko.KMM:
        # small factors: the GeKMM runs as the GeMKM of the transposed buffer, the result is transposed into Z
        assert plan[0][2].startswith("mkm_") and plan[-1][2].endswith("_z"), plan
    else:
        assert plan[0][2].startswith("transpose_"), plan
    check(fk, mm, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=72, opX=ko.OP_T, opFs=ko.OP_N, batch=3, share_f=True)
    check(fk, mm, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=73, opX=ko.OP_T, opFs=ko.OP_N, batch=2)


@pytest.mark.parametrize("M,Ps,dt", [(64, [8] * 5, np.float32), (16, [8] * 3, np.float32), (100, [16] * 3, np.float32),
                                     (3, [16] * 4, np.float32), (256, [32] * 3, np.float32), (64, [16] * 3, np.float64),
                                     (68, [8] * 4, np.float64), (128, [4, 8, 16], np.float32), (20, [8] * 6, np.float32)])
def test_gekmm_with_transposed_x_as_gemkm(fk, M, Ps, dt):
    """GeKMM with op(X) = T and square factors up to 32x32: the buffer is the X of a GeMKM with transposed factors; the
    whole-row GeMKM kernels run on it and one transposition, which also adds beta * Y, writes Z (column counts with and
    without whole 16-byte tiles, chains that need the two-part plan, batches, shared factors and a shared Y)."""
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=81, opX=ko.OP_T, opFs=ko.OP_T)
    plan = fk.last_plan()
    assert not plan[0][2].startswith(("transpose_", "kmm_")) and plan[-1][2].endswith("_z"), plan
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=2.0, beta=0.0, seed=82, opX=ko.OP_T, opFs=ko.OP_N)
    assert fk.last_plan()[-1][2].endswith("_z"), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=83, opX=ko.OP_T, opFs=ko.OP_N, batch=3, share_f=True)
    assert fk.last_plan()[-1][2].endswith("_z"), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=-1.0, seed=84, opX=ko.OP_T, opFs=ko.OP_T, batch=2, share_y=True)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=85, opX=ko.OP_T, opFs=ko.OP_N, integer=True)
    # without a second temporary the call keeps to the GeKMM kernels
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.5, seed=86, opX=ko.OP_T, opFs=ko.OP_N, use_temp2=False)
    assert not fk.last_plan()[-1][2].endswith("_z"), fk.last_plan()


@pytest.mark.parametrize("M,Ps", [(16, [8] * 7), (20, [16] * 5)])
def test_large_gekmm_with_few_columns_as_gemkm(fk, M, Ps):
    """fp32 GeKMM with fewer than 64 columns, square factors up to 32x32 and 64 MB of X or more: X is transposed into a
    temporary, the GeMKM kernels run on it and the result is transposed into Z (with beta * Y)."""
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=91)
    plan = fk.last_plan()
    assert plan[0][2].endswith("_x") and plan[-1][2].endswith("_z"), plan
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=92, opFs=ko.OP_T)
    assert fk.last_plan()[-1][2].endswith("_z"), fk.last_plan()


@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
@pytest.mark.parametrize("share_f,share_y", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("M,Ps,Qs", [(16, [32] * 3, [16] * 3), (8, [32, 32], [64, 64]), (5, [3, 4], [2, 5])])
def test_strided_batched(fk, mm, share_f, share_y, M, Ps, Qs):
    """batch combinations of reference tests/src/general-tests-NN.cpp:94-100"""
    check(fk, mm, M, Ps, Qs, np.float32, alpha=1.0, beta=1.0, batch=3, share_f=share_f, share_y=share_y)
    check(fk, mm, M, Ps, Qs, np.float64, alpha=1.0, beta=1.0, batch=2, share_f=share_f, share_y=share_y)


@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
@pytest.mark.parametrize("Ps,Qs", [([4, 4, 4], [4, 4, 4]), ([4] * 4, [4] * 4), ([8, 8], [8, 8]), ([2] * 5, [3] * 5)])
def test_single_temporary_uses_z_as_scratch(fk, mm, Ps, Qs):
    check(fk, mm, 8, Ps, Qs, np.float32, alpha=1.5, beta=0.5, use_temp2=False)


def test_single_temporary_with_z_smaller_than_an_intermediate_is_rejected(fk):
    """A shrinking chain needs both temporaries (include/fastkron.h: temp2 is required when Z is smaller
    than the temporary); with one, the call must fail instead of writing past Z."""
    fk.set_options(fusion=False)
    try:
        X, Fs, _ = make_case(ko.MKM, 4, [16] * 3, [2] * 3, np.float32, with_y=False)
        _, e = run_gpu(fk, ko.MKM, 4, [16] * 3, [2] * 3, X, Fs, None, 1.0, 0.0, use_temp2=False)
        assert e == 4
    finally:
        fk.set_options(fusion=True)


def test_alpha_beta_and_null_y(fk):
    check(fk, ko.MKM, 8, [8, 8], [8, 8], np.float32, alpha=-0.75, beta=0.0)
    check(fk, ko.MKM, 8, [8, 8], [8, 8], np.float64, alpha=0.0, beta=3.0)
    # beta != 0 with Y == NULL: the beta term is skipped, as in the reference kernels
    X, Fs, _ = make_case(ko.MKM, 4, [4, 4], [4, 4], np.float32, with_y=False)
    want = oracle_answer(ko.MKM, 4, [4, 4], [4, 4], X, Fs, None, 2.0, 0.0)
    got, e = run_gpu(fk, ko.MKM, 4, [4, 4], [4, 4], X, Fs, None, 2.0, 5.0)
    assert e == 0 and normwise(got, want) <= 1e-5


@pytest.mark.parametrize("mm,name", [(ko.MKM, "mkm"), (ko.KMM, "kmm")])
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_forward_keeps_every_intermediate(fk, mm, name, dt):
    import torch
    M, Ps, Qs = 6, [4, 3, 5], [2, 4, 3]
    X, Fs, _ = make_case(mm, M, Ps, Qs, dt, with_y=False)
    Zw, Iw = oracle_answer(mm, M, Ps, Qs, X, Fs, None, 1.0, 0.0, keep_intermediates=True)
    ye, sizes = fk.sizes_forward(M, Ps, Qs)
    dev = "cuda:0"
    tX = torch.from_numpy(X).to(dev)
    tFs = [torch.from_numpy(f).to(dev) for f in Fs]
    Z = torch.full((ye,), float("nan"), dtype=tX.dtype, device=dev)
    inters = [torch.full((s,), float("nan"), dtype=tX.dtype, device=dev) for s in sizes]
    e = fk.xforward(name, M, Ps, Qs, tX, tFs, Z, inters)
    torch.cuda.synchronize()
    assert e == 0
    assert normwise(Z.cpu().numpy(), Zw) <= TOL[dt]
    for got, want in zip(inters, Iw):
        assert normwise(got.cpu().numpy(), want) <= TOL[dt]


# ---- the five benchmark configurations at a row count the oracle finishes quickly ----
BENCH = [
    ("c1", ko.MKM, 16, [8] * 5, [8] * 5, np.float32, 1.0, 0.0, 1),
    ("c2", ko.MKM, 8, [16] * 4, [16] * 4, np.float32, 1.0, 0.0, 1),
    ("c3", ko.MKM, 2, [64] * 3, [64] * 3, np.float64, 1.0, 0.0, 1),
    ("c4", ko.KMM, 64, [4] * 6, [4] * 6, np.float32, 1.5, 0.5, 1),
    ("c5", ko.MKM, 8, [32] * 3, [16] * 3, np.float32, 1.0, 1.0, 8),
]


@pytest.mark.parametrize("name,mm,M,Ps,Qs,dt,alpha,beta,batch", BENCH, ids=[b[0] for b in BENCH])
def test_benchmark_configurations_reduced_rows(fk, name, mm, M, Ps, Qs, dt, alpha, beta, batch):
    check(fk, mm, M, Ps, Qs, dt, alpha=alpha, beta=beta, batch=batch, seed=7)


@pytest.mark.parametrize("tune", [False, True])
def test_tuned_and_online_plans_agree(tune):
    import fastkron_amd
    h = fastkron_amd.FastKron(tune=tune)
    try:
        check(h, ko.MKM, 32, [8] * 4, [8] * 4, np.float32, alpha=1.0, beta=0.0, seed=3)
        check(h, ko.MKM, 16, [16] * 3, [16] * 3, np.float32, alpha=2.0, beta=1.0, seed=4)
        check(h, ko.KMM, 32, [4] * 5, [4] * 5, np.float64, alpha=2.0, beta=1.0, seed=5)
    finally:
        h.close()


def test_whole_row_kernel_for_four_16x16_factors(fk):
    """16x16^4 fp32 rows run as ONE launch of the register-resident row kernel, with and without Y,
    batched, and with transposed factors (handled by the factor strides)."""
    check(fk, ko.MKM, 101, [16] * 4, [16] * 4, np.float32, alpha=1.0, beta=0.0, seed=11)
    plan = fk.last_plan()
    assert len(plan) == 1 and "1x65536" in plan[0][2], plan
    check(fk, ko.MKM, 97, [16] * 4, [16] * 4, np.float32, alpha=-1.5, beta=0.75, seed=12)
    check(fk, ko.MKM, 40, [16] * 4, [16] * 4, np.float32, alpha=2.0, beta=1.0, seed=13, batch=3)
    assert len(fk.last_plan()) == 1 and "1x65536" in fk.last_plan()[0][2], fk.last_plan()
    check(fk, ko.MKM, 96, [16] * 4, [16] * 4, np.float32, alpha=2.0, beta=1.0, seed=14, opFs=ko.OP_T)
    assert len(fk.last_plan()) == 1
    check(fk, ko.MKM, 96, [16] * 4, [16] * 4, np.float32, alpha=1.0, beta=0.0, seed=15, integer=True)
    # fewer than 96 rows: a row is 20 us of one CU's work, so three factors go to the wave-per-block kernel (16 blocks
    # per row, spread over the CUs) and the first one runs across the blocks
    for M, kw in [(5, dict(alpha=1.0, beta=0.0)), (3, dict(alpha=-1.5, beta=0.75)), (2, dict(alpha=2.0, beta=1.0, batch=3)),
                  (2, dict(alpha=2.0, beta=1.0, opFs=ko.OP_T)), (2, dict(alpha=1.0, beta=0.0, integer=True))]:
        check(fk, ko.MKM, M, [16] * 4, [16] * 4, np.float32, seed=17 + M, **kw)
        plan = fk.last_plan()
        if "batch" not in kw:                      # (factors that differ per batch entry run one launch per factor)
            assert len(plan) == 2 and "_3_1x4096_" in plan[0][2], plan
    # five factors: the last four are fused by the row kernel only when the row is exactly 16^4 long
    check(fk, ko.MKM, 2, [2] + [16] * 4, [2] + [16] * 4, np.float32, alpha=1.0, beta=0.5, seed=16)


def test_whole_row_kernel_for_five_8x8_factors(fk):
    """8x8^5 fp32 rows run as ONE launch of the register-resident 4x4x1-MFMA row kernel."""
    check(fk, ko.MKM, 5, [8] * 5, [8] * 5, np.float32, alpha=1.0, beta=0.0, seed=21)
    plan = fk.last_plan()
    assert len(plan) == 1 and "1x32768" in plan[0][2], plan
    check(fk, ko.MKM, 3, [8] * 5, [8] * 5, np.float32, alpha=-1.5, beta=0.75, seed=22)
    check(fk, ko.MKM, 2, [8] * 5, [8] * 5, np.float32, alpha=2.0, beta=1.0, seed=23, batch=3)
    check(fk, ko.MKM, 2, [8] * 5, [8] * 5, np.float32, alpha=2.0, beta=1.0, seed=24, opFs=ko.OP_T)
    check(fk, ko.MKM, 2, [8] * 5, [8] * 5, np.float32, alpha=1.0, beta=0.0, seed=25, integer=True)
    check(fk, ko.MKM, 2, [3] + [8] * 5, [2] + [8] * 5, np.float32, alpha=1.0, beta=0.5, seed=26)


ROW_8X5_F64 = "mkm_hip_gfx950_512_d_8x8_8x8_5_1x32768_valu_NN_strided_0_3"


def test_whole_row_kernel_for_five_8x8_fp64_factors(fk):
    """8x8^5 fp64 rows run as ONE launch of the register-resident row kernel (vector-ALU FMAs with the factor in scalar
    registers) from 32 rows on; below that the chain is merged into 64x64 products as before."""
    check(fk, ko.MKM, 130, [8] * 5, [8] * 5, np.float64, alpha=1.0, beta=0.0, seed=41)
    assert [k for _, _, k in fk.last_plan()] == [ROW_8X5_F64], fk.last_plan()
    check(fk, ko.MKM, 128, [8] * 5, [8] * 5, np.float64, alpha=-1.5, beta=0.75, seed=42)
    assert [k for _, _, k in fk.last_plan()] == [ROW_8X5_F64], fk.last_plan()
    check(fk, ko.MKM, 128, [8] * 5, [8] * 5, np.float64, alpha=2.0, beta=1.0, seed=43, opFs=ko.OP_T)      # factors stored the other way round
    assert [k for _, _, k in fk.last_plan()] == [ROW_8X5_F64], fk.last_plan()
    check(fk, ko.MKM, 11, [8] * 5, [8] * 5, np.float64, alpha=2.0, beta=1.0, seed=44, batch=3)            # factors per batch entry
    assert [k for _, _, k in fk.last_plan()] == [ROW_8X5_F64], fk.last_plan()
    check(fk, ko.MKM, 33, [8] * 5, [8] * 5, np.float64, alpha=1.0, beta=0.5, seed=45, batch=2, share_f=True, share_y=True)
    assert [k for _, _, k in fk.last_plan()] == [ROW_8X5_F64], fk.last_plan()
    check(fk, ko.MKM, 128, [8] * 5, [8] * 5, np.float64, alpha=1.0, beta=0.0, seed=46, integer=True)
    check(fk, ko.MKM, 128, [8] * 5, [8] * 5, np.float64, alpha=1.0, beta=0.0, seed=47, use_temp2=False)
    check(fk, ko.MKM, 129, [8] * 5, [8] * 5, np.float64, alpha=0.5, beta=-1.0, seed=48, opX=ko.OP_T)      # X copied transposed first
    assert fk.last_plan()[-1][2] == ROW_8X5_F64, fk.last_plan()
    check(fk, ko.MKM, 31, [8] * 5, [8] * 5, np.float64, alpha=1.0, beta=1.0, seed=49)
    assert ROW_8X5_F64 not in [k for _, _, k in fk.last_plan()], fk.last_plan()
    # six and seven factors: the row kernel on the blocks of 32768 columns, the leading factor(s) across them
    check(fk, ko.MKM, 5, [8] * 6, [8] * 6, np.float64, alpha=1.5, beta=0.5, seed=50)
    plan = fk.last_plan()
    assert len(plan) == 2 and plan[0] == (1, 5, ROW_8X5_F64), plan
    check(fk, ko.MKM, 4, [8] * 6, [8] * 6, np.float64, alpha=1.0, beta=1.0, seed=51, opFs=ko.OP_T, y_is_z=True)
    check(fk, ko.MKM, 2, [8] * 6, [8] * 6, np.float64, alpha=1.0, beta=0.0, seed=52, batch=2, share_f=True)
    check(fk, ko.MKM, 1, [8] * 7, [8] * 7, np.float64, alpha=-1.0, beta=0.5, seed=53)
    plan = fk.last_plan()
    assert len(plan) == 2 and plan[0][2] == ROW_8X5_F64 and "64x64" in plan[1][2], plan


ROW_32X3_PERSISTENT = "mkm_hip_gfx950_1024_f_32x32_32x32_3_1x32768_mfma16x16x4_NN_strided_0_3"


def test_persistent_whole_row_kernel_for_three_32x32_factors(fk):
    """32x32^3 fp32 from three rows per CU on: one persistent workgroup of 16 waves per CU that goes from row to row with
    the next row's loads in flight (three block slots per lane, rotating with a period of three rows).  Row counts that
    give the workgroups 3 or 4 rows each, batches whose factors are restaged between rows, Z == Y."""
    check(fk, ko.MKM, 770, [32] * 3, [32] * 3, np.float32, alpha=1.5, beta=0.5, seed=81)
    assert [k for _, _, k in fk.last_plan()] == [ROW_32X3_PERSISTENT], fk.last_plan()
    check(fk, ko.MKM, 1030, [32] * 3, [32] * 3, np.float32, alpha=1.0, beta=0.0, seed=82, opFs=ko.OP_T)
    assert [k for _, _, k in fk.last_plan()] == [ROW_32X3_PERSISTENT], fk.last_plan()
    check(fk, ko.MKM, 97, [32] * 3, [32] * 3, np.float32, alpha=2.0, beta=1.0, seed=83, batch=8)          # factors per batch entry
    assert [k for _, _, k in fk.last_plan()] == [ROW_32X3_PERSISTENT], fk.last_plan()
    check(fk, ko.MKM, 390, [32] * 3, [32] * 3, np.float32, alpha=1.0, beta=-1.0, seed=84, batch=2, share_f=True, share_y=True)
    check(fk, ko.MKM, 768, [32] * 3, [32] * 3, np.float32, alpha=-0.5, beta=2.0, seed=85, y_is_z=True)
    check(fk, ko.MKM, 767, [32] * 3, [32] * 3, np.float32, alpha=1.0, beta=0.0, seed=86)                  # below: two workgroups per CU
    assert ROW_32X3_PERSISTENT not in [k for _, _, k in fk.last_plan()], fk.last_plan()
    # four factors: the kernel on the 32 blocks of every row, the leading factor across them
    check(fk, ko.MKM, 25, [32] * 4, [32] * 4, np.float32, alpha=1.0, beta=0.5, seed=87)
    assert fk.last_plan()[0][2] == ROW_32X3_PERSISTENT, fk.last_plan()


RECT_PAIRS = [
    # P, Q, dtype: the shapes the pair kernel has exact rectangular tiles for
    (32, 64, np.float32), (64, 32, np.float32), (32, 64, np.float64),
]


@pytest.mark.parametrize("P,Q,dt", RECT_PAIRS)
def test_pair_kernel_for_two_rectangular_factors(fk, P, Q, dt):
    """Two factors of 32x64 / 64x32 (reference tests/src/general-tests-NN.cpp:94-100 runs 32x64 chains): one launch of
    the pair kernel on exact tiles (a P x P row in, a Q x Q row out), and for three factors the two-part plan with the
    pair on the blocks of a row and the leading factor across them."""
    t = "d" if dt == np.float64 else "f"
    name = f"mkm_hip_gfx950_256_{t}_{P}x{Q}_{P}x{Q}_2_1x{P * P}_mfma16x16x4_NN_strided_0_3"
    check(fk, ko.MKM, 37, [P] * 2, [Q] * 2, dt, alpha=1.0, beta=0.0, seed=61)
    assert [k for _, _, k in fk.last_plan()] == [name], fk.last_plan()
    check(fk, ko.MKM, 5, [P] * 2, [Q] * 2, dt, alpha=-1.5, beta=0.75, seed=62)
    check(fk, ko.MKM, 9, [P] * 2, [Q] * 2, dt, alpha=2.0, beta=1.0, seed=63, opFs=ko.OP_T)
    check(fk, ko.MKM, 6, [P] * 2, [Q] * 2, dt, alpha=1.0, beta=1.0, seed=64, batch=3)
    check(fk, ko.MKM, 6, [P] * 2, [Q] * 2, dt, alpha=1.0, beta=0.5, seed=65, batch=2, share_f=True, share_y=True)
    check(fk, ko.MKM, 4, [P] * 2, [Q] * 2, dt, alpha=1.0, beta=0.0, seed=66, integer=True)
    if P <= Q:
        check(fk, ko.MKM, 7, [P] * 2, [Q] * 2, dt, alpha=1.5, beta=0.5, seed=67, y_is_z=True)
    # three factors: the pair runs on the M * P blocks of P*P columns, the leading factor across the blocks
    check(fk, ko.MKM, 3, [P] * 3, [Q] * 3, dt, alpha=1.5, beta=0.5, seed=68)
    plan = fk.last_plan()
    assert len(plan) == 2 and plan[0][2] == name and plan[0][:2] == (1, 2), plan
    check(fk, ko.MKM, 3, [P] * 3, [Q] * 3, dt, alpha=1.0, beta=1.0, seed=69, batch=2, share_f=True)    # reference: batched, X shared
    assert len(fk.last_plan()) == 2, fk.last_plan()
    check(fk, ko.MKM, 3, [P] * 3, [Q] * 3, dt, alpha=1.0, beta=1.0, seed=70, batch=2)                  # factors per batch entry: no two-part plan
    check(fk, ko.MKM, 2, [16, P, P], [8, Q, Q], dt, alpha=1.0, beta=0.0, seed=71)                      # another leading factor
    assert fk.last_plan()[0][2] == name, fk.last_plan()
    if P <= Q:        # (with shrinking factors Z is smaller than the temporary, and the second temporary is mandatory)
        check(fk, ko.MKM, 2, [P] * 3, [Q] * 3, dt, alpha=1.0, beta=0.0, seed=72, use_temp2=False)      # one temporary: no two-part plan


@pytest.mark.parametrize("P,Q,dt", [(64, 64, np.float32), (32, 32, np.float32), (32, 32, np.float64),
                                    (24, 24, np.float32), (24, 24, np.float64)] + RECT_PAIRS)
def test_pair_kernel_rows_shared_between_waves(fk, P, Q, dt):
    """With few rows the pair kernel hands each row to 2 or 4 waves, one share of the output column blocks each; with
    more rows than one workgroup per CU holds waves, a wave produces whole rows.  Row counts on both sides of every
    switch (256 CUs x 4 waves: 4 shares up to 256 rows, 2 up to 512), odd ones included."""
    for i, M in enumerate((1, 3, 255, 256, 257, 511, 512, 513, 1025)):
        if P == 64 and Q == 64 and M < 512:
            continue                                   # (single steps by the rules of thumb)
        check(fk, ko.MKM, M, [P] * 2, [Q] * 2, dt, alpha=1.0 + i, beta=0.5 * (i % 3), seed=300 + i)
        plan = fk.last_plan()
        assert len(plan) == 1 and "_2_1x" in plan[0][2], plan
    check(fk, ko.MKM, 100, [P] * 2, [Q] * 2, dt, alpha=1.0, beta=1.0, seed=320, batch=3)
    check(fk, ko.MKM, 200, [P] * 2, [Q] * 2, dt, alpha=1.0, beta=0.0, seed=321, batch=2, share_f=True)


def test_pair64_fp64_blocks_shared_between_waves(fk):
    """dgemkm 64x64^2 with few blocks: four waves per block up to 2 blocks per CU, two up to 4 (each wave loads the block
    whole and produces its own output columns); a block per wave from 8 per CU on."""
    pair = "mkm_hip_gfx950_512_d_64x64_64x64_2_1x4096_mfma4x4x4_NN_strided_0_3"
    for i, M in enumerate((320, 511, 512, 513, 1023, 1024, 2049)):
        check(fk, ko.MKM, M, [64] * 2, [64] * 2, np.float64, alpha=1.0 + i, beta=0.5 * (i % 3), seed=340 + i)
        assert [k for _, _, k in fk.last_plan()] == [pair], (M, fk.last_plan())
    check(fk, ko.MKM, 200, [64] * 2, [64] * 2, np.float64, alpha=1.0, beta=1.0, seed=350, batch=3)     # 600 blocks
    assert [k for _, _, k in fk.last_plan()] == [pair], fk.last_plan()
    check(fk, ko.MKM, 170, [64] * 2, [64] * 2, np.float64, alpha=-1.0, beta=0.5, seed=351, batch=2, share_f=True, opFs=ko.OP_T)
    assert [k for _, _, k in fk.last_plan()] == [pair], fk.last_plan()
    check(fk, ko.MKM, 400, [64] * 2, [64] * 2, np.float64, alpha=1.5, beta=0.5, seed=352, y_is_z=True)
    check(fk, ko.MKM, 6, [64] * 3, [64] * 3, np.float64, alpha=1.0, beta=0.0, seed=353)                # 384 blocks of a chain
    assert fk.last_plan()[0][2] == pair, fk.last_plan()


def test_whole_row_kernel_for_three_32x16_factors(fk):
    """32x16^3 fp32 rows (non-square, which the reference never fuses) run as ONE launch."""
    check(fk, ko.MKM, 5, [32] * 3, [16] * 3, np.float32, alpha=1.0, beta=0.0, seed=31)
    plan = fk.last_plan()
    assert len(plan) == 1 and "32x16" in plan[0][2] and "1x32768" in plan[0][2], plan
    check(fk, ko.MKM, 3, [32] * 3, [16] * 3, np.float32, alpha=-1.5, beta=0.75, seed=32)
    check(fk, ko.MKM, 4, [32] * 3, [16] * 3, np.float32, alpha=1.0, beta=1.0, seed=33, batch=5)
    check(fk, ko.MKM, 4, [32] * 3, [16] * 3, np.float32, alpha=1.0, beta=1.0, seed=34, batch=3, share_f=True)
    check(fk, ko.MKM, 2, [32] * 3, [16] * 3, np.float32, alpha=2.0, beta=1.0, seed=35, opFs=ko.OP_T)
    check(fk, ko.MKM, 2, [32] * 3, [16] * 3, np.float32, alpha=1.0, beta=0.0, seed=36, integer=True)
    check(fk, ko.MKM, 2, [2] + [32] * 3, [3] + [16] * 3, np.float32, alpha=1.0, beta=0.5, seed=37)


@pytest.mark.parametrize("M,Ps", [(3, [64]), (2, [16, 16]), (5, [32, 32]), (2, [64, 64, 64]), (7, [16] * 4), (4, [64, 16, 32]),
                                  (5, [128]), (3, [128, 128]), (40, [128, 64])])
@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_mfma_step_kernel(fk, M, Ps, dt):
    """Steps with 16/32/64-wide square factors run on the matrix cores (fp64 and fp32), including tiles
    with fewer than 16 slices and mixed chains."""
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=41)
    # (a few rows of 16x16^4: the first factor runs across the blocks on the plain kernel)
    if Ps != [16] * 4:
        assert all("_mfma" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=42, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=43, batch=2)


@pytest.mark.parametrize("M,Ps", [(64, [4] * 6), (100, [4] * 3), (16, [4] * 6), (130, [8] * 2), (64, [8] * 4),
                                  (70, [4] * 5), (33, [8] * 3)])
def test_kmm_register_kernel(fk, M, Ps):
    """KMM with 4x4 / 8x8 fp32 factors: three (two) factors per launch held in registers, lanes along M,
    including column counts that are not a multiple of 64 and chains with a generic remainder."""
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=51)
    assert any("mfma4x4x1" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=52, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=53, batch=2)
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=2.0, beta=1.0, seed=54, use_temp2=False)


def test_misaligned_buffers_get_a_plan_without_the_refusing_kernel(fk):
    """The 16x16^4 row kernel stores 128-bit vectors; a Z that is only 4-byte aligned must still give the
    right answer (the library selects again without the kernels that refuse the buffers)."""
    import torch
    M, Ps = 96, [16] * 4
    K = 65536
    X, Fs, _ = make_case(ko.MKM, M, Ps, Ps, np.float32, seed=61, with_y=False)
    want = oracle_answer(ko.MKM, M, Ps, Ps, X, Fs, None, 1.0, 0.0)
    dev = "cuda:0"
    tX = torch.from_numpy(X).to(dev)
    tFs = [torch.from_numpy(f).to(dev) for f in Fs]
    Zbuf = torch.full((M * K + 1,), float("nan"), dtype=torch.float32, device=dev)
    Z = Zbuf[1:]                                       # data_ptr() is 4 bytes past a 256-byte boundary
    t1 = torch.empty(M * K, dtype=torch.float32, device=dev)
    t2 = torch.empty(M * K, dtype=torch.float32, device=dev)
    e = fk.xgemkm(M, Ps, Ps, tX, tFs, Z, 1.0, 0.0, None, t1, t2)
    torch.cuda.synchronize()
    assert e == 0
    assert not any("_16x16_16x16_4_" in k for _, _, k in fk.last_plan()), fk.last_plan()
    assert normwise(Z.cpu().numpy(), want) <= 1e-5


@pytest.mark.parametrize("which", ["x", "y", "z"])
@pytest.mark.parametrize("M,Ps,dt", [(96, [16] * 4, np.float32), (16, [16] * 3, np.float32), (100, [32] * 3, np.float32),
                                     (8, [64, 64], np.float64), (8, [32, 32], np.float32), (64, [64], np.float64),
                                     (4, [128, 128], np.float32), (6, [64, 64], np.float32)])
def test_one_misaligned_operand_at_a_time(fk, which, M, Ps, dt):
    """X, Y or Z alone starts one element past a 256-byte boundary: kernels with 16-byte accesses to that operand
    must not be chosen, and the answer must still be right."""
    import torch
    K = int(np.prod(Ps))
    X, Fs, Y = make_case(ko.MKM, M, Ps, Ps, dt, seed=62, with_y=True)
    want = oracle_answer(ko.MKM, M, Ps, Ps, X, Fs, Y, 1.5, 0.5)
    dev = "cuda:0"
    tdt = torch.float32 if dt == np.float32 else torch.float64

    def place(host, shifted):
        buf = torch.full((host.size + 64,), float("nan"), dtype=tdt, device=dev)
        v = buf[1:1 + host.size] if shifted else buf[:host.size]
        v.copy_(torch.from_numpy(host.reshape(-1)))
        return v

    tX, tY = place(X, which == "x"), place(Y, which == "y")
    Z = place(np.full(M * K, np.nan, dt), which == "z")
    tFs = [torch.from_numpy(f).to(dev) for f in Fs]
    t1 = torch.empty(M * K, dtype=tdt, device=dev)
    t2 = torch.empty(M * K, dtype=tdt, device=dev)
    e = fk.xgemkm(M, Ps, Ps, tX, tFs, Z, 1.5, 0.5, tY, t1, t2)
    torch.cuda.synchronize()
    assert e == 0
    assert normwise(Z.cpu().numpy(), want) <= TOL[dt], (which, fk.last_plan())


@pytest.mark.parametrize("which", ["none", "y", "z"])
def test_32x16_row_kernel_with_results_off_16_byte_boundaries(fk, which):
    """The 32x16^3 row kernel writes Z and reads Y 16 bytes per lane when their rows start on 16-byte boundaries, element
    by element otherwise: either way one launch and the right answer."""
    import torch
    M, Ps, Qs = 6, [32] * 3, [16] * 3
    K, L = 32768, 4096
    X, Fs, Y = make_case(ko.MKM, M, Ps, Qs, np.float32, seed=63, with_y=True)
    want = oracle_answer(ko.MKM, M, Ps, Qs, X, Fs, Y, 1.5, 0.5)
    dev = "cuda:0"

    def place(host, shifted):
        buf = torch.full((host.size + 64,), float("nan"), dtype=torch.float32, device=dev)
        v = buf[1:1 + host.size] if shifted else buf[:host.size]
        v.copy_(torch.from_numpy(host.reshape(-1)))
        return v

    tX, tY = place(X, False), place(Y, which == "y")
    Z = place(np.full(M * L, np.nan, np.float32), which == "z")
    tFs = [torch.from_numpy(f).to(dev) for f in Fs]
    t1 = torch.empty(M * K, dtype=torch.float32, device=dev)
    t2 = torch.empty(M * K, dtype=torch.float32, device=dev)
    e = fk.xgemkm(M, Ps, Qs, tX, tFs, Z, 1.5, 0.5, tY, t1, t2)
    torch.cuda.synchronize()
    assert e == 0
    plan = fk.last_plan()
    assert len(plan) == 1 and "32x16" in plan[0][2], plan
    assert normwise(Z.cpu().numpy(), want) <= TOL[np.float32], (which, plan)


@pytest.mark.parametrize("M,Ps,dt", [(8, [16] * 5, np.float32), (4, [8] * 6, np.float32), (2, [32] * 4, np.float32),
                                     (8, [16] * 4, np.float64), (2, [64] * 3, np.float64), (16, [4] * 8, np.float32),
                                     (4, [8] * 5, np.float64), (3, [4, 4] + [8] * 5, np.float32)])
def test_strided_entry_point_with_a_single_batch_entry(fk, M, Ps, dt):
    """batchCount = 1 with the natural strides (strideF = P*Q): the two-part plan turns rows into batch entries of
    its second part, which must not inherit the caller's factor strides."""
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=105, batch=1, strided=True)
    strided_plan = fk.last_plan()
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=105)
    assert [k for _, _, k in fk.last_plan()] == [k for _, _, k in strided_plan]
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=106, batch=1, strided=True)


@pytest.mark.parametrize("mm,name", [(ko.MKM, "mkm"), (ko.KMM, "kmm")])
def test_forward_strided_batched(fk, mm, name):
    import ctypes
    import torch
    from fastkron_amd import capi
    M, Ps, Qs, B = 5, [4, 3, 8], [2, 5, 8], 3
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X, Fs, _ = make_case(mm, M, Ps, Qs, np.float64, seed=71, with_y=False, batch=B)
    Zw, Iw = oracle_answer(mm, M, Ps, Qs, X, Fs, None, 1.0, 0.0, batch=B, keep_intermediates=True)
    ye, sizes = fk.sizes_forward(M, Ps, Qs)
    dev = "cuda:0"
    tX = torch.from_numpy(X).to(dev)
    tFs = [torch.from_numpy(f).to(dev) for f in Fs]
    Z = torch.full((B * ye,), float("nan"), dtype=torch.float64, device=dev)
    inters = [torch.full((B * s,), float("nan"), dtype=torch.float64, device=dev) for s in sizes]
    lib = fk.lib
    fp = capi.arr_ptr([f.data_ptr() for f in tFs])
    ip = capi.arr_ptr([t.data_ptr() for t in inters])
    sF = capi.arr_u64([p * q for p, q in zip(Ps, Qs)])
    if mm == ko.MKM:
        e = lib.dmkmForwardStridedBatched(fk.h, capi.BACKEND_HIP, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs),
                                          ctypes.c_void_p(tX.data_ptr()), capi.OP_N, M * K, fp, capi.OP_N, sF,
                                          ctypes.c_void_p(Z.data_ptr()), M * L, B, ip, None)
    else:
        e = lib.dkmmForwardStridedBatched(fk.h, capi.BACKEND_HIP, len(Ps), capi.arr_u32(Qs), capi.arr_u32(Ps), M,
                                          fp, capi.OP_N, sF, ctypes.c_void_p(tX.data_ptr()), capi.OP_N, M * K,
                                          ctypes.c_void_p(Z.data_ptr()), M * L, B, ip, None)
    torch.cuda.synchronize()
    assert e == 0
    assert normwise(Z.cpu().numpy(), Zw) <= 1e-12
    for got, want in zip(inters, Iw):
        assert normwise(got.cpu().numpy(), want) <= 1e-12


def test_tuned_plans_persist_to_a_file(tmp_path):
    """fastKronOptionsTune times the candidate plans once, writes the winner to the tuning file, and a
    new handle pointed at that file uses it without tuning."""
    import fastkron_amd
    db = str(tmp_path / "tuned.db")
    h = fastkron_amd.FastKron(tune=True)
    h.set_tuned_db(db)
    try:
        check(h, ko.MKM, 16, [8] * 3, [8] * 3, np.float32, alpha=1.0, beta=0.0, seed=81)
        plan = h.last_plan()
    finally:
        h.close()
    text = open(db).read()
    assert "16x512*(8x8^3)_NN_f" in text
    h2 = fastkron_amd.FastKron(tune=False)
    h2.set_tuned_db(db)
    try:
        check(h2, ko.MKM, 16, [8] * 3, [8] * 3, np.float32, alpha=1.0, beta=0.0, seed=82)
        assert h2.last_plan() == plan
    finally:
        h2.close()


@pytest.mark.parametrize("M,Ps,tag,tag_b", [(8, [8] * 4, "1x32768", "1x32768"), (128, [8] * 3, "1x32768", "1x32768"),
                                            (1024, [8] * 2, "1x32768", "1x32768"), (16, [16] * 3, "1x4096", "1x65536"),
                                            (512, [16] * 2, "1x4096", "1x65536"), (32, [16] * 3, "1x4096", "1x65536")])
def test_row_kernels_with_fewer_factors(fk, M, Ps, tag, tag_b):
    """Shorter chains of 8x8 / 16x16 factors reuse the whole-row kernels: 8^(5-N) (16^(4-N)) consecutive rows
    form one contiguous block and the missing leading factors are identities.  Two or three 16x16 factors shared
    by the batch go to the wave-per-block kernel instead; with per-batch factors the workgroup kernel runs them."""
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=91)
    plan = fk.last_plan()
    assert len(plan) == 1 and tag in plan[0][2], plan
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=92, batch=2)
    plan = fk.last_plan()
    assert len(plan) == 1 and tag_b in plan[0][2], plan


def test_row_kernels_need_whole_blocks(fk):
    """A row count that is not a whole number of blocks takes the kernels without that requirement instead."""
    check(fk, ko.MKM, 12, [8] * 4, [8] * 4, np.float32, alpha=1.0, beta=0.0, seed=93)
    assert all("generic" in k or "small_fused" in k for _, _, k in fk.last_plan())


@pytest.mark.parametrize("M,Ps", [(4, [8] * 6), (2, [8] * 7), (3, [4, 4] + [8] * 5), (2, [16] * 5), (1, [16] * 6),
                                  (2, [4, 4, 4] + [16] * 4), (2, [8, 8] + [16] * 4)])
def test_long_chains_split_into_row_kernel_plus_leading_kmm(fk, M, Ps):
    """Chains longer than a whole-row kernel takes: trailing factors by the row kernel on M*K_A virtual rows,
    leading factors as a batched KMM over the row blocks (2-3 launches instead of N)."""
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=101)
    plan = fk.last_plan()
    assert len(plan) <= 3 and any("kmm_" in k for _, _, k in plan) and any("mkm_" in k for _, _, k in plan), plan
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=102, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=103, batch=2, share_f=True)
    # per-batch factors cannot use the split (the KMM part flattens batch and rows): still correct
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=104, batch=2)


@pytest.mark.parametrize("M,Ps", [(64, [8]), (70, [8] * 3), (64, [16]), (100, [16, 16]), (64, [4]), (80, [4, 4]), (64, [4] * 4)])
def test_kmm_register_kernel_more_tiles(fk, M, Ps):
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=111)
    # groups of 4x4 / 8x8 factors run on the register kernel; single factors are left to the plain kernel
    plan = fk.last_plan()
    assert all("mfma4x4x1" in k or hi == lo or "_16x16_16x16_2_" in k for lo, hi, k in plan), plan
    if len(Ps) >= 2 and Ps[0] < 16:
        assert any("mfma4x4x1" in k for _, _, k in plan), plan
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=112, batch=3)


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("M,P", [(1, 64), (7, 64), (64, 64), (600, 64), (3, 32), (50, 32), (2100, 32)])
def test_pair_kernel(fk, M, P, dt):
    """Two fused 64x64 / 32x32 factors (fp64, fp32): chained matrix-core products, one wave per row."""
    check(fk, ko.MKM, M, [P, P], [P, P], dt, alpha=1.5, beta=0.5, seed=121)
    plan = fk.last_plan()
    # few 64x64 blocks: two single-factor launches fill the device better than a wave per block (fp64: except where
    # two or four waves share a block, 320 to 1024 blocks)
    if P == 64 and (M < 512 if dt == np.float32 else (M < 320 or 1024 < M < 2048)):
        assert len(plan) == 2 and all("_64x64_64x64_1_" in k for _, _, k in plan), plan
    else:
        assert len(plan) == 1 and f"_2_1x{P * P}_" in plan[0][2], plan
    check(fk, ko.MKM, M, [P, P], [P, P], dt, alpha=1.0, beta=0.0, seed=122, opFs=ko.OP_T)
    check(fk, ko.MKM, M, [P, P], [P, P], dt, alpha=1.0, beta=1.0, seed=123, batch=3)
    check(fk, ko.MKM, M, [P, P], [P, P], dt, alpha=2.0, beta=0.0, seed=124, batch=2, share_f=True)
    check(fk, ko.MKM, M, [P, P], [P, P], dt, alpha=1.0, beta=0.0, seed=125, integer=True)


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("M,Ps", [(32, [64] * 3), (1, [32] * 3), (3, [32] * 4), (128, [16, 64, 64]), (2, [128, 32, 32])])
def test_chains_split_into_pair_kernel_plus_leading_kmm_step(fk, M, Ps, dt):
    """Chains of 32- or 64-wide factors: trailing pair fused per block, leading factors as KMM-layout
    matrix-core steps across the blocks."""
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=131)
    plan = fk.last_plan()
    # (fp32 chains that end in three 32x32 factors fuse those three instead of two, from 96 blocks of 32^3 on)
    fused = 3 if dt == np.float32 and Ps[-3:] == [32] * 3 and M * int(np.prod(Ps[:-3])) >= 96 else 2
    assert len(plan) == len(Ps) - fused + 1 and plan[0][2].startswith("mkm_") and all("kmm_" in k for _, _, k in plan[1:]), plan
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=132, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=133, batch=2, share_f=True)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=134, batch=2)


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("M,Ps", [(16, [64]), (100, [32]), (37, [64, 64]), (5, [128]), (48, [16, 32]), (1000, [32, 32]),
                                  (20, [128, 64])])
def test_kmm_layout_mfma_step_kernel(fk, M, Ps, dt):
    """GeKMM with 16..128-wide square factors on the matrix cores, tiles of 16 consecutive columns of X,
    including column counts that are not a multiple of 16."""
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=141)
    # (exceptions found by tuning: single 16x16 factors go to the plain kernel, fp32 64x64 and 128x128 and fp64 128x128 to
    # the padded step)
    assert all(("kmm_" in k and "generic" not in k) or Ps[lo] == 16 or "anyxany" in k for lo, _, k in fk.last_plan()), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=142, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=143, batch=2)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=144, integer=True)


@pytest.mark.parametrize("M,Ps", [(64, [64]), (192, [64]), (128, [64, 64]), (64, [16, 64])])
def test_kmm_layout_fp64_64x64_step_on_4x4x4_matrix_instruction(fk, M, Ps):
    """dgekmm with 64x64 factors, a multiple of 64 columns of X and eight batch entries or more: 64-column tiles, 4x4x4
    instruction (single problems of this size run on the tiles passed through LDS)."""
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=1.5, beta=0.5, seed=151, batch=8)
    assert any("mfma4x4x4" in k for _, _, k in fk.last_plan()), fk.last_plan()
    # (one factor for all entries: the launch walks the tiles of all entries as one sequence)
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=1.5, beta=0.5, seed=157, batch=9, share_f=True)
    assert any("mfma4x4x4" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=1.5, beta=0.5, seed=156)
    assert not any("mfma4x4x4" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=1.0, beta=0.0, seed=152, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=1.0, beta=1.0, seed=153, batch=3)
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=2.0, beta=0.0, seed=154, batch=2, share_f=True)
    check(fk, ko.KMM, M, Ps, Ps, np.float64, alpha=1.0, beta=0.0, seed=155, integer=True)


def test_tuning_tool_writes_plans_for_the_given_shapes(tmp_path, capsys):
    """`python -m fastkron_amd.tune`: tunes each shape through the C API and keeps the plans in the file."""
    from fastkron_amd import tune
    db = str(tmp_path / "plans.txt")
    assert tune.main(["--db", db, "--mmtype", "mkm", "--type", "float", "-m", "16", "32", "--same-factors", "3", "8,8"]) == 0
    assert tune.main(["--db", db, "--mmtype", "kmm", "--type", "double", "-m", "64", "--distinct-factors", "4,4", "8,8"]) == 0
    out = capsys.readouterr().out
    assert out.count("GFLOP/s") == 3
    text = open(db).read()
    assert "16x512*(8x8^3)_NN_f" in text and "32x512*(8x8^3)_NN_f" in text and "(4x4(x)8x8)*32x64_NN_d" in text


def test_two_part_plan_also_applies_with_tuning_enabled():
    import fastkron_amd
    h = fastkron_amd.FastKron(tune=True)
    try:
        check(h, ko.MKM, 2, [64] * 3, [64] * 3, np.float64, alpha=1.0, beta=0.0, seed=161)
        plan = h.last_plan()          # whichever the tuner measured fastest: the two-part plan or one chain of launches
        assert 1 <= len(plan) <= 3, plan
    finally:
        h.close()


def test_eight_wave_build_of_the_16x16_block_kernel(tmp_path):
    """The 8-wave build (128 values per lane, whole next block prefetched) is an alternative for the tuner; a
    tuned-plan file naming it forces it here.  Several blocks per workgroup, Y, per-batch factors, short chains."""
    import fastkron_amd
    name = "mkm_hip_gfx950_512_f_16x16_16x16_4_1x65536_mfma16x16x4_NN_strided_0_3"
    db = tmp_path / "plans.txt"
    db.write_text("".join(f"{prob} 0.1 1 0 {n - 1} {name}\n" for prob, n in
                          [("600x65536*(16x16^4)_NN_f", 4), ("3x65536*(16x16^4)_NN_f", 4),
                           ("2x65536*(16x16^4)_NN_f_stridedBatched_3", 4), ("64x4096*(16x16^3)_NN_f", 3),
                           ("512x256*(16x16^2)_NN_f", 2), ("2x65536*(16x16^4)_NT_f", 4)]))
    h = fastkron_amd.FastKron()
    h.set_tuned_db(str(db))
    try:
        for M, n, kw in [(600, 4, dict(alpha=1.0, beta=0.0)), (3, 4, dict(alpha=1.5, beta=0.5)),
                         (2, 4, dict(alpha=1.0, beta=1.0, batch=3)), (64, 3, dict(alpha=2.0, beta=1.0)),
                         (512, 2, dict(alpha=1.0, beta=0.0)), (2, 4, dict(alpha=1.0, beta=0.0, opFs=ko.OP_T))]:
            check(h, ko.MKM, M, [16] * n, [16] * n, np.float32, seed=171 + M, **kw)
            assert h.last_plan() == [(0, n - 1, name)], h.last_plan()
    finally:
        h.close()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_two_part_plan_with_three_leading_launches(fk, dt):
    """32x32^5: fused trailing pair (fp64; three factors in fp32), then three (two) KMM-layout steps that ping-pong
    between the second temporary and Z (not possible when Y is Z: then the chain runs as single steps)."""
    check(fk, ko.MKM, 1, [32] * 5, [32] * 5, dt, alpha=1.5, beta=0.5, seed=181)
    plan = fk.last_plan()
    launches = 3 if dt == np.float32 else 4
    assert len(plan) == launches and plan[0][2].startswith("mkm_") and all(k.startswith("kmm_") for _, _, k in plan[1:]), plan


WHOLE_COLUMN_4X6 = "kmm_hip_gfx950_512_f_4x4_4x4_6_8x4096_mfma4x4x1_NN_strided_0_3"


@pytest.mark.parametrize("M", [1024, 1096, 1536])
def test_kmm_six_4x4_factors_in_one_launch(fk, M):
    """sgekmm with 4x4^6 between 1024 and 2048 columns (and no multiple of 256 x 8): one launch, every workgroup owns 8
    columns and all 4096 rows of them."""
    Ps = [4] * 6
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=191)
    assert [k for _, _, k in fk.last_plan()] == [WHOLE_COLUMN_4X6], fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=192, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=195, integer=True, use_temp2=False)
    assert [k for _, _, k in fk.last_plan()] == [WHOLE_COLUMN_4X6], fk.last_plan()
    # column counts that are not a multiple of 8, fewer than 128 column tiles or more than there are CUs: two launches
    check(fk, ko.KMM, M + 12, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=196)
    assert len(fk.last_plan()) == 2, fk.last_plan()
    check(fk, ko.KMM, M // 4, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=198)
    assert len(fk.last_plan()) == 2, fk.last_plan()
    check(fk, ko.KMM, M // 2, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=197, batch=5)
    assert len(fk.last_plan()) == 2, fk.last_plan()


def test_whole_column_4x4_kernel_on_few_columns_and_batches(tmp_path):
    """The whole-column kernel where the online rules prefer two launches (fewer than 128 column tiles), as a tuned plan
    may name it: 8, 72 and 512 columns, batches with per-batch and shared factors."""
    import fastkron_amd
    db = tmp_path / "plans.txt"
    keys = ["(4x4^6)*4096x8_NN_f", "(4x4^6)*4096x72_NN_f", "(4x4^6)*4096x512_NN_f", "(4x4^6)*4096x72_NN_f_stridedBatched_3",
            "(4x4^6)*4096x8_NN_f_stridedBatched_2_Fs3f", "(4x4^6)*4096x72_NT_f"]
    db.write_text("".join(f"{k} 0.1 M0 S0 1 0 5 {WHOLE_COLUMN_4X6}\n" for k in keys))
    h = fastkron_amd.FastKron()
    h.set_tuned_db(str(db))
    try:
        Ps = [4] * 6
        for M, kw in [(8, dict(alpha=1.5, beta=0.5)), (72, dict(alpha=1.0, beta=0.0)), (512, dict(alpha=2.0, beta=1.0)),
                      (72, dict(alpha=1.0, beta=1.0, batch=3)), (8, dict(alpha=2.0, beta=0.0, batch=2, share_f=True)),
                      (72, dict(alpha=1.0, beta=0.0, opFs=ko.OP_T))]:
            check(h, ko.KMM, M, Ps, Ps, np.float32, seed=199 + M, **kw)
            assert [k for _, _, k in h.last_plan()] == [WHOLE_COLUMN_4X6], h.last_plan()
    finally:
        h.close()


TWO_PHASE_4X6 = "kmm_hip_gfx950_256_f_4x4_4x4_6_256x4096_mfma4x4x1_NN_strided_0_3"


def test_kmm_six_4x4_factors_in_two_phases_of_one_launch(fk):
    """sgekmm with 4x4^6 from 2048 columns on: one launch whose workgroups pass an intermediate through a temporary of
    the call and wait for each other per block of 256 columns.  With and without Y, transposed factors, one temporary
    only, a batch (16 column blocks: more workgroups than are resident at once)."""
    Ps = [4] * 6
    check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=291)
    assert [k for _, _, k in fk.last_plan()] == [TWO_PHASE_4X6], fk.last_plan()
    check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=292, opFs=ko.OP_T)
    check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=2.0, beta=0.0, seed=293, integer=True, use_temp2=False)
    assert [k for _, _, k in fk.last_plan()] == [TWO_PHASE_4X6], fk.last_plan()
    check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=294, batch=2)
    assert [k for _, _, k in fk.last_plan()] == [TWO_PHASE_4X6], fk.last_plan()
    check(fk, ko.KMM, 4096, Ps, Ps, np.float32, alpha=-1.0, beta=0.25, seed=295)
    assert [k for _, _, k in fk.last_plan()] == [TWO_PHASE_4X6], fk.last_plan()
    # the same call again and again: every launch leaves the counters as it found them
    for i in range(5):
        check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=296 + i)
    assert fk.sync_error() == 0


def test_two_phase_4x4_kernel_when_workgroups_run_the_jobs_of_others(fk):
    """A workgroup of the two-phase kernel that waits too long for the others runs their missing jobs itself (what keeps
    the launch from deadlocking when not all workgroups are resident).  With the threshold at 0 every workgroup does so
    at once: jobs then run twice, with the same values, and the result must not change."""
    from fastkron_amd import capi
    Ps = [4] * 6
    lib = capi.load()
    try:
        assert lib.fastKronSetSyncHelpAfter(0) == 0
        check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=391)
        assert [k for _, _, k in fk.last_plan()] == [TWO_PHASE_4X6], fk.last_plan()
        check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=392, batch=2)
        check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=393)
    finally:
        lib.fastKronSetSyncHelpAfter(100000)
    check(fk, ko.KMM, 2048, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=394)
    assert fk.sync_error() == 0


def test_two_phase_4x4_kernel_on_column_counts_it_is_not_chosen_for(tmp_path):
    """Any multiple of 256 columns runs on the two-phase kernel when a tuned plan names it: fewer column blocks than
    XCDs (workgroups without a block leave at once), blocks of different batch entries, shared factors."""
    import fastkron_amd
    db = tmp_path / "plans.txt"
    db.write_text("".join(f"{prob} 0.1 M0 S0 1 0 5 {TWO_PHASE_4X6}\n" for prob in
                          ["(4x4^6)*4096x256_NN_f", "(4x4^6)*4096x768_NN_f", "(4x4^6)*4096x512_NN_f_stridedBatched_3",
                           "(4x4^6)*4096x256_NN_f_stridedBatched_5_Fs3f", "(4x4^6)*4096x1280_NT_f"]))
    h = fastkron_amd.FastKron()
    h.set_tuned_db(str(db))
    try:
        Ps = [4] * 6
        for M, kw in [(256, dict(alpha=1.5, beta=0.5)), (768, dict(alpha=1.0, beta=0.0)),
                      (512, dict(alpha=1.0, beta=1.0, batch=3)), (256, dict(alpha=2.0, beta=0.5, batch=5, share_f=True)),
                      (1280, dict(alpha=1.0, beta=-1.0, opFs=ko.OP_T))]:
            check(h, ko.KMM, M, Ps, Ps, np.float32, seed=301 + M, **kw)
            assert [k for _, _, k in h.last_plan()] == [TWO_PHASE_4X6], h.last_plan()
        assert h.sync_error() == 0
    finally:
        h.close()


@pytest.mark.parametrize("mm,M,Ps,dt,launches", [
    (ko.MKM, 96, [4] * 8, np.float32, 1),         # -> 16x16^4: one whole-block launch
    (ko.MKM, 4, [4] * 8, np.float32, 2),          # the same with few rows: three factors per 4096-block + one across
    (ko.MKM, 16, [2] * 12, np.float32, 1),        # -> 16x16^3
    (ko.MKM, 4, [4] * 7, np.float32, 2),          # -> 4, 16x16^3: block kernel on 16 virtual rows + leading 4x4
    (ko.MKM, 3, [4] * 7, np.float32, None),       # same, but 12 virtual rows are no whole block: shorter launches
    (ko.MKM, 5, [2, 4, 2, 4, 8, 2], np.float32, None),
    (ko.MKM, 8, [4] * 6, np.float64, 1),          # -> 16x16^3: chains of 2x2 / 4x4 alone become 16x16 in fp64 too
    (ko.MKM, 24, [8] * 5, np.float64, None),      # -> 8, 64x64^2 (8x8 factors: 64x64 products; from 32 rows on 8x8^5 has a row kernel)
    (ko.MKM, 2048, [8] * 4, np.float64, 1),       # -> 64x64^2: one launch of the pair kernel
    (ko.MKM, 3, [2] * 9, np.float64, None),       # -> 2, 16, 16
    (ko.MKM, 16, [2] * 9, np.float64, 2),         # the same with whole blocks of rows: two 16x16 in one launch + the 2x2
    (ko.MKM, 4, [2, 4, 8, 4, 2], np.float64, None),   # an 8x8 in the chain: 64x64 products
    (ko.KMM, 64, [4] * 6, np.float64, 2),         # -> 16x16^3 on the KMM layout: a pair and a single step
    (ko.KMM, 20, [2] * 7, np.float64, None),
])
def test_small_factors_are_merged_into_their_kronecker_products(fk, mm, M, Ps, dt, launches):
    """Adjacent 2x2 / 4x4 (fp64: 8x8) factors are replaced by their product (16x16 in fp32, 64x64 in fp64),
    computed on the device, so that the kernels for those sizes apply."""
    check(fk, mm, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=201)
    plan = fk.last_plan()
    assert sum(hi - lo + 1 for lo, hi, _ in plan) < len(Ps), plan           # the chain that ran is shorter
    if launches is not None:
        assert len(plan) == launches, plan
    check(fk, mm, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=202, opFs=ko.OP_T)
    check(fk, mm, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=203, batch=2, share_f=True)
    check(fk, mm, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=204, integer=True)
    # per-batch factors are not merged (one product per batch element would be needed): still correct
    check(fk, mm, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=205, batch=2)
    assert sum(hi - lo + 1 for lo, hi, _ in fk.last_plan()) == len(Ps)


FUSED_SMALL = [
    # M, Ps, Qs                               shapes without a matrix-core kernel: several factors per launch through LDS
    (10, [3] * 7, [3] * 7),                   # K = 2187: two launches
    (33, [5, 3, 7, 2], [5, 3, 7, 2]),         # distinct sizes, one launch, ragged row tile
    (5, [3, 5, 2], [4, 2, 6]),                # rectangular factors: the piece grows and shrinks between the steps
    (3, [6] * 5, [6] * 5),                    # even, not a power of two
    (40, [2, 3, 2, 3, 2, 3, 2, 3], [3, 2, 3, 2, 3, 2, 3, 2]),
    (7, [7, 5, 8], [5, 8, 3]),                # P up to 8, any Q
    (4, [3] * 10, [3] * 10),                  # reference tests/src/general-tests-NN.cpp shape family, K = 59049
    (50, [5, 5], [2, 3]),
]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
@pytest.mark.parametrize("M,Ps,Qs", FUSED_SMALL)
def test_small_factors_of_any_shape_are_fused_through_lds(fk, mm, M, Ps, Qs, dt):
    check(fk, mm, M, Ps, Qs, dt, alpha=1.5, beta=0.5, seed=301)
    plan = fk.last_plan()
    # (in the KMM layout only groups of three or more factors of at most 6 rows are fused: the plain kernel is
    # as fast as the fused one beyond that)
    if mm == ko.MKM or (len(Ps) >= 3 and max(Ps) <= 6):
        assert len(plan) < len(Ps) and any("small_fused" in k for _, _, k in plan), plan
    check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=0.0, seed=302, opFs=ko.OP_T)
    check(fk, mm, M, Ps, Qs, dt, alpha=2.0, beta=1.0, seed=303, batch=3)          # per-batch factors
    check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=0.0, seed=304, batch=2, share_f=True)
    if np.prod([max(p, q) for p, q in zip(Ps, Qs)]) < 50000:
        check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=1.0, seed=305, integer=True)


ANY_SHAPE = [
    # M, Ps, Qs: one factor per launch on the matrix cores, zero padded to multiples of 4 (P) and 16 (Q)
    (20, [31, 33], [31, 33]),
    (5, [31, 33], [63, 37]),            # ragged in every dimension: P % 4, Q % 16, slices % 16
    (16, [50, 50], [50, 50]),
    (3, [100], [128]),
    (33, [127], [9]),                   # a single output block, mostly padding
    (4, [30, 64], [64, 30]),
    (2, [128, 36], [36, 128]),
    (3, [129, 200], [200, 129]),        # beyond 128: more lane registers, the factor in slabs of output columns
    (2, [255], [297]),
    (4, [17], [512]),
]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
@pytest.mark.parametrize("M,Ps,Qs", ANY_SHAPE)
def test_any_shape_step_on_the_matrix_cores(fk, mm, M, Ps, Qs, dt):
    check(fk, mm, M, Ps, Qs, dt, alpha=1.5, beta=0.5, seed=401)
    # (online rule: fp64 factors of more than 128 rows that leave the padded groups of four part empty run on the plain
    # kernel in the KMM layout; 255 rows stay here)
    ruled_out = mm == ko.KMM and dt == np.float64 and all(p > 128 and ((p + 3) // 4) % 4 for p in Ps)
    assert ruled_out or any("anyxany" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=0.0, seed=402, opFs=ko.OP_T)
    check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=0.0, seed=403, opX=ko.OP_T)       # X stored transposed
    assert ruled_out or any("anyxany" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, mm, M, Ps, Qs, dt, alpha=2.0, beta=1.0, seed=404, batch=3)
    check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=1.0, seed=405, integer=True)
    check(fk, mm, M, Ps, Qs, dt, alpha=1.0, beta=0.0, seed=406, use_temp2=False)


@pytest.mark.parametrize("M,Ps,launches", [
    (5, [16] * 3, 1),               # a block per row
    (32, [16, 16], 1),              # two factors: 16 rows per block, identity in the leading slot
    (3, [16] * 4, 2),               # three trailing factors in place on 48 virtual rows + one leading launch
    (1, [16] * 5, 2),               # the two leading factors as one KMM-layout pair launch
    (2, [4, 8, 16, 16, 16], None),  # merged leading factors
])
def test_fp64_16x16_block_kernel(fk, M, Ps, launches):
    """fp64 chains of 16x16 factors: three factors per launch on blocks of 4096 doubles held in one wave's registers."""
    check(fk, ko.MKM, M, Ps, Ps, np.float64, alpha=1.5, beta=0.5, seed=501)
    plan = fk.last_plan()
    assert any("_d_16x16_16x16_3_" in k for _, _, k in plan), plan
    if launches is not None:
        assert len(plan) == launches, plan
    check(fk, ko.MKM, M, Ps, Ps, np.float64, alpha=1.0, beta=0.0, seed=502, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, np.float64, alpha=1.0, beta=1.0, seed=503, batch=3, share_f=True)
    check(fk, ko.MKM, M, Ps, Ps, np.float64, alpha=2.0, beta=0.0, seed=504, batch=2)          # per-batch factors: other kernels
    check(fk, ko.MKM, M, Ps, Ps, np.float64, alpha=1.0, beta=1.0, seed=505, integer=True)


@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
def test_more_batches_than_a_grid_dimension_holds(fk, mm):
    """70000 small problems in one strided-batched call: the batch index is a grid dimension of at most 65535,
    so the launches go out in chunks."""
    check(fk, mm, 2, [4, 3], [3, 4], np.float32, alpha=1.5, beta=0.5, seed=601, batch=70000)
    check(fk, mm, 3, [2, 2, 2], [2, 2, 2], np.float64, alpha=1.0, beta=0.0, seed=602, batch=66000, share_f=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M,Ps,launches", [(16, [16, 16], 1), (37, [16] * 4, 2), (100, [16] * 3, 2), (5, [3, 16, 16], 2),
                                           (2048, [16, 16], 1)])
def test_kmm_layout_pair_of_16x16_factors(fk, M, Ps, launches, dt):
    """GeKMM chains of 16x16 factors: two factors per launch, tiles of 16 columns of X including ragged ones."""
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=701)
    plan = fk.last_plan()
    assert any("_16x16_16x16_2_16x256_" in k for _, _, k in plan) and len(plan) == launches, plan
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=702, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=703, batch=3)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=704, integer=True)


@pytest.mark.parametrize("M,Ps,launches", [(96, [32] * 3, 1), (101, [32] * 3, 1), (128, [32] * 3, 1), (3, [32] * 4, 2),
                                           (24, [4, 32, 32, 32], 2), (1, [32] * 5, 3)])
def test_whole_row_kernel_for_three_32x32_factors(fk, M, Ps, launches):
    """fp32 32x32^3 on rows (or contiguous blocks) of 32768 columns: one launch, one LDS exchange; longer chains
    apply the three trailing factors block by block and the leading ones in the KMM layout.  (With fewer than 96
    blocks the pair kernel plus one more step is faster and is chosen instead.)"""
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=1001)
    plan = fk.last_plan()
    assert any("_f_32x32_32x32_3_1x32768_" in k for _, _, k in plan) and len(plan) == launches, plan
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=1002, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=1003, batch=3, share_f=True)
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=2.0, beta=0.0, seed=1004, batch=2)
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=1005, integer=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M,Ps,launches", [(16, [12, 12], 1), (37, [9, 9], 1), (5, [15, 15], 1), (100, [10] * 4, 2),
                                           (33, [13] * 3, 2), (1, [11, 11], None)])
def test_kmm_layout_pair_of_factors_of_9_to_15(fk, M, Ps, launches, dt):
    """GeKMM chains of PxP factors with 9 <= P <= 15: the 16x16 pair kernel with zero-padded operands and masked
    rows; a single column of X (M = 1) takes another kernel."""
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=711)
    plan = fk.last_plan()
    if launches is not None:
        assert any("_16x16_16x16_2_16x256_" in k for _, _, k in plan) and len(plan) == launches, plan
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=712, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=713, batch=3)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=2.0, beta=0.0, seed=714, opX=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=715, integer=True)


@pytest.mark.parametrize("M,Ps", [(5, [16] * 3), (7, [16, 16, 16]), (48, [16, 16]), (3, [2, 8, 16, 16])])
def test_fp32_16x16_wave_per_block_kernel_where_the_workgroup_kernel_needs_whole_blocks(fk, M, Ps):
    """fp32 16x16^3 with a row count that is no multiple of 16: one wave per 4096-element block instead of the
    workgroup kernel that packs 16 rows into a 16^4 block."""
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=801)
    plan = fk.last_plan()
    if M % 16:
        assert any("_f_16x16_16x16_3_1x4096_" in k for _, _, k in plan), plan
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=802, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=803, batch=2, share_f=True)
    check(fk, ko.MKM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=804, integer=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M,Ps,launches", [(5, [10] * 3, 1), (7, [12] * 3, 1), (24, [12, 12], 1), (3, [9] * 3, 1),
                                           (2, [15] * 3, 1), (3, [10] * 4, 2), (2, [12] * 5, None), (4, [13] * 3, 1)])
def test_wave_per_block_kernel_with_factors_of_9_to_15(fk, M, Ps, launches, dt):
    """Two or three PxP factors with 9 <= P <= 15 on blocks of P^3 elements: the 16x16x3 wave-per-block kernel with
    zero-padded operands and masked lanes; longer chains apply the three trailing factors block by block."""
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=901)
    plan = fk.last_plan()
    assert any("_16x16_16x16_3_1x4096_" in k for _, _, k in plan), plan
    if launches is not None:
        assert len(plan) == launches, plan
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=902, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=903, batch=3, share_f=True)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=2.0, beta=0.0, seed=904, batch=2)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=905, integer=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("M,Ps,launches", [(16, [24, 24], 1), (5, [31, 31], 1), (7, [17, 17], 1), (3, [24] * 3, 2),
                                           (2, [20] * 4, 3), (40, [28, 28], 1)])
def test_pair_kernel_with_factors_of_17_to_31(fk, M, Ps, launches, dt):
    """Two fused PxP factors, 17 <= P <= 31, on the 32x32 pair kernel with zero-padded operands (the reference fuses
    square factors up to 32x32, reference src/kernel_db/kernel_db.cpp:164-181); longer chains take it for their two
    trailing factors and run the leading ones across the blocks."""
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.5, beta=0.5, seed=181)
    plan = fk.last_plan()
    assert len(plan) == launches and "_32x32_32x32_2_1x1024" in plan[0][2], plan
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=0.0, seed=182, opFs=ko.OP_T)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=1.0, beta=1.0, seed=183, batch=2)
    check(fk, ko.MKM, M, Ps, Ps, dt, alpha=2.0, beta=0.0, seed=184, integer=True)


# ---- single steps with 32x32 / 64x64 / 128x128 factors on tiles of 16 KB passed through LDS (both layouts and types) ----
@pytest.mark.parametrize("mm,M,Ps,kw", [
    (ko.MKM, 4, [128, 128], {}), (ko.MKM, 3, [64, 64], dict(alpha=1.5, beta=0.5)),
    (ko.MKM, 5, [128, 128], dict(alpha=2.0, beta=-1.0, batch=2, opFs=ko.OP_T)), (ko.MKM, 2, [64, 64, 64], {}),
    (ko.MKM, 1, [128, 128, 128], dict(beta=1.0)), (ko.MKM, 600, [128, 128], {}),
    (ko.KMM, 64, [128, 128], {}), (ko.KMM, 128, [64, 64], dict(alpha=1.5, beta=0.5)),
    (ko.KMM, 32, [128, 128], dict(alpha=2.0, beta=-1.0, batch=2, opFs=ko.OP_T)), (ko.KMM, 192, [64, 64, 64], {}),
    (ko.KMM, 64, [128, 128], dict(batch=3, share_f=True, beta=1.0, share_y=True)),
    (ko.MKM, 7, [128, 128], dict(use_temp2=False, beta=0.25)),
    (ko.KMM, 256, [32, 32], dict(alpha=1.5, beta=0.5)), (ko.KMM, 128, [32, 32, 32], dict(batch=2, opFs=ko.OP_T, beta=1.0))])
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_wide_step_kernel(fk, mm, M, Ps, kw, dt):
    if dt == np.float64 and mm == ko.KMM:
        M = M // 2                      # fp64 tiles hold half as many columns
    check(fk, mm, M, Ps, Ps, dt, seed=71, **kw)
    if dt == np.float64 and Ps[0] == 64 and mm == ko.KMM:
        return                          # the 4x4x4 KMM step is preferred for fp64 64x64
    assert all("mfma16x16x4lds" in k for _, _, k in fk.last_plan()), fk.last_plan()


@pytest.mark.parametrize("mm,M,Ps", [(ko.KMM, 16, [128, 128]), (ko.KMM, 48, [64, 64]), (ko.KMM, 100, [128, 128]),
                                     (ko.KMM, 64, [32, 32])])
def test_wide_step_kernel_needs_whole_tiles(fk, mm, M, Ps):
    """Fewer columns than a tile's 32 (64, 128) in the KMM layout, or not a multiple of it: the streaming step runs."""
    check(fk, mm, M, Ps, Ps, np.float32, seed=72, alpha=1.5, beta=0.5)
    assert not any("mfma16x16x4lds" in k for _, _, k in fk.last_plan()), fk.last_plan()


@pytest.mark.parametrize("M,Ps", [(32, [16, 16]), (96, [16] * 4), (64, [12, 12]), (32, [9, 9, 9, 9]), (48, [16, 16]), (160, [15, 15])])
def test_kmm_pairs_of_16x16_with_two_columns_per_lane(fk, M, Ps):
    """sgekmm with pairs of 16x16 (9x9 ... 15x15) factors: with a multiple of 32 columns a lane owns two neighbouring
    columns and moves them as 8-byte elements (48 columns: one column per lane as before)."""
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=211)
    assert any("_2_16x256_" in k for _, _, k in fk.last_plan()), fk.last_plan()
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=212, opFs=ko.OP_T)
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=213, batch=3)
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=2.0, beta=0.0, seed=214, batch=2, share_f=True)
    check(fk, ko.KMM, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=215, integer=True, use_temp2=False)


@pytest.mark.parametrize("mm,M,Ps,launches", [(ko.KMM, 64, [8] * 3, 1), (ko.KMM, 128, [8] * 5, 2), (ko.KMM, 192, [8] * 6, 2),
                                              (ko.KMM, 64, [4, 8, 8, 8], 2), (ko.MKM, 2, [8] * 8, 2), (ko.KMM, 80, [8] * 3, 2)])
def test_kmm_three_fused_8x8_factors(fk, mm, M, Ps, launches):
    """sgekmm chains of 8x8 factors: three per launch on 512 rows by 64 columns per workgroup (a multiple of 64 columns;
    80 columns keep the two-factor kernel), also for the leading factors of a long sgemkm chain."""
    check(fk, mm, M, Ps, Ps, np.float32, alpha=1.5, beta=0.5, seed=221)
    plan = fk.last_plan()
    assert len(plan) == launches and (M % 64 != 0 and mm == ko.KMM or any("_8x8_8x8_3_64x512_" in k for _, _, k in plan)), plan
    check(fk, mm, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=222, opFs=ko.OP_T)
    check(fk, mm, M, Ps, Ps, np.float32, alpha=1.0, beta=1.0, seed=223, batch=3)
    check(fk, mm, M, Ps, Ps, np.float32, alpha=2.0, beta=0.0, seed=224, batch=2, share_f=True)
    check(fk, mm, M, Ps, Ps, np.float32, alpha=1.0, beta=0.0, seed=225, integer=True, use_temp2=False)


# ---- Z == Y: the epilogue reads Y and writes Z through one buffer (allowed with two temporaries, reference
# include/fastkron.h:274-277, src/handle/handle.cpp:120-122).  Every kernel family that has a Y epilogue: each reads
# Y and writes Z from registers laid out its own way, and must read an element before it writes it. ----
IN_PLACE = [
    # kernel family, mm, M, Ps, Qs, dtype, extra
    ("whole-column 4x4^6", ko.KMM, 1032, [4] * 6, [4] * 6, np.float32, {}),
    ("4x4x3 register kernel, two launches", ko.KMM, 100, [4] * 6, [4] * 6, np.float32, {}),
    ("32x16^3 row kernel, batched", ko.MKM, 8, [32] * 3, [16] * 3, np.float32, dict(batch=3)),
    ("16x16^4 row kernel", ko.MKM, 6, [16] * 4, [16] * 4, np.float32, {}),
    ("8x8^5 row kernel", ko.MKM, 5, [8] * 5, [8] * 5, np.float32, {}),
    ("8x8^5 row kernel fp64", ko.MKM, 128, [8] * 5, [8] * 5, np.float64, {}),
    ("32x32^3 row kernel", ko.MKM, 3, [32] * 3, [32] * 3, np.float32, {}),
    ("16x16^3 wave-per-block fp64", ko.MKM, 8, [16] * 3, [16] * 3, np.float64, {}),
    ("16x16^3 wave-per-block fp32", ko.MKM, 8, [16] * 3, [16] * 3, np.float32, {}),
    ("64x64 pair fp64", ko.MKM, 600, [64] * 2, [64] * 2, np.float64, {}),
    ("64x64 pair fp32", ko.MKM, 600, [64] * 2, [64] * 2, np.float32, {}),
    ("32x32 pair fp64", ko.MKM, 40, [32] * 2, [32] * 2, np.float64, {}),
    ("padded 24x24 pair", ko.MKM, 16, [24] * 2, [24] * 2, np.float32, {}),
    ("two-part plan fp32", ko.MKM, 4, [16] * 5, [16] * 5, np.float32, {}),
    ("two-part plan fp64, KMM-layout 64x64 step", ko.MKM, 2, [64] * 3, [64] * 3, np.float64, {}),
    ("two-part plan 8x8^7", ko.MKM, 2, [8] * 7, [8] * 7, np.float32, {}),
    ("GeKMM as GeMKM + transposition", ko.KMM, 64, [8] * 5, [8] * 5, np.float32, dict(opX=ko.OP_T)),
    ("GeKMM as GeMKM + transposition fp64", ko.KMM, 64, [16] * 3, [16] * 3, np.float64, dict(opX=ko.OP_T, opFs=ko.OP_T)),
    ("transposed copy of X first", ko.MKM, 64, [8] * 5, [8] * 5, np.float32, dict(opX=ko.OP_T)),
    ("8x8^3 KMM kernel", ko.KMM, 128, [8] * 3, [8] * 3, np.float32, {}),
    ("16x16^2 KMM kernel", ko.KMM, 96, [16] * 2, [16] * 2, np.float32, {}),
    ("16x16^2 KMM kernel fp64", ko.KMM, 96, [16] * 2, [16] * 2, np.float64, {}),
    ("64x64 KMM step fp64", ko.KMM, 128, [64], [64], np.float64, {}),
    ("wide step 128x128", ko.MKM, 64, [128] * 2, [128] * 2, np.float32, {}),
    ("wide step KMM 64x64", ko.KMM, 256, [64] * 2, [64] * 2, np.float32, {}),
    ("streaming step 16x16", ko.MKM, 33, [16], [16], np.float32, {}),
    ("padded step 31x63", ko.MKM, 16, [31] * 2, [63] * 2, np.float32, {}),
    ("padded step 50x50 fp64 KMM", ko.KMM, 48, [50] * 2, [50] * 2, np.float64, {}),
    ("LDS-fused small factors", ko.MKM, 16, [3] * 7, [3] * 7, np.float32, {}),
    ("LDS-fused small factors KMM", ko.KMM, 64, [5] * 4, [5] * 4, np.float64, {}),
    ("LDS-fused rectangular", ko.MKM, 16, [2] * 5, [4] * 5, np.float32, {}),
    ("merged 4x4^8", ko.MKM, 8, [4] * 8, [4] * 8, np.float32, {}),
    ("generic", ko.MKM, 7, [297], [127], np.float32, {}),
    ("generic KMM", ko.KMM, 20, [5, 1, 7], [1, 6, 2], np.float64, {}),
]


@pytest.mark.parametrize("family,mm,M,Ps,Qs,dt,extra", IN_PLACE, ids=[c[0] for c in IN_PLACE])
def test_z_is_y(fk, family, mm, M, Ps, Qs, dt, extra):
    check(fk, mm, M, Ps, Qs, dt, alpha=1.5, beta=0.5, seed=501, y_is_z=True, **extra)
    check(fk, mm, M, Ps, Qs, dt, alpha=-1.0, beta=2.0, seed=502, y_is_z=True, integer=True, **extra)


def test_z_is_y_needs_the_second_temporary(fk):
    """reference src/handle/handle.cpp:120-122"""
    import torch
    Ps = [8] * 3
    X = torch.zeros(4 * 512, device="cuda:0")
    Fs = [torch.zeros(64, device="cuda:0") for _ in Ps]
    Z = torch.zeros(4 * 512, device="cuda:0")
    t1 = torch.zeros(4 * 512, device="cuda:0")
    assert fk.xgemkm(4, Ps, Ps, X, Fs, Z, 1.0, 1.0, Z, t1, None) == 4


def test_z_is_y_at_full_size_on_the_two_phase_4x4_kernel(fk):
    from tests.gpu_util import sampled_check
    err_rows, err_sum = sampled_check(fk, ko.KMM, 2048, [4] * 6, [4] * 6, np.float32, alpha=1.5, beta=0.5, y_is_z=True)
    assert [k for _, _, k in fk.last_plan()] == [TWO_PHASE_4X6], fk.last_plan()
    assert err_rows <= 1e-5 and err_sum <= 1e-5, (err_rows, err_sum)
    err_rows, err_sum = sampled_check(fk, ko.MKM, 1024, [16] * 4, [16] * 4, np.float32, alpha=2.0, beta=-0.5, y_is_z=True)
    assert err_rows <= 1e-5 and err_sum <= 1e-5, (err_rows, err_sum)
    err_rows, err_sum = sampled_check(fk, ko.MKM, 256, [64] * 3, [64] * 3, np.float64, alpha=1.0, beta=1.0, y_is_z=True)
    assert err_rows <= 1e-12 and err_sum <= 1e-12, (err_rows, err_sum)


def test_two_part_plan_in_row_chunks(monkeypatch):
    """FASTKRON_CHUNK_MB: the rows of a two-part plan go through its two parts in chunks that share one stretch of
    temp1 (off by default).  Chunks of 1 MB: 16 rows of 16^4 fp32 at a time, the last chunk ragged; with Y, Z == Y."""
    import fastkron_amd
    monkeypatch.setenv("FASTKRON_CHUNK_MB", "1")
    h = fastkron_amd.FastKron()
    monkeypatch.delenv("FASTKRON_CHUNK_MB")
    try:
        check(h, ko.MKM, 5, [16] * 5, [16] * 5, np.float32, alpha=1.5, beta=0.5, seed=601)       # 4 MB per row: row by row
        assert len(h.last_plan()) == 2, h.last_plan()
        check(h, ko.MKM, 37, [8] * 6, [8] * 6, np.float32, alpha=1.0, beta=0.0, seed=602)        # 1 MB per row
        check(h, ko.MKM, 70, [16] * 4, [16] * 4, np.float64, alpha=2.0, beta=1.0, seed=603, y_is_z=True)   # 2 rows per chunk
        check(h, ko.MKM, 3, [64] * 3, [64] * 3, np.float64, alpha=1.0, beta=0.0, seed=604)
    finally:
        h.close()
