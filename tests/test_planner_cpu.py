"""Host-side tests of the launch planner through the C ABI in plan-only mode (include/fastkron_ext.h): every
argument check, the planner and each kernel's check of the concrete buffers run, nothing is launched, no GPU is
needed.  Covered here: which kernels a problem gets, what the launches are handed (strides, batch counts), and the
fallback to plainer kernels when a buffer does not have the alignment a kernel's vector accesses need
(the reference's counterpart is the optimisation level of a kernel, reference src/kernels/kernel_opt.h:42-84,
checked per problem in KMMKernel::canCompute, src/kernels/kmmkernel.cpp:85-126)."""
import ctypes

import pytest

from fastkron_amd import capi

BASE = 0x7000_0000_0000          # fake device addresses, 4 GiB apart; never dereferenced in plan-only mode
GAP = 1 << 32


@pytest.fixture
def planner():
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.fastKronInit(ctypes.byref(h), capi.BACKEND_HIP) == capi.SUCCESS
    assert lib.fastKronSetPlanOnly(h, 1) == capi.SUCCESS
    yield lib, h
    lib.fastKronDestroy(h)


@pytest.fixture
def online_planner(monkeypatch):
    """A plan-only handle without the shipped tuned plans: the online rules alone."""
    monkeypatch.setenv("FASTKRON_SHIPPED_PLANS", "0")
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.fastKronInit(ctypes.byref(h), capi.BACKEND_HIP) == capi.SUCCESS
    assert lib.fastKronSetPlanOnly(h, 1) == capi.SUCCESS
    yield lib, h
    lib.fastKronDestroy(h)


def plan(planner, mm, dt, M, Ps, Qs, batch=None, alpha=1.0, beta=0.0, with_y=False, offs=None, strides=None,
         strideF=None, opX=capi.OP_N, opF=capi.OP_N, temp2=True, y_is_z=False):
    """Runs one call in plan-only mode.  `offs` shifts the fake base pointers of x / z / y / t1 / t2 by bytes,
    `strides` overrides the element strides of x / z / y.  Returns (error, kernel names, launch records)."""
    lib, h = planner
    offs = offs or {}
    K, L = 1, 1
    for p, q in zip(Ps, Qs):
        K, L = K * p, L * q
    ptr = {n: BASE + i * GAP + offs.get(n, 0) for i, n in enumerate(["x", "z", "y", "t1", "t2"])}
    if y_is_z:
        ptr["y"] = ptr["z"]
    fs = capi.arr_ptr([BASE + (8 + i) * GAP + offs.get("f", 0) for i in range(len(Ps))])
    sc = ctypes.c_float if dt == "s" else ctypes.c_double
    X, Z = ctypes.c_void_p(ptr["x"]), ctypes.c_void_p(ptr["z"])
    Y = ctypes.c_void_p(ptr["y"]) if (with_y or y_is_z) else None
    t1, t2 = ctypes.c_void_p(ptr["t1"]), (ctypes.c_void_p(ptr["t2"]) if temp2 else None)
    PsA, QsA = capi.arr_u32(Ps), capi.arr_u32(Qs)
    if batch is None:
        if mm == "mkm":
            e = getattr(lib, dt + "gemkm")(h, capi.BACKEND_HIP, M, len(Ps), PsA, QsA, X, opX, fs, opF, Z, sc(alpha), sc(beta),
                                           Y, t1, t2)
        else:
            e = getattr(lib, dt + "gekmm")(h, capi.BACKEND_HIP, len(Ps), QsA, PsA, M, fs, opF, X, opX, Z, sc(alpha), sc(beta),
                                           Y, t1, t2)
    else:
        st = {"x": M * K, "z": M * L, "y": M * L}
        st.update(strides or {})
        sF = capi.arr_u64(strideF if strideF is not None else [p * q for p, q in zip(Ps, Qs)])
        if mm == "mkm":
            e = getattr(lib, dt + "gemkmStridedBatched")(h, capi.BACKEND_HIP, M, len(Ps), PsA, QsA, X, opX, st["x"], fs, opF,
                                                         sF, Z, st["z"], sc(alpha), sc(beta), batch, Y, st["y"], t1, t2)
        else:
            e = getattr(lib, dt + "gekmmStridedBatched")(h, capi.BACKEND_HIP, len(Ps), QsA, PsA, M, fs, opF, sF, X, opX,
                                                         st["x"], Z, st["z"], sc(alpha), sc(beta), batch, Y, st["y"], t1, t2)
    buf = ctypes.create_string_buffer(1 << 16)
    lib.fastKronGetLastPlan(h, buf, len(buf))
    names = [s.split(":")[1] for s in buf.value.decode().split(";")[1:]]
    lib.fastKronGetLastLaunches(h, buf, len(buf))
    launches = []
    for line in buf.value.decode().splitlines():
        rec = dict(kv.split("=", 1) for kv in line.split())
        rec["f_batch"] = [int(v) for v in rec["f_batch"].split(",")]
        launches.append(rec)
    return e, names, launches


# ---- a strided-batched call with one batch entry must not carry its strides into any launch ----
@pytest.mark.parametrize("dt,M,P,N", [("s", 8, 16, 5), ("s", 4, 8, 6), ("s", 2, 32, 4), ("d", 8, 16, 4), ("d", 2, 64, 3),
                                      ("s", 16, 4, 8), ("d", 4, 8, 5), ("s", 4, 12, 4)])
def test_single_entry_batches_carry_no_strides(planner, dt, M, P, N):
    e, names, launches = plan(planner, "mkm", dt, M, [P] * N, [P] * N, batch=1)
    assert e == capi.SUCCESS
    assert len(launches) >= 1
    for rec in launches:
        assert rec["f_batch"] == [0] * len(rec["f_batch"]), (names, rec)
    # ... and it gets the plan of the plain entry point
    e2, names2, launches2 = plan(planner, "mkm", dt, M, [P] * N, [P] * N)
    assert e2 == capi.SUCCESS and names2 == names
    assert [r["batch"] for r in launches2] == [r["batch"] for r in launches]


def test_two_part_plan_reads_leading_factors_with_stride_zero(planner):
    """M rows become batch entries of the leading part: per-entry factor strides there would walk off F."""
    e, names, launches = plan(planner, "mkm", "s", 8, [16] * 5, [16] * 5, batch=1)
    assert e == capi.SUCCESS and len(launches) == 2
    assert "_16x16_16x16_4_1x65536" in launches[0]["kernel"] and int(launches[0]["M"]) == 8 * 16
    assert int(launches[1]["batch"]) == 8 and launches[1]["f_batch"] == [0]
    # per-batch leading factors rule the two-part plan out altogether
    e, names, launches = plan(planner, "mkm", "s", 8, [16] * 5, [16] * 5, batch=2)
    assert e == capi.SUCCESS
    assert all(int(r["batch"]) == 2 for r in launches), launches
    # shared factors (stride 0) with several batch entries keep it
    e, names, launches = plan(planner, "mkm", "s", 8, [16] * 5, [16] * 5, batch=2, strideF=[0] * 5)
    assert e == capi.SUCCESS and int(launches[-1]["batch"]) == 16 and launches[-1]["f_batch"] == [0]


def test_fp64_rows_of_five_8x8_factors_get_the_whole_row_kernel(online_planner):
    """dgemkm 8x8^5 from 32 rows on: one launch of the fp64 row kernel on the chain as given (no 64x64 products); with
    fewer rows, with eight factors or in the KMM layout the chain is merged as before."""
    row = "mkm_hip_gfx950_512_d_8x8_8x8_5_1x32768_valu_NN_strided_0_3"
    for M, opF in [(1024, capi.OP_N), (32, capi.OP_T)]:
        e, names, launches = plan(online_planner, "mkm", "d", M, [8] * 5, [8] * 5, opF=opF, beta=0.5, with_y=True)
        assert e == capi.SUCCESS and names == [row], names
    e, names, _ = plan(online_planner, "mkm", "d", 31, [8] * 5, [8] * 5)
    assert e == capi.SUCCESS and row not in names and any("64x64" in n for n in names), names
    # six or seven factors: the row kernel on the blocks of 32768 columns, the leading factor(s) across the blocks
    e, names, launches = plan(online_planner, "mkm", "d", 1024, [8] * 6, [8] * 6)
    assert e == capi.SUCCESS and len(names) == 2 and names[0] == row and int(launches[0]["M"]) == 8192, (names, launches)
    e, names, launches = plan(online_planner, "mkm", "d", 16, [8] * 7, [8] * 7)
    assert e == capi.SUCCESS and len(names) == 2 and names[0] == row and "64x64" in names[1], names
    e, names, _ = plan(online_planner, "mkm", "d", 3, [8] * 6, [8] * 6)           # 24 blocks: merged as before
    assert e == capi.SUCCESS and row not in names and any("64x64" in n for n in names), names
    e, names, _ = plan(online_planner, "mkm", "d", 16, [8] * 8, [8] * 8)
    assert e == capi.SUCCESS and row not in names, names
    e, names, _ = plan(online_planner, "kmm", "d", 1024, [8] * 5, [8] * 5)
    assert e == capi.SUCCESS and row not in names, names
    # per-batch factors: every batch entry reads its own five factors
    e, names, launches = plan(online_planner, "mkm", "d", 16, [8] * 5, [8] * 5, batch=4)
    assert e == capi.SUCCESS and names == [row] and launches[0]["f_batch"] == [64] * 5, (names, launches)


def test_rows_of_three_32x32_factors_choose_the_kernel_by_row_count(online_planner):
    """sgemkm 32x32^3: from three rows per CU on the persistent kernel (one workgroup of 16 waves per CU), from 96 rows on
    the kernel with two workgroups of 8 waves per CU, below that the pair kernel and a step; the same on the blocks of
    a longer chain."""
    pers = "mkm_hip_gfx950_1024_f_32x32_32x32_3_1x32768_mfma16x16x4_NN_strided_0_3"
    two = "mkm_hip_gfx950_512_f_32x32_32x32_3_1x32768_mfma16x16x4_NN_strided_0_3"
    for M, want in [(1024, [pers]), (768, [pers]), (767, [two]), (96, [two])]:
        e, names, _ = plan(online_planner, "mkm", "s", M, [32] * 3, [32] * 3, beta=0.5, with_y=True)
        assert e == capi.SUCCESS and names == want, (M, names)
    e, names, _ = plan(online_planner, "mkm", "s", 95, [32] * 3, [32] * 3)
    assert e == capi.SUCCESS and pers not in names and two not in names and len(names) == 2, names
    e, names, launches = plan(online_planner, "mkm", "s", 24, [32] * 4, [32] * 4)          # 768 blocks
    assert e == capi.SUCCESS and names[0] == pers and int(launches[0]["M"]) == 768, (names, launches)
    e, names, _ = plan(online_planner, "mkm", "s", 96, [32] * 3, [32] * 3, batch=8)         # 768 rows in all
    assert e == capi.SUCCESS and names == [pers], names
    # a misaligned operand sends both away (16-byte accesses)
    e, names, _ = plan(online_planner, "mkm", "s", 1024, [32] * 3, [32] * 3, offs={"x": 4})
    assert e == capi.SUCCESS and pers not in names and two not in names, names


def test_rectangular_pairs_get_the_pair_kernel_and_the_two_part_plan(online_planner):
    """Two 32x64 / 64x32 factors: one launch on exact tiles; three: the pair on the blocks of a row (M * P virtual rows of
    P*P columns, Q*Q out) and the leading factor across the blocks as a KMM problem with one batch entry per row."""
    for dt, P, Q in [("s", 32, 64), ("s", 64, 32), ("d", 32, 64)]:
        name = f"mkm_hip_gfx950_256_{'f' if dt == 's' else 'd'}_{P}x{Q}_{P}x{Q}_2_1x{P * P}_mfma16x16x4_NN_strided_0_3"
        e, names, launches = plan(online_planner, "mkm", dt, 40, [P] * 2, [Q] * 2, beta=0.5, with_y=True)
        assert e == capi.SUCCESS and names == [name], names
        e, names, launches = plan(online_planner, "mkm", dt, 3, [P] * 3, [Q] * 3, beta=0.5, with_y=True)
        assert e == capi.SUCCESS and len(names) == 2 and names[0] == name, names
        assert int(launches[0]["M"]) == 3 * P and int(launches[0]["out"], 16) == BASE + 3 * GAP, launches      # into temp1
        assert int(launches[1]["M"]) == Q * Q and int(launches[1]["batch"]) == 3, launches
        assert int(launches[1]["in"], 16) == BASE + 3 * GAP and int(launches[1]["out"], 16) == BASE + 1 * GAP, launches
    # fp64 64x32 has no such kernel (a 64 x 64 tile of doubles per row in flight): one launch per factor
    e, names, _ = plan(online_planner, "mkm", "d", 40, [64] * 2, [32] * 2)
    assert e == capi.SUCCESS and len(names) == 2 and all("_2_1x" not in n for n in names), names
    # the leading factors of a two-part plan are shared between the rows: per-batch factors rule it out
    e, names, _ = plan(online_planner, "mkm", "s", 3, [32] * 3, [64] * 3, batch=2)
    assert e == capi.SUCCESS and len(names) == 3, names


def test_pairs_of_64x64_fp64_factors_by_block_count(online_planner):
    """dgemkm 64x64^2: the pair kernel from 8 blocks per CU on (a block per wave) and between 1.25 and 4 blocks per CU
    (a block shared by waves); otherwise two single steps."""
    pair = "mkm_hip_gfx950_512_d_64x64_64x64_2_1x4096_mfma4x4x4_NN_strided_0_3"
    for M, fused in [(256, False), (319, False), (320, True), (512, True), (1024, True), (1025, False), (2047, False),
                     (2048, True), (16384, True)]:
        e, names, _ = plan(online_planner, "mkm", "d", M, [64] * 2, [64] * 2)
        assert e == capi.SUCCESS and (names == [pair]) == fused and len(names) == (1 if fused else 2), (M, names)
    e, names, launches = plan(online_planner, "mkm", "d", 8, [64] * 3, [64] * 3)            # 512 blocks of a longer chain
    assert e == capi.SUCCESS and names[0] == pair and int(launches[0]["M"]) == 512, (names, launches)


# ---- kernels with 16-byte global accesses are only chosen for buffers that allow them ----
VECTOR_CASES = [
    # (label, mm, dt, M, Ps, Qs, batch, beta, substring of the kernel expected on aligned buffers)
    ("row16x4", "mkm", "s", 128, [16] * 4, [16] * 4, None, 0.5, "_16x16_16x16_4_1x65536"),
    ("row16x3", "mkm", "s", 64, [16] * 3, [16] * 3, None, 0.5, "_16x16_16x16_3_1x4096"),
    ("row16x3d", "mkm", "d", 64, [16] * 3, [16] * 3, None, 0.5, "_d_16x16_16x16_3_1x4096"),
    ("row32x3", "mkm", "s", 128, [32] * 3, [32] * 3, None, 0.5, "_32x32_32x32_3_1x32768"),
    ("pair32", "mkm", "s", 64, [32] * 2, [32] * 2, None, 0.5, "_32x32_32x32_2_1x1024"),
    ("pair64d", "mkm", "d", 2048, [64] * 2, [64] * 2, None, 0.5, "_d_64x64_64x64_2_1x4096"),
    ("step64", "mkm", "s", 64, [64], [64], None, 0.5, "_64x64_64x64_1_"),
    ("kmm64d", "kmm", "d", 64, [64], [64], 8, 0.5, "kmm_hip_gfx950_256_d_64x64_64x64_1_64x64"),
    ("row8x5", "mkm", "s", 64, [8] * 5, [8] * 5, None, 0.5, "_8x8_8x8_5_1x32768"),
    ("row32x16", "mkm", "s", 64, [32] * 3, [16] * 3, None, 0.5, "_32x16_32x16_3_1x32768"),
    ("kmm4x6", "kmm", "s", 1032, [4] * 6, [4] * 6, None, 0.5, "_4x4_4x4_6_8x4096"),
    ("kmm4x6 two-phase", "kmm", "s", 2048, [4] * 6, [4] * 6, None, 0.5, "_4x4_4x4_6_256x4096"),
    ("wide128", "mkm", "s", 8, [128] * 2, [128] * 2, None, 0.5, "_128x128_128x128_1_1x4096_mfma16x16x4lds"),
    ("wide64k", "kmm", "s", 64, [64] * 2, [64] * 2, None, 0.5, "_64x64_64x64_1_64x64_mfma16x16x4lds"),
]


@pytest.mark.parametrize("case", VECTOR_CASES, ids=[c[0] for c in VECTOR_CASES])
def test_aligned_buffers_get_the_specialised_kernel(planner, case):
    _, mm, dt, M, Ps, Qs, batch, beta, want = case
    e, names, _ = plan(planner, mm, dt, M, Ps, Qs, batch=batch, beta=beta, with_y=True)
    assert e == capi.SUCCESS
    assert any(want in n for n in names), names


@pytest.mark.parametrize("which", ["x", "z", "y"])
@pytest.mark.parametrize("case", VECTOR_CASES, ids=[c[0] for c in VECTOR_CASES])
def test_a_buffer_off_by_one_element_still_gets_a_plan_that_accepts_it(planner, case, which):
    """The base pointer of X, Z or Y is moved by one element: whatever plan comes back passed every kernel's own
    check of these buffers (plan-only mode runs them), and the call does not fail."""
    _, mm, dt, M, Ps, Qs, batch, beta, want = case
    esize = 4 if dt == "s" else 8
    e, names, launches = plan(planner, mm, dt, M, Ps, Qs, batch=batch, beta=beta, with_y=True, offs={which: esize})
    assert e == capi.SUCCESS and len(launches) >= 1, names


VECTOR_KERNELS_NEEDING = {
    # kernels whose 16-byte accesses make them refuse a misaligned operand: label -> operands they vector-access
    "row16x4": "xzy", "row16x3": "x", "row16x3d": "x", "row32x3": "xzy", "pair32": "x", "pair64d": "xzy", "step64": "x",
    "kmm64d": "xzy", "wide128": "xzy", "wide64k": "xzy",
}


@pytest.mark.parametrize("label,which", [(k, w) for k, ws in VECTOR_KERNELS_NEEDING.items() for w in ws])
def test_misaligned_operand_rules_the_vector_kernel_out(planner, label, which):
    case = [c for c in VECTOR_CASES if c[0] == label][0]
    _, mm, dt, M, Ps, Qs, batch, beta, want = case
    esize = 4 if dt == "s" else 8
    e, names, _ = plan(planner, mm, dt, M, Ps, Qs, batch=batch, beta=beta, with_y=True, offs={which: esize})
    assert e == capi.SUCCESS
    assert not any(want in n for n in names), (which, names)


@pytest.mark.parametrize("label", ["row16x4", "row32x3", "pair64d", "row16x3"])
@pytest.mark.parametrize("which", ["x", "z", "y"])
def test_odd_batch_strides_rule_the_vector_kernel_out(planner, label, which):
    """Batch entries one element further apart than the operand is long: entry 1 is misaligned although entry 0 is not."""
    case = [c for c in VECTOR_CASES if c[0] == label][0]
    _, mm, dt, M, Ps, Qs, _, beta, want = case
    K, L = 1, 1
    for p, q in zip(Ps, Qs):
        K, L = K * p, L * q
    odd = {"x": M * K + 1, "z": M * L + 1, "y": M * L + 1}[which]
    e, names, launches = plan(planner, mm, dt, M, Ps, Qs, batch=3, beta=beta, with_y=True, strides={which: odd},
                              strideF=[0] * len(Ps))
    assert e == capi.SUCCESS
    needs = VECTOR_KERNELS_NEEDING[label]
    if which in needs:
        assert not any(want in n for n in names), (which, names)


def test_batches_beyond_one_grid_dimension_are_checked_chunk_by_chunk(planner):
    e, names, launches = plan(planner, "mkm", "s", 1, [16, 16], [16, 16], batch=70000, strideF=[0, 0])
    assert e == capi.SUCCESS
    assert [int(r["batch"]) for r in launches] == [65535, 70000 - 65535] * (len(launches) // 2)
    first, second = launches[0], launches[1]
    assert int(second["in"], 16) - int(first["in"], 16) == 65535 * 256 * 4


# ---- tuned-plan files are not trusted ----
def test_tuned_plans_that_do_not_fit_the_problem_are_ignored(planner, tmp_path):
    lib, h = planner
    e, online, _ = plan(planner, "mkm", "s", 8, [8, 8, 8], [8, 8, 8])
    generic = "gekmm_hip_gfx950_256_f_generic_1"
    key = "8x512*(8x8^3)_NN_f"
    bad = [
        f"{key} 0.01 1 0 5 {generic}",                       # factor index beyond the chain
        f"{key} 0.01 2 2 2 {generic} 0 0 {generic}",         # factor 1 never applied
        f"{key} 0.01 3 0 0 {generic} 1 1 {generic} 2 2 {generic}",   # first factor first
        f"{key} 0.01 1 0 2 {generic}",                       # a one-factor kernel given three factors
        f"{key} 0.01 1 0 2 mkm_hip_gfx950_1024_f_16x16_16x16_4_1x65536_mfma16x16x4_NN_strided_0_3",   # wrong factor size
    ]
    for line in bad:
        f = tmp_path / "tuned.db"
        f.write_text(line + "\n")
        assert lib.fastKronSetTunedDB(h, str(f).encode()) == capi.SUCCESS
        e, names, _ = plan(planner, "mkm", "s", 8, [8, 8, 8], [8, 8, 8])
        assert e == capi.SUCCESS and names == online, line
    good = f"{key} 0.01 3 2 2 {generic} 1 1 {generic} 0 0 {generic}"
    f = tmp_path / "tuned.db"
    f.write_text(good + "\n")
    lib.fastKronSetTunedDB(h, str(f).encode())
    e, names, _ = plan(planner, "mkm", "s", 8, [8, 8, 8], [8, 8, 8])
    assert e == capi.SUCCESS and names == [generic] * 3


# ---- op(X) = T: a transposed copy of X ahead of the launches when that saves passes over the data ----
def test_transposed_x_is_copied_first_when_the_whole_row_kernels_then_apply(planner):
    e, names, launches = plan(planner, "mkm", "s", 64, [8] * 5, [8] * 5, opX=capi.OP_T)
    assert e == capi.SUCCESS
    assert names[0].startswith("transpose_") and "_8x8_8x8_5_1x32768" in names[1] and len(names) == 2, names
    # the launches read the copy (temp2), not X
    assert int(launches[0]["in"], 16) == BASE + 4 * GAP
    # the same for the two-part plan of a longer chain and for GeKMM
    e, names, _ = plan(planner, "mkm", "s", 8, [16] * 5, [16] * 5, opX=capi.OP_T)
    assert e == capi.SUCCESS and names[0].startswith("transpose_") and len(names) == 3, names
    # GeKMM with 64x64 factors (with small factors it runs as a GeMKM, below)
    e, names, _ = plan(planner, "kmm", "s", 64, [64] * 2, [64] * 2, opX=capi.OP_T)
    assert e == capi.SUCCESS and names[0].startswith("transpose_") and names[0].endswith("_x") and len(names) == 3, names


def test_gekmm_with_transposed_x_runs_as_the_gemkm_of_that_buffer(online_planner):
    """op(X) = T in a GeKMM means the buffer holds M x K, the X of a GeMKM with transposed factors: the whole-row GeMKM
    kernels run on it, their result goes to temp1 and one transposition (with beta * Y) writes Z."""
    planner = online_planner
    e, names, launches = plan(planner, "kmm", "s", 64, [8] * 5, [8] * 5, opX=capi.OP_T, beta=0.5, with_y=True)
    assert e == capi.SUCCESS and "mkm_" in names[0] and "_8x8_8x8_5_1x32768" in names[0] and names[-1].endswith("_z"), names
    assert len(names) == 2 and len(launches) == 1
    # the launch reads the caller's X, writes temp1, and leaves alpha in and beta * Y out
    assert int(launches[0]["in"], 16) == BASE and int(launches[0]["out"], 16) == BASE + 3 * GAP
    assert launches[0]["y"] == "(nil)"
    # a longer chain: the two-part GeMKM plan, with temp2 and Z as its temporaries
    e, names, launches = plan(planner, "kmm", "s", 1024, [8] * 6, [8] * 6, opX=capi.OP_T)
    assert e == capi.SUCCESS and len(names) == 3 and names[-1].endswith("_z"), names
    assert int(launches[-1]["out"], 16) == BASE + 3 * GAP
    # Y in place (Y == Z, beta != 0): Z cannot serve as a temporary
    e, names, launches = plan(planner, "kmm", "s", 1024, [8] * 6, [8] * 6, opX=capi.OP_T, beta=1.0, y_is_z=True)
    assert e == capi.SUCCESS and names[-1].endswith("_z"), names
    assert all(int(r["out"], 16) != BASE + GAP for r in launches), launches
    # 64x64 factors and larger only with fewer than 64 columns (and fp64 chains of three 64x64 factors)
    e, names, _ = plan(planner, "kmm", "s", 1024, [64] * 2, [64] * 2, opX=capi.OP_T)
    assert e == capi.SUCCESS and not names[-1].endswith("_z"), names
    e, names, _ = plan(planner, "kmm", "s", 16, [128] * 3, [128] * 3, opX=capi.OP_T)
    assert e == capi.SUCCESS and names[-1].endswith("_z"), names
    e, names, _ = plan(planner, "kmm", "d", 256, [64] * 3, [64] * 3, opX=capi.OP_T)
    assert e == capi.SUCCESS and names[-1].endswith("_z"), names
    e, names, _ = plan(planner, "kmm", "d", 16, [8] * 5, [8] * 5, opX=capi.OP_T)
    assert e == capi.SUCCESS and names[-1].endswith("_z"), names
    # X not transposed: only large fp32 problems with fewer than 64 columns go this way, X transposed into temp2 first
    e, names, launches = plan(planner, "kmm", "s", 16, [8] * 8, [8] * 8)
    assert e == capi.SUCCESS and names[0].endswith("_x") and names[-1].endswith("_z") and len(names) == 4, names
    assert int(launches[0]["in"], 16) == BASE + 4 * GAP and int(launches[-1]["out"], 16) == BASE + 3 * GAP, launches
    e, names, _ = plan(planner, "kmm", "s", 48, [16] * 4, [16] * 4)
    assert e == capi.SUCCESS and not names[-1].endswith("_z"), names
    e, names, _ = plan(planner, "kmm", "d", 16, [8] * 8, [8] * 8)
    assert e == capi.SUCCESS and not names[-1].endswith("_z"), names
    # rectangular factors stay on the GeKMM kernels
    e, names, _ = plan(planner, "kmm", "s", 256, [32] * 3, [16] * 3, opX=capi.OP_T)
    assert e == capi.SUCCESS and not names[-1].endswith("_z"), names


def test_transposed_x_is_read_in_place_when_a_copy_does_not_pay_or_does_not_fit(planner):
    # one small factor: the plain kernel reads the transposed X directly, a copy would add a pass
    e, names, _ = plan(planner, "mkm", "s", 64, [8], [8], opX=capi.OP_T)
    assert e == capi.SUCCESS and not any(n.startswith("transpose_") for n in names), names
    # shrinking chain: X (M x 32768) is larger than a temporary (M x 16384)
    e, names, _ = plan(planner, "mkm", "s", 64, [32] * 3, [16] * 3, opX=capi.OP_T)
    assert e == capi.SUCCESS and not any(n.startswith("transpose_") for n in names), names
    # no second temporary and a plan of several launches: temp1 cannot hold the copy
    e, names, _ = plan(planner, "mkm", "s", 8, [16] * 5, [16] * 5, opX=capi.OP_T, temp2=False)
    assert e == capi.SUCCESS and not any(n.startswith("transpose_") for n in names), names
    # no second temporary but a single launch: the copy goes to temp1
    e, names, launches = plan(planner, "mkm", "s", 64, [8] * 5, [8] * 5, opX=capi.OP_T, temp2=False)
    assert e == capi.SUCCESS and names[0].startswith("transpose_") and len(names) == 2, names
    assert int(launches[0]["in"], 16) == BASE + 3 * GAP


def test_copy_into_the_only_temporary_is_decided_on_every_calls_own_buffers(online_planner):
    """Without a second temporary the transposed copy of X sits in temp1, so the launches behind it must be one launch.
    How many they are depends on the buffers of the call at hand: a second call of the same shape whose temp1 (or Z) is
    off the alignment of the whole-row kernel gets several launches and must then read the transposed X in place;
    no launch may ever read and write the same buffer."""
    for dt, M, P, N in [("s", 1024, 16, 4), ("s", 1024, 64, 2), ("d", 1024, 32, 2)]:
        e, names, launches = plan(online_planner, "mkm", dt, M, [P] * N, [P] * N, opX=capi.OP_T, temp2=False)
        assert e == capi.SUCCESS and names[0].startswith("transpose_") and len(names) == 2, (dt, P, names)
        for offs in ({"t1": 4}, {"z": 4}, {"t1": 4, "z": 4}):
            e, names, launches = plan(online_planner, "mkm", dt, M, [P] * N, [P] * N, opX=capi.OP_T, temp2=False, offs=offs)
            assert e == capi.SUCCESS, (dt, P, offs)
            for rec in launches:
                assert rec["in"] != rec["out"], (dt, P, offs, names, rec)
            if any(n.startswith("transpose_") for n in names):
                assert len(names) == 2, (dt, P, offs, names)
        # and the aligned call still gets the copy afterwards
        e, names, _ = plan(online_planner, "mkm", dt, M, [P] * N, [P] * N, opX=capi.OP_T, temp2=False)
        assert e == capi.SUCCESS and names[0].startswith("transpose_") and len(names) == 2, (dt, P, names)


def test_leaving_plan_only_mode_drops_its_stand_in_workspace():
    """Plan-only mode on a handle without a device uses a stand-in address for the merged-factor workspace; once the
    mode is left, a call must not plan on it (it would be handed to kernels): without a device and a workspace the
    chain is then not merged, and fastKronInitHIP allocates the real one."""
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.fastKronInit(ctypes.byref(h), capi.BACKEND_HIP) == capi.SUCCESS
    try:
        assert lib.fastKronSetPlanOnly(h, 1) == capi.SUCCESS
        e, names, _ = plan((lib, h), "mkm", "s", 1024, [4] * 8, [4] * 8)
        assert e == capi.SUCCESS and len(names) == 1 and "16x16" in names[0], names       # merged into 16x16^4
        assert lib.fastKronSetPlanOnly(h, 0) == capi.SUCCESS
        assert lib.fastKronSetPlanOnly(h, 1) == capi.SUCCESS
        e, names, _ = plan((lib, h), "mkm", "s", 1024, [4] * 8, [4] * 8)
        assert e == capi.SUCCESS and len(names) == 1 and "16x16" in names[0], names       # the stand-in is back, as before
    finally:
        lib.fastKronDestroy(h)


def test_transposition_rules_that_came_from_tuned_plans(online_planner):
    planner = online_planner
    copied = lambda names: names[0].startswith("transpose_")
    # a padded-step first launch on a 128-wide factor counts twice in the MKM layout, also with 16 rows ...
    e, names, _ = plan(planner, "mkm", "s", 16, [128] * 3, [128] * 3, opX=capi.OP_T)
    assert e == capi.SUCCESS and copied(names) and len(names) == 4, names
    # ... in the KMM layout only while X is at most 64 MB
    e, names, _ = plan(planner, "kmm", "s", 1024, [128] * 2, [128] * 2, opX=capi.OP_T)
    assert e == capi.SUCCESS and copied(names), names
    e, names, _ = plan(planner, "kmm", "s", 320, [128] * 3, [128] * 3, opX=capi.OP_T)
    assert e == capi.SUCCESS and not copied(names) and len(names) == 3, names
    # equal launch counts: the copy goes first, except in the KMM layout with fewer than 64 columns
    e, names, _ = plan(planner, "mkm", "d", 256, [16] * 4, [16] * 4, opX=capi.OP_T)
    assert e == capi.SUCCESS and copied(names), names
    e, names, _ = plan(planner, "kmm", "d", 16, [16] * 6, [16] * 6, opX=capi.OP_T)
    assert e == capi.SUCCESS and not copied(names), names


# ---- online rules for chains outside the specialised kernels ----
def test_lds_fused_groups_get_balanced_depth(online_planner):
    """The LDS-fused kernel taken as deep as it goes would leave a single plain launch (or two): the last two groups share
    the factors about equally instead."""
    planner = online_planner
    e, names, _ = plan(planner, "mkm", "s", 1024, [2] * 7, [4] * 7)
    assert e == capi.SUCCESS and len(names) == 2 and all("small_fused" in n for n in names), names
    e, names, _ = plan(planner, "kmm", "s", 1024, [3] * 7, [3] * 7)
    assert e == capi.SUCCESS and len(names) == 2 and all("small_fused" in n for n in names), names
    # a chain that one group holds stays one launch
    e, names, _ = plan(planner, "mkm", "s", 1024, [3] * 7, [3] * 7)
    assert e == capi.SUCCESS and len(names) == 1 and "small_fused" in names[0], names


def test_padded_step_rules_for_rectangular_and_large_odd_factors(online_planner):
    planner = online_planner
    # shrinking factors with 16 rows: padded matrix-core step, not the plain kernel
    for dt in ("s", "d"):
        e, names, _ = plan(planner, "mkm", dt, 1024, [16] * 5, [8] * 5)
        assert e == capi.SUCCESS and len(names) == 5 and all("anyxany" in n for n in names), names
    # fp64, KMM layout, more than 128 rows: plain kernel when the padded groups of four stay part empty
    e, names, _ = plan(planner, "kmm", "d", 1024, [129] * 2, [129] * 2)
    assert e == capi.SUCCESS and all("generic" in n for n in names), names
    e, names, _ = plan(planner, "kmm", "d", 1024, [255] * 2, [255] * 2)
    assert e == capi.SUCCESS and all("anyxany" in n for n in names), names
    e, names, _ = plan(planner, "kmm", "s", 1024, [200] * 2, [200] * 2)
    assert e == capi.SUCCESS and all("anyxany" in n for n in names), names


# ---- the plans that ship with the library (fastkron_amd/gfx950_plans.txt) ----
def _parse_key(key):
    """'MxK*(PxQ^N)_NN_f' / '(PxQ^N)*KxM_TT_d' (factor lists as 'AxB(x)CxD') -> (mm, dt, M, Ps, Qs, opX, opF)."""
    import re
    m = re.match(r"^(\d+)x(\d+)\*\((.*)\)_([NT])([NT])_([fd])$", key)
    if m:
        mm, M, facs, ox, of, dt = "mkm", int(m.group(1)), m.group(3), m.group(4), m.group(5), m.group(6)
    else:
        m = re.match(r"^\((.*)\)\*(\d+)x(\d+)_([NT])([NT])_([fd])$", key)
        assert m, key
        mm, M, facs, ox, of, dt = "kmm", int(m.group(3)), m.group(1), m.group(4), m.group(5), m.group(6)
    Ps, Qs = [], []
    for f in facs.split("(x)"):
        pq, _, n = f.partition("^")
        p, q = pq.split("x")
        Ps += [int(p)] * int(n or 1)
        Qs += [int(q)] * int(n or 1)
    op = {"N": capi.OP_N, "T": capi.OP_T}
    return mm, ("s" if dt == "f" else "d"), M, Ps, Qs, op[ox], op[of]


def _shipped_records():
    import os
    path = os.path.join(os.path.dirname(capi.LIB_PATH), "..", "gfx950_plans.txt")
    recs = []
    for line in open(path):
        if line.startswith("#") or not line.strip():
            continue
        tok = line.split()
        i = 2
        flags = {}
        while tok[i][0] in "MSX":
            flags[tok[i][0]] = int(tok[i][1:])
            i += 1
        n = int(tok[i])
        steps = [(int(tok[i + 1 + 3 * k]), int(tok[i + 2 + 3 * k]), tok[i + 3 + 3 * k]) for k in range(n)]
        recs.append((tok[0], flags, steps))
    return recs


def test_every_shipped_plan_is_what_a_default_handle_runs(planner):
    recs = _shipped_records()
    assert len(recs) >= 3
    for key, flags, steps in recs:
        if "stridedBatched" in key:
            continue
        mm, dt, M, Ps, Qs, opX, opF = _parse_key(key)
        e, names, launches = plan(planner, mm, dt, M, Ps, Qs, opX=opX, opF=opF)
        assert e == capi.SUCCESS, key
        want = [k for _, _, k in steps]
        got = [n for n in names if not n.startswith("transpose_")]
        assert got == want, (key, names, want)
        assert any(n.startswith("transpose_") for n in names) == bool(flags.get("X", 0)), (key, names)


def test_shipped_plans_can_be_switched_off(monkeypatch):
    """FASTKRON_SHIPPED_PLANS=0: a handle created then selects online, as if the file were not there."""
    import ctypes
    recs = [r for r in _shipped_records() if "stridedBatched" not in r[0]]
    monkeypatch.setenv("FASTKRON_SHIPPED_PLANS", "0")
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.fastKronInit(ctypes.byref(h), capi.BACKEND_HIP) == capi.SUCCESS
    assert lib.fastKronSetPlanOnly(h, 1) == capi.SUCCESS
    try:
        differ = 0
        for key, flags, steps in recs:
            mm, dt, M, Ps, Qs, opX, opF = _parse_key(key)
            e, names, _ = plan((lib, h), mm, dt, M, Ps, Qs, opX=opX, opF=opF)
            assert e == capi.SUCCESS
            got = [n for n in names if not n.startswith("transpose_")]
            differ += got != [k for _, _, k in steps] or any(n.startswith("transpose_") for n in names) != bool(flags.get("X", 0))
        assert differ == len(recs)          # every record is there because tuning beat the online plan
    finally:
        lib.fastKronDestroy(h)


# ---- non-temporal hints: what a launch is told about its input and output ----
def _hints(launches):
    return [(int(r["stream_in"]), int(r["stream_out"])) for r in launches]


def test_large_cold_operands_are_streamed(planner):
    """One launch over 134 MB in and out (sgemkm 1024 x 8^5): both hints; the same call on 256 rows: none."""
    e, names, launches = plan(planner, "mkm", "s", 1024, [8] * 5, [8] * 5)
    assert e == capi.SUCCESS and len(launches) == 1 and _hints(launches) == [(1, 1)]
    e, names, launches = plan(planner, "mkm", "s", 256, [8] * 5, [8] * 5)
    assert e == capi.SUCCESS and _hints(launches) == [(0, 0)]


def test_intermediates_that_fit_the_memory_side_cache_are_not_streamed(planner):
    """sgemkm 128 x 8^6 runs two launches around an intermediate of 134 MB: the first launch streams X in but stores
    ordinarily, the second loads ordinarily and streams Z out.  With 256 rows (268 MB) everything is streamed."""
    e, names, launches = plan(planner, "mkm", "s", 128, [8] * 6, [8] * 6)
    assert e == capi.SUCCESS and len(launches) == 2 and _hints(launches) == [(1, 0), (0, 1)]
    e, names, launches = plan(planner, "mkm", "s", 256, [8] * 6, [8] * 6)
    assert e == capi.SUCCESS and len(launches) == 2 and _hints(launches) == [(1, 1), (1, 1)]


def test_a_transposed_copy_is_not_streamed_back_in(planner):
    """op(X) = T behind a transposed copy: the copy (134 MB) was written a moment ago, so the launch that reads it
    loads ordinarily."""
    e, names, launches = plan(planner, "mkm", "s", 1024, [8] * 5, [8] * 5, opX=capi.OP_T, opF=capi.OP_T)
    assert e == capi.SUCCESS and names[0].startswith("transpose_") and len(launches) == 1
    assert _hints(launches) == [(0, 1)]


def test_two_part_plans_keep_their_intermediate_ordinary(planner):
    """sgemkm 16 x 16^6 (two-part plan, 1 GB per buffer): beyond the cache everything streams; 2 x 16^5 (8 MB): nothing."""
    e, names, launches = plan(planner, "mkm", "s", 2, [16] * 5, [16] * 5)
    assert e == capi.SUCCESS and all(h == (0, 0) for h in _hints(launches))
    e, names, launches = plan(planner, "mkm", "s", 32, [16] * 5, [16] * 5)     # 134 MB per buffer
    assert e == capi.SUCCESS and len(launches) >= 2
    hints = _hints(launches)
    assert hints[0][0] == 1 and hints[-1][1] == 1                  # X in and Z out are streamed
    assert all(h[1] == 0 for h in hints[:-1]) and all(h[0] == 0 for h in hints[1:])   # nothing in between is


def test_a_small_result_behind_a_large_input_is_streamed_out(planner):
    """8 x 512 x (32x16)^3 with Y: 537 MB of X, 67 MB of Z; the launch moves far more than the caches hold."""
    e, names, launches = plan(planner, "mkm", "s", 512, [32] * 3, [16] * 3, batch=8, beta=1.0, with_y=True)
    assert e == capi.SUCCESS and len(launches) == 1 and _hints(launches) == [(1, 1)]


# ---- a kernel that refuses the call's buffers is replaced by the next one in line ----
@pytest.mark.parametrize("which,expect", [("z", "_128x128_128x128_1_1x2048_mfma16x16x4_NN"), ("y", "_128x128_128x128_1_1x2048_mfma16x16x4_NN"),
                                          ("x", "anyxany")])
def test_a_refusing_kernel_is_replaced_by_the_next_in_line(planner, which, expect):
    """sgemkm 8 x 128^2: the wide step kernel needs X, Z and Y on 16-byte boundaries, the streaming step only X, the
    padded step nothing: an operand one element off moves the plan down that list, not to the plain kernel."""
    e, names, launches = plan(planner, "mkm", "s", 8, [128] * 2, [128] * 2, beta=0.5, with_y=True, offs={which: 4})
    assert e == capi.SUCCESS and len(launches) == 2
    assert all(expect in n for n in names), names
