"""GPU parity at the full sizes of the five benchmark configurations (and of three more shapes large enough for their
kernels' streaming stores), where the oracle cannot answer the whole problem in seconds.  Two checks per configuration, both against the oracle and both through the C ABI:

* sampled rows (MKM) / columns (KMM): every row of X is an independent chain, so the oracle's answer for a few
  rows taken out of the full problem must match the same rows of the full result (first, last, the rows next to
  workgroup boundaries, random ones);
* a checksum over every output element: Z = alpha * X (F1 x ... x FN) + beta * Y is linear in the rows, so the sum
  of all rows of Z equals the oracle's answer (in fp64) for the single row sum(X) with sum(Y) as Y.  A wrong
  element anywhere in Z, a row written twice or not at all, shows up here.
"""
import numpy as np
import pytest

from tests.gpu_util import TOL, normwise, run_gpu, seeded
from oracle import kron_oracle as ko

pytestmark = pytest.mark.gpu

@pytest.fixture(scope="module")
def fk():
    import fastkron_amd
    h = fastkron_amd.FastKron()
    yield h
    h.close()


FULL = [
    # name, mm, M, Ps, Qs, dtype, alpha, beta, batch        (bench.py's configurations)
    ("c1", ko.MKM, 1024, [8] * 5, [8] * 5, np.float32, 1.0, 0.0, 1),
    ("c2", ko.MKM, 1024, [16] * 4, [16] * 4, np.float32, 1.0, 0.0, 1),
    ("c3", ko.MKM, 256, [64] * 3, [64] * 3, np.float64, 1.0, 0.0, 1),
    ("c4", ko.KMM, 2048, [4] * 6, [4] * 6, np.float32, 1.5, 0.5, 1),
    ("c5", ko.MKM, 512, [32] * 3, [16] * 3, np.float32, 1.0, 1.0, 8),
    ("dgemkm 1024 x 8^5 (fp64 row kernel)", ko.MKM, 1024, [8] * 5, [8] * 5, np.float64, 1.5, 0.5, 1),
    # sizes at which three more kernels stream their results (system-scope 16-byte stores)
    ("16x16^3 on 8192 rows", ko.MKM, 8192, [16] * 3, [16] * 3, np.float32, 1.5, 0.5, 1),
    ("32x32^3 on 2048 rows", ko.MKM, 2048, [32] * 3, [32] * 3, np.float32, 1.0, 0.0, 1),
    ("KMM 32x32^3 on 1024 columns", ko.KMM, 1024, [32] * 3, [32] * 3, np.float32, 2.0, 0.0, 1),
]


def _rows(M, seed):
    rng = np.random.default_rng(seed)
    picks = {0, 1, M - 1, M - 2, M // 2, M // 2 - 1, 255 % M, 256 % M, 7 % M}
    picks.update(int(r) for r in rng.integers(0, M, size=4))
    return sorted(picks)


def _oracle(mm, M, Ps, Qs, X, Fs, Y, alpha, beta, dt):
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = np.ascontiguousarray(X, dtype=dt).reshape(1, -1)
    Fs = [np.ascontiguousarray(f, dtype=dt).reshape(1, -1) for f in Fs]
    Y = np.ascontiguousarray(Y, dtype=dt).reshape(1, -1) if Y is not None else None
    return ko.sliced_multiply(mm, M, Ps, Qs, X, Fs, alpha=alpha, beta=beta, Y=Y, batch=1, strideX=M * K,
                              strideF=[p * q for p, q in zip(Ps, Qs)], strideZ=M * L, strideY=M * L).reshape(-1)


@pytest.mark.parametrize("name,mm,M,Ps,Qs,dt,alpha,beta,batch", FULL, ids=[f[0] for f in FULL])
def test_full_size_configuration(fk, name, mm, M, Ps, Qs, dt, alpha, beta, batch):
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = seeded(11, (batch, M * K), dt)
    Fs = [seeded(12 + i, (batch, p * q), dt) for i, (p, q) in enumerate(zip(Ps, Qs))]
    Y = seeded(40, (batch, M * L), dt) if beta != 0 else None
    Z, e = run_gpu(fk, mm, M, Ps, Qs, X, Fs, Y, alpha, beta, batch=batch)
    assert e == 0
    assert not np.isnan(Z).any()
    Z = Z.reshape(batch, -1)
    picks = _rows(M, 5)
    for b in range(batch):
        fb = [f[b] for f in Fs]
        if mm == ko.MKM:            # element (m, k) at m*K + k
            x2, z2 = X[b].reshape(M, K), Z[b].reshape(M, L)
            y2 = Y[b].reshape(M, L) if Y is not None else None
            xs, zs, ys = x2[picks], z2[picks], (y2[picks] if y2 is not None else None)
            xsum, zsum = x2.sum(0, dtype=np.float64), z2.sum(0, dtype=np.float64)
            ysum = y2.sum(0, dtype=np.float64) if y2 is not None else None
        else:                       # X is K x M, Z is L x M: the chains are the columns
            x2, z2 = X[b].reshape(K, M), Z[b].reshape(L, M)
            y2 = Y[b].reshape(L, M) if Y is not None else None
            xs, zs, ys = x2[:, picks], z2[:, picks], (y2[:, picks] if y2 is not None else None)
            xsum, zsum = x2.sum(1, dtype=np.float64), z2.sum(1, dtype=np.float64)
            ysum = y2.sum(1, dtype=np.float64) if y2 is not None else None
        # sampled chains against the oracle in the call's own precision
        want = _oracle(mm, len(picks), Ps, Qs, xs, fb, ys, alpha, beta, dt)
        err = normwise(np.ascontiguousarray(zs).reshape(-1), want)
        assert err <= TOL[dt], f"batch {b}: sampled chains off by {err:.3e}"
        # checksum over all chains against the oracle in fp64
        want = _oracle(mm, 1, Ps, Qs, xsum, fb, ysum, alpha, beta, np.float64)
        err = normwise(zsum, want)
        assert err <= TOL[dt], f"batch {b}: checksum over all chains off by {err:.3e}"


@pytest.mark.parametrize("M,Ps,dt", [(1024, [8] * 5, np.float32), (16, [8] * 7, np.float32), (1024, [16] * 3, np.float64)])
def test_full_size_gekmm_with_transposed_x(fk, M, Ps, dt):
    """GeKMM with op(X) = T at sizes where the final transposition streams Z: sampled columns and the checksum over all
    columns against the oracle (X is stored M x K, Z and Y are L x M)."""
    from tests.gpu_util import oracle_answer
    K = int(np.prod(Ps))
    alpha, beta = 1.5, 0.5
    X = seeded(21, (M * K,), dt)
    Fs = [seeded(22 + i, (p * p,), dt) for i, p in enumerate(Ps)]
    Y = seeded(50, (K * M,), dt)
    Z, e = run_gpu(fk, ko.KMM, M, Ps, Ps, X, Fs, Y, alpha, beta, opX=ko.OP_T)
    assert e == 0 and not np.isnan(Z).any()
    assert fk.last_plan()[-1][2].endswith("_z"), fk.last_plan()
    x2, z2, y2 = X.reshape(M, K), Z.reshape(K, M), Y.reshape(K, M)
    picks = _rows(M, 6)
    want = oracle_answer(ko.KMM, len(picks), Ps, Ps, np.ascontiguousarray(x2[picks]), Fs, np.ascontiguousarray(y2[:, picks]),
                         alpha, beta, opX=ko.OP_T)
    err = normwise(np.ascontiguousarray(z2[:, picks]).reshape(-1), np.asarray(want).reshape(-1))
    assert err <= TOL[dt], f"sampled columns off by {err:.3e}"
    want = oracle_answer(ko.KMM, 1, Ps, Ps, x2.sum(0, dtype=np.float64), [f.astype(np.float64) for f in Fs],
                         y2.sum(1, dtype=np.float64), alpha, beta, opX=ko.OP_T)
    err = normwise(z2.sum(1, dtype=np.float64), np.asarray(want).reshape(-1))
    assert err <= TOL[dt], f"checksum over all columns off by {err:.3e}"


@pytest.mark.parametrize("mm,M,Ps,dt", [
    (ko.MKM, 2064, [16] * 5, np.float32),      # 2.16e9 elements: whole-block kernel on virtual rows + leading launch
    (ko.MKM, 1040, [3] * 13, np.float32),      # 1.66e9 elements through the LDS-fused kernel
    (ko.KMM, 4160, [64] * 3, np.float64),      # 1.09e9 doubles (8.7 GB per buffer) in the KMM layout
])
def test_element_offsets_beyond_32_bits(fk, mm, M, Ps, dt):
    """Buffers whose element or byte offsets do not fit 32 bits: operands are generated on the device, a few
    chains (the last ones included) are checked against the oracle."""
    import torch
    K = int(np.prod(Ps))
    tdt = torch.float32 if dt == np.float32 else torch.float64
    g = torch.Generator(device="cuda").manual_seed(5)
    X = torch.rand(M * K, device="cuda", dtype=tdt, generator=g) - 0.5
    Fs = [torch.rand(p * p, device="cuda", dtype=tdt, generator=g) - 0.5 for p in Ps]
    Z = torch.empty(M * K, device="cuda", dtype=tdt)
    t1, t2 = torch.empty_like(Z), torch.empty_like(Z)
    fn = fk.xgemkm if mm == ko.MKM else fk.xgekmm
    assert fn(M, Ps, Ps, X, Fs, Z, 1.0, 0.0, None, t1, t2) == 0
    torch.cuda.synchronize()
    picks = [0, 1, M // 2, M - 2, M - 1]
    if mm == ko.MKM:
        xs, zs = X.view(M, K)[picks].cpu().numpy(), Z.view(M, K)[picks].cpu().numpy()
    else:
        xs = X.view(K, M)[:, picks].contiguous().cpu().numpy()
        zs = Z.view(K, M)[:, picks].contiguous().cpu().numpy()
    del X, Z, t1, t2
    want = _oracle(mm, len(picks), Ps, Ps, xs, [f.cpu().numpy() for f in Fs], None, 1.0, 0.0, dt)
    err = normwise(np.ascontiguousarray(zs).reshape(-1), want)
    assert err <= TOL[dt], err
