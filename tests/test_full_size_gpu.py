"""GPU parity at the full sizes of the five benchmark configurations, where the oracle cannot answer the whole
problem in seconds.  Two checks per configuration, both against the oracle and both through the C ABI:

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
