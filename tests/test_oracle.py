"""Pins oracle/kron_oracle.c without re-typing its formula: numpy.kron + matmul, the brute-force
defining sum, closed forms, and the sizes the reference library itself returned."""
import numpy as np
import pytest

from oracle import kron_oracle as ko
from tests.kron_ref import (kmm_dense, kmm_intermediate_dense, mkm_dense, mkm_intermediate_dense, normwise)

SHAPES = [
    # (M, Ps, Qs)
    (3, [4], [5]),
    (2, [2, 3], [3, 2]),
    (4, [8, 8], [8, 8]),
    (5, [4, 4, 4], [4, 4, 4]),
    (3, [2, 3, 5], [4, 1, 2]),          # Q = 1 factor (reference general-tests-NN.cpp:79-80 style)
    (2, [1, 4], [4, 2]),                # P = 1 factor
    (3, [5, 2, 6], [2, 5, 4]),          # distinct shapes, reference general-tests-NN.cpp:102-166
    (2, [32, 32], [16, 16]),            # non-square 32x16 (config-5 factor shape)
    (1, [3, 3, 3, 3], [2, 2, 2, 2]),
]


def rand(rng, shape, dt):
    return rng.uniform(-1, 1, size=shape).astype(dt)


@pytest.mark.parametrize("M,Ps,Qs", SHAPES)
@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float64, 1e-14)])
def test_mkm_matches_numpy_kron(M, Ps, Qs, dt, tol):
    rng = np.random.default_rng(1)
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = rand(rng, (M, K), dt)
    Fs = [rand(rng, (p, q), dt) for p, q in zip(Ps, Qs)]
    Y = rand(rng, (M, L), dt)
    Z = ko.sliced_multiply(ko.MKM, M, Ps, Qs, X, Fs, alpha=1.5, beta=-0.5, Y=Y).reshape(M, L)
    assert normwise(Z, mkm_dense(X, Fs, 1.5, -0.5, Y)) < tol


@pytest.mark.parametrize("M,Ps,Qs", SHAPES)
@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float64, 1e-14)])
def test_kmm_matches_numpy_kron(M, Ps, Qs, dt, tol):
    rng = np.random.default_rng(2)
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = rand(rng, (K, M), dt)
    Fs = [rand(rng, (q, p), dt) for p, q in zip(Ps, Qs)]      # KMM factors are Q x P
    Y = rand(rng, (L, M), dt)
    Z = ko.sliced_multiply(ko.KMM, M, Ps, Qs, X, Fs, alpha=2.0, beta=1.0, Y=Y).reshape(L, M)
    assert normwise(Z, kmm_dense(X, Fs, 2.0, 1.0, Y)) < tol


@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
@pytest.mark.parametrize("opX", [ko.OP_N, ko.OP_T])
@pytest.mark.parametrize("opF", [ko.OP_N, ko.OP_T])
def test_transposed_operands(mm, opX, opF):
    """opX/opF = T: the buffer holds the transpose of the operand (reference tests/testBase.h:264-306)."""
    rng = np.random.default_rng(3)
    M, Ps, Qs = 3, [2, 4, 3], [3, 2, 4]
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    dt = np.float64
    if mm == ko.MKM:
        opXm = rand(rng, (M, K), dt)
        opFs = [rand(rng, (p, q), dt) for p, q in zip(Ps, Qs)]
        want = mkm_dense(opXm, opFs)
    else:
        opXm = rand(rng, (K, M), dt)
        opFs = [rand(rng, (q, p), dt) for p, q in zip(Ps, Qs)]
        want = kmm_dense(opXm, opFs)
    Xbuf = opXm if opX == ko.OP_N else np.ascontiguousarray(opXm.T)
    Fbufs = [f if opF == ko.OP_N else np.ascontiguousarray(f.T) for f in opFs]
    Z = ko.sliced_multiply(mm, M, Ps, Qs, Xbuf, Fbufs, opX=opX, opFs=opF).reshape(want.shape)
    assert normwise(Z, want) < 1e-14


@pytest.mark.parametrize("mm", [ko.MKM, ko.KMM])
def test_bruteforce_agrees_with_numpy_and_steps(mm):
    rng = np.random.default_rng(4)
    M, Ps, Qs = 2, [3, 2, 4], [2, 3, 2]
    K = int(np.prod(Ps))
    if mm == ko.MKM:
        X = rand(rng, (M, K), np.float64)
        Fs = [rand(rng, (p, q), np.float64) for p, q in zip(Ps, Qs)]
        want = mkm_dense(X, Fs)
    else:
        X = rand(rng, (K, M), np.float64)
        Fs = [rand(rng, (q, p), np.float64) for p, q in zip(Ps, Qs)]
        want = kmm_dense(X, Fs)
    brute = ko.kron_bruteforce(mm, M, Ps, Qs, X, Fs)
    assert normwise(brute, want) < 1e-14
    steps = ko.sliced_multiply(mm, M, Ps, Qs, X, Fs).reshape(want.shape)
    assert normwise(steps, brute) < 1e-14


def test_closed_forms():
    rng = np.random.default_rng(5)
    # N = 1 is a plain GEMM
    X = rand(rng, (7, 6), np.float64)
    F = rand(rng, (6, 9), np.float64)
    Z = ko.sliced_multiply(ko.MKM, 7, [6], [9], X, [F]).reshape(7, 9)
    assert normwise(Z, X @ F) < 1e-15
    # identity factors: Z = alpha X + beta Y
    Ps = [4, 2, 3]
    K = 24
    X = rand(rng, (5, K), np.float64)
    Y = rand(rng, (5, K), np.float64)
    Z = ko.sliced_multiply(ko.MKM, 5, Ps, Ps, X, [np.eye(p) for p in Ps], alpha=3.0, beta=0.25, Y=Y)
    assert normwise(Z.reshape(5, K), 3.0 * X + 0.25 * Y) < 1e-15
    # all-ones inputs: every entry is alpha * prod(P) + beta
    Ps, Qs = [8, 8, 8], [4, 8, 2]
    X = np.ones((2, 512), np.float32)
    Fs = [np.ones((p, q), np.float32) for p, q in zip(Ps, Qs)]
    Y = np.ones((2, 64), np.float32)
    Z = ko.sliced_multiply(ko.MKM, 2, Ps, Qs, X, Fs, alpha=2.0, beta=1.0, Y=Y)
    assert np.all(Z == 2.0 * 512 + 1.0)
    # KMM with M = 1 equals MKM on the same vector (reference src/handle/handle.cpp:134-138)
    Ps, Qs = [3, 4], [2, 5]
    x = rand(rng, (12,), np.float64)
    Fk = [rand(rng, (q, p), np.float64) for p, q in zip(Ps, Qs)]
    zk = ko.sliced_multiply(ko.KMM, 1, Ps, Qs, x.reshape(12, 1), Fk)
    zm = ko.sliced_multiply(ko.MKM, 1, Ps, Qs, x.reshape(1, 12), Fk, opFs=ko.OP_T)
    assert normwise(zk, zm) < 1e-15


def test_mixed_product_property():
    """(F1 (x) F2)(G1 (x) G2) = F1 G1 (x) F2 G2: two chained calls equal one call on the products."""
    rng = np.random.default_rng(6)
    M = 3
    F = [rand(rng, (4, 3), np.float64), rand(rng, (2, 5), np.float64)]
    G = [rand(rng, (3, 2), np.float64), rand(rng, (5, 4), np.float64)]
    X = rand(rng, (M, 8), np.float64)
    t = ko.sliced_multiply(ko.MKM, M, [4, 2], [3, 5], X, F)
    two = ko.sliced_multiply(ko.MKM, M, [3, 5], [2, 4], t, G)
    one = ko.sliced_multiply(ko.MKM, M, [4, 2], [2, 4], X, [F[0] @ G[0], F[1] @ G[1]])
    assert normwise(two, one) < 1e-14


def test_strided_batches_and_broadcast():
    rng = np.random.default_rng(7)
    M, Ps, Qs, B = 3, [4, 2], [2, 3], 4
    K, L = 8, 6
    X = rand(rng, (B, M, K), np.float64)
    Fs = [rand(rng, (B, p, q), np.float64) for p, q in zip(Ps, Qs)]
    Y = rand(rng, (B, M, L), np.float64)
    Z = ko.sliced_multiply(ko.MKM, M, Ps, Qs, X, Fs, alpha=1.0, beta=1.0, Y=Y, batch=B).reshape(B, M, L)
    for b in range(B):
        assert normwise(Z[b], mkm_dense(X[b], [f[b] for f in Fs], 1.0, 1.0, Y[b])) < 1e-14
    # stride 0 on the factors and on Y: shared by every batch
    Zs = ko.sliced_multiply(ko.MKM, M, Ps, Qs, X, [f[0] for f in Fs], alpha=1.0, beta=2.0, Y=Y[0],
                            batch=B, strideF=[0, 0], strideY=0).reshape(B, M, L)
    for b in range(B):
        assert normwise(Zs[b], mkm_dense(X[b], [f[0] for f in Fs], 1.0, 2.0, Y[0])) < 1e-14


def test_kmm_strided_batches_and_broadcast():
    """GeKMM batches: X is K x M per entry, factors Q x P, every entry against numpy.kron of its own factors."""
    rng = np.random.default_rng(17)
    M, Ps, Qs, B = 5, [4, 2, 3], [2, 3, 2], 3
    K, L = 24, 12
    X = rand(rng, (B, K, M), np.float64)
    Fs = [rand(rng, (B, q, p), np.float64) for p, q in zip(Ps, Qs)]
    Y = rand(rng, (B, L, M), np.float64)
    Z = ko.sliced_multiply(ko.KMM, M, Ps, Qs, X, Fs, alpha=1.5, beta=0.5, Y=Y, batch=B).reshape(B, L, M)
    for b in range(B):
        assert normwise(Z[b], kmm_dense(X[b], [f[b] for f in Fs], 1.5, 0.5, Y[b])) < 1e-14
    # shared factors, shared Y, and X shared against per-entry factors
    Zs = ko.sliced_multiply(ko.KMM, M, Ps, Qs, X, [f[0] for f in Fs], alpha=1.0, beta=2.0, Y=Y[0], batch=B,
                            strideF=[0, 0, 0], strideY=0).reshape(B, L, M)
    for b in range(B):
        assert normwise(Zs[b], kmm_dense(X[b], [f[0] for f in Fs], 1.0, 2.0, Y[0])) < 1e-14
    Zx = ko.sliced_multiply(ko.KMM, M, Ps, Qs, X[0], Fs, batch=B, strideX=0).reshape(B, L, M)
    for b in range(B):
        assert normwise(Zx[b], kmm_dense(X[0], [f[b] for f in Fs])) < 1e-14
    # opX = T: the buffer of an entry is M x K
    Xt = np.ascontiguousarray(X.transpose(0, 2, 1))
    Zt = ko.sliced_multiply(ko.KMM, M, Ps, Qs, Xt, Fs, batch=B, opX=ko.OP_T).reshape(B, L, M)
    for b in range(B):
        assert normwise(Zt[b], kmm_dense(X[b], [f[b] for f in Fs])) < 1e-14


def test_kmm_forward_intermediates_layout():
    rng = np.random.default_rng(18)
    M, Ps, Qs = 3, [3, 4, 2], [2, 3, 5]
    X = rand(rng, (24, M), np.float64)
    Fs = [rand(rng, (q, p), np.float64) for p, q in zip(Ps, Qs)]
    Z, inter = ko.sliced_multiply(ko.KMM, M, Ps, Qs, X, Fs, keep_intermediates=True)
    assert normwise(Z.reshape(-1, M), kmm_dense(X, Fs)) < 1e-14
    for j in (1, 2):   # Intermediates[j-1] is the output of the step multiplying factor j
        assert normwise(inter[j - 1].reshape(-1, M), kmm_intermediate_dense(X, Fs, j)) < 1e-14
    # batched: every entry keeps its own intermediates, entry after entry
    B = 2
    Xb = rand(rng, (B, 24, M), np.float64)
    Fb = [rand(rng, (B, q, p), np.float64) for p, q in zip(Ps, Qs)]
    Zb, interb = ko.sliced_multiply(ko.KMM, M, Ps, Qs, Xb, Fb, batch=B, keep_intermediates=True)
    for b in range(B):
        fsb = [f[b] for f in Fb]
        assert normwise(Zb.reshape(B, -1, M)[b], kmm_dense(Xb[b], fsb)) < 1e-14
        for j in (1, 2):
            assert normwise(interb[j - 1].reshape(B, -1, M)[b], kmm_intermediate_dense(Xb[b], fsb, j)) < 1e-14


def test_forward_intermediates_layout():
    rng = np.random.default_rng(8)
    M, Ps, Qs = 2, [3, 4, 2], [2, 3, 5]
    X = rand(rng, (M, 24), np.float64)
    Fs = [rand(rng, (p, q), np.float64) for p, q in zip(Ps, Qs)]
    Z, inter = ko.sliced_multiply(ko.MKM, M, Ps, Qs, X, Fs, keep_intermediates=True)
    y, sizes = ko.gekmm_sizes_forward(M, Ps, Qs)
    assert y == M * 30 and sizes == [M * 3 * 3 * 5, M * 3 * 4 * 5]
    assert normwise(Z.reshape(M, -1), mkm_dense(X, Fs)) < 1e-14
    for j in (1, 2):   # Intermediates[j-1] is the output of the step multiplying factor j
        assert normwise(inter[j - 1].reshape(M, -1), mkm_intermediate_dense(X, Fs, j)) < 1e-14


def test_sizes_match_values_returned_by_the_reference_library():
    # yElems / tmpElems the reference x86 build returned for the benchmark configurations
    assert ko.gekmm_sizes(1024, [8] * 5, [8] * 5) == (33554432, 33554432)
    assert ko.gekmm_sizes(1024, [16] * 4, [16] * 4) == (67108864, 67108864)
    assert ko.gekmm_sizes(256, [64] * 3, [64] * 3) == (67108864, 67108864)
    assert ko.gekmm_sizes(2048, [4] * 6, [4] * 6) == (8388608, 8388608)
    assert ko.gekmm_sizes(512, [32] * 3, [16] * 3) == (2097152, 8388608)
    assert ko.gekmm_sizes(4, [8, 8], [32, 32]) == (4096, 4096)      # growing chain
    assert ko.gekmm_sizes(4, [8], [32]) == (128, 128)               # N = 1: M * max(K, L)
    assert ko.gekmm_sizes(4, [32], [8]) == (32, 128)


def test_flop_counts_of_the_benchmark_configurations():
    assert ko.flop(1024, [8] * 5, [8] * 5) == 2684354560
    assert ko.flop(1024, [16] * 4, [16] * 4) == 8589934592
    assert ko.flop(256, [64] * 3, [64] * 3) == 25769803776
    assert ko.flop(2048, [4] * 6, [4] * 6) == 402653184
    assert 8 * ko.flop(512, [32] * 3, [16] * 3) == 7516192768


@pytest.mark.parametrize("dt,tol", [(np.float32, 5e-6), (np.float64, 1e-13)])
def test_fast_variant_matches_numpy(dt, tol):
    rng = np.random.default_rng(9)
    for M, Ps, Qs in [(5, [8, 8, 8], [8, 8, 8]), (3, [32, 32], [16, 16]), (2, [3, 5, 2], [4, 2, 3]),
                      (2, [16, 16, 16], [16, 16, 16])]:
        K, L = int(np.prod(Ps)), int(np.prod(Qs))
        X = rand(rng, (M, K), dt)
        Fs = [rand(rng, (p, q), dt) for p, q in zip(Ps, Qs)]
        Y = rand(rng, (M, L), dt)
        Z = ko.sliced_multiply_fast(M, Ps, Qs, X, Fs, 1.25, 0.5, Y).reshape(M, L)
        assert normwise(Z, mkm_dense(X, Fs, 1.25, 0.5, Y)) < tol
