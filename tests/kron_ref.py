"""Independent numpy statements of the Kronecker product results used to pin the oracle.

Nothing here shares code with oracle/kron_oracle.c: results are built from numpy.kron + matmul, the
construction the reference's own python tests use (reference tests/python/test_torch.py:15-38).
"""
import functools

import numpy as np


def kron_chain(mats):
    return functools.reduce(np.kron, mats)


def mkm_dense(X, Fs, alpha=1.0, beta=0.0, Y=None):
    """X (M,K); Fs[i] (P_i,Q_i) -> alpha * X @ (F1 (x) ... (x) FN) + beta * Y, float64."""
    Z = alpha * (np.asarray(X, np.float64) @ kron_chain([np.asarray(f, np.float64) for f in Fs]))
    if Y is not None:
        Z = Z + beta * np.asarray(Y, np.float64)
    return Z


def kmm_dense(X, Fs, alpha=1.0, beta=0.0, Y=None):
    """X (K,M); Fs[i] (Q_i,P_i) -> alpha * (F1 (x) ... (x) FN) @ X + beta * Y, float64."""
    Z = alpha * (kron_chain([np.asarray(f, np.float64) for f in Fs]) @ np.asarray(X, np.float64))
    if Y is not None:
        Z = Z + beta * np.asarray(Y, np.float64)
    return Z


def mkm_intermediate_dense(X, Fs, j):
    """Output of the step that multiplies factor j (0-based) in the rotated layout the steps use:
    columns ordered (q_j .. q_{N-1}, k_0 .. k_{j-1}).  Built from a Kronecker product with identities
    for the factors not yet applied, followed by an explicit axis swap."""
    X = np.asarray(X, np.float64)
    M = X.shape[0]
    mats = [np.eye(f.shape[0]) for f in Fs[:j]] + [np.asarray(f, np.float64) for f in Fs[j:]]
    R = X @ kron_chain(mats)
    kpre = int(np.prod([f.shape[0] for f in Fs[:j]])) if j > 0 else 1
    lsuf = int(np.prod([f.shape[1] for f in Fs[j:]]))
    return R.reshape(M, kpre, lsuf).swapaxes(1, 2).reshape(M, kpre * lsuf)


def kmm_intermediate_dense(X, Fs, j):
    """KMM counterpart: X (K, M), Fs[i] (Q_i, P_i); rows of the result ordered (q_j .. q_{N-1}, k_0 .. k_{j-1}).
    Identities stand in for the factors not yet applied; the row blocks are then swapped explicitly."""
    X = np.asarray(X, np.float64)
    M = X.shape[1]
    mats = [np.eye(f.shape[1]) for f in Fs[:j]] + [np.asarray(f, np.float64) for f in Fs[j:]]
    R = kron_chain(mats) @ X
    kpre = int(np.prod([f.shape[1] for f in Fs[:j]])) if j > 0 else 1
    lsuf = int(np.prod([f.shape[0] for f in Fs[j:]]))
    return R.reshape(kpre, lsuf, M).swapaxes(0, 1).reshape(kpre * lsuf, M)


def normwise(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    d = np.max(np.abs(a - b)) if a.size else 0.0
    s = np.max(np.abs(b)) if b.size else 1.0
    return d / (s if s > 0 else 1.0)


def eq_val(x, y, tol=1e-5):
    """The element-wise rule of the reference's own harness (reference tests/testBase.h:136-146)."""
    x = np.asarray(x, np.float64).reshape(-1)
    y = np.asarray(y, np.float64).reshape(-1)
    small = (np.abs(x) <= tol) & (np.abs(y) <= tol)
    den = np.where(np.abs(y) <= tol, x, y)
    den = np.where(den == 0, 1.0, den)
    rel = np.abs((x - y) / den) <= tol
    return bool(np.all(small | rel))
