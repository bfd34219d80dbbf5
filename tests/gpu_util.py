"""Helpers for the GPU parity tests: seeded inputs, a call through the C-ABI library, the oracle's
answer for the same buffers."""
import numpy as np

from oracle import kron_oracle as ko

TOL = {np.float32: 1e-5, np.float64: 1e-12}        # normwise bounds stated for fp32 / fp64 results


def seeded(seed, shape, dt, integer=False):
    rng = np.random.default_rng(seed)
    if integer:                                      # the reference's own tests fill with rand() % 3 + 1
        return rng.integers(1, 4, size=shape).astype(dt)
    return rng.uniform(-1.0, 1.0, size=shape).astype(dt)


def normwise(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    s = np.max(np.abs(b))
    return float(np.max(np.abs(a - b)) / (s if s > 0 else 1.0))


def make_case(mm, M, Ps, Qs, dt, seed=0, opX=ko.OP_N, opFs=ko.OP_N, batch=1, with_y=True, integer=False,
              share_f=False, share_y=False):
    """Flat host buffers laid out as the C API expects, batches included."""
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = seeded(seed, (batch, M * K), dt, integer)
    Fs = [seeded(seed + 1 + i, (1 if share_f else batch, p * q), dt, integer) for i, (p, q) in enumerate(zip(Ps, Qs))]
    Y = seeded(seed + 100, (1 if share_y else batch, M * L), dt, integer) if with_y else None
    return X, Fs, Y


def oracle_answer(mm, M, Ps, Qs, X, Fs, Y, alpha, beta, opX=ko.OP_N, opFs=ko.OP_N, batch=1,
                  share_f=False, share_y=False, keep_intermediates=False):
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    return ko.sliced_multiply(mm, M, Ps, Qs, X, Fs, alpha=alpha, beta=beta, Y=Y, opX=opX, opFs=opFs, batch=batch,
                              strideX=M * K, strideF=[0 if share_f else p * q for p, q in zip(Ps, Qs)],
                              strideZ=M * L, strideY=0 if share_y else M * L,
                              keep_intermediates=keep_intermediates)


def run_gpu(fk, mm, M, Ps, Qs, X, Fs, Y, alpha, beta, opX=ko.OP_N, opFs=ko.OP_N, batch=1,
            share_f=False, share_y=False, use_temp2=True, strided=None, poison=True, y_is_z=False):
    """Calls the library on device copies of the host buffers; returns Z as numpy and the error code.
    y_is_z: the call gets one buffer as Y and as Z (the in-place epilogue the API allows with two temporaries,
    reference include/fastkron.h:274-277)."""
    import torch
    from fastkron_amd import capi
    dev = "cuda:0"
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    tX = torch.from_numpy(X).to(dev)
    tFs = [torch.from_numpy(f).to(dev) for f in Fs]
    tY = torch.from_numpy(Y).to(dev) if Y is not None else None
    ye, te = fk.sizes(M, Ps, Qs)
    assert ye == M * L
    tdt = tX.dtype
    fill = float("nan") if poison else 0.0
    Z = torch.full((batch * max(ye, te if not use_temp2 else ye),), fill, dtype=tdt, device=dev)
    if y_is_z:
        assert tY is not None and not share_y and use_temp2
        Z[: batch * ye] = tY.reshape(-1)
        tY = Z
    t1 = torch.full((batch * te,), fill, dtype=tdt, device=dev)
    t2 = torch.full((batch * te,), fill, dtype=tdt, device=dev) if use_temp2 else None
    strided = (batch > 1) if strided is None else strided
    if strided:
        fn = fk.xgemkm_strided_batched if mm == ko.MKM else fk.xgekmm_strided_batched
        e = fn(M, Ps, Qs, tX, M * K, tFs, [0 if share_f else p * q for p, q in zip(Ps, Qs)], Z, M * L, batch,
               alpha, beta, tY, 0 if share_y else M * L, t1, t2, opX, opFs)
    else:
        fn = fk.xgemkm if mm == ko.MKM else fk.xgekmm
        e = fn(M, Ps, Qs, tX, tFs, Z, alpha, beta, tY, t1, t2, opX, opFs)
    torch.cuda.synchronize()
    return Z[: batch * M * L].cpu().numpy(), e


def chains_of(mm, M, cols, buf, transposed=False):
    """The operand as a (chains x cols) array: rows of an MKM operand, columns of a KMM one (op = T swaps the storage)."""
    row_major = (mm == ko.MKM) != transposed
    return buf.reshape(M, cols) if row_major else buf.reshape(cols, M).T


def sampled_check(fk, mm, M, Ps, Qs, dt, alpha=1.5, beta=0.5, opX=ko.OP_N, opFs=ko.OP_N, seed=11, picks=None,
                  y_is_z=False, use_temp2=True):
    """A problem too large for the oracle to answer whole: rows (MKM) / columns (KMM) are independent chains, so the
    oracle's answer for a few of them must match the same chains of the full result, and Z is linear in the chains,
    so the sum over all chains of Z must equal the oracle's fp64 answer for the single chain sum(X) (with sum(Y)):
    a checksum over every output element.  Returns the two normwise errors."""
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = seeded(seed, (1, M * K), dt)
    Fs = [seeded(seed + 1 + i, (1, p * q), dt) for i, (p, q) in enumerate(zip(Ps, Qs))]
    Y = seeded(seed + 29, (1, M * L), dt) if beta != 0 else None
    Z, e = run_gpu(fk, mm, M, Ps, Qs, X, Fs, Y, alpha, beta, opX=opX, opFs=opFs, y_is_z=y_is_z, use_temp2=use_temp2)
    assert e == 0, f"fastKronError {e}"
    assert not np.isnan(Z).any()
    if picks is None:
        rng = np.random.default_rng(seed)
        picks = sorted({0, 1, M - 1, M - 2, M // 2, M // 2 - 1, 255 % M, 256 % M, 7 % M} |
                       {int(r) for r in rng.integers(0, M, size=4)})
    xc = chains_of(mm, M, K, X[0], transposed=(opX == ko.OP_T))
    zc = chains_of(mm, M, L, Z)
    yc = chains_of(mm, M, L, Y[0]) if Y is not None else None

    def oracle(n, xs, ys, odt):
        # the sub-problem in the untransposed layout of its kind: n x K (MKM) or K x n (KMM)
        lay = (lambda a: np.ascontiguousarray(a)) if mm == ko.MKM else (lambda a: np.ascontiguousarray(a.T))
        out = ko.sliced_multiply(mm, n, Ps, Qs, lay(xs.astype(odt)).reshape(1, -1), [f.astype(odt) for f in Fs], alpha=alpha,
                                 beta=beta, Y=(lay(ys.astype(odt)).reshape(1, -1) if ys is not None else None), opX=ko.OP_N,
                                 opFs=opFs, batch=1, strideX=n * K, strideF=[p * q for p, q in zip(Ps, Qs)],
                                 strideZ=n * L, strideY=n * L).reshape(-1)
        return chains_of(mm, n, L, out)

    want = oracle(len(picks), xc[picks], yc[picks] if yc is not None else None, dt)
    err_rows = normwise(np.ascontiguousarray(zc[picks]), np.ascontiguousarray(want))
    want = oracle(1, xc.sum(0, dtype=np.float64)[None, :], yc.sum(0, dtype=np.float64)[None, :] if yc is not None else None,
                  np.float64)
    err_sum = normwise(zc.sum(0, dtype=np.float64), np.ascontiguousarray(want).reshape(-1))
    return err_rows, err_sum
