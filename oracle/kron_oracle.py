"""ctypes front end of the CPU checker `libkronoracle.so` (built from kron_oracle.c by `make -C oracle`).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline leg of the
benchmark.  The shipped library never imports or calls it.

The functions mirror the argument meaning of the FastKron C API (reference include/fastkron.h:249-449):
`Ps`/`Qs` are the factor row/column counts, MKM factors are P x Q, KMM factors are Q x P, strides are in
elements with 0 meaning "shared by all batches".
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkronoracle.so")

MKM, KMM = 0, 1
OP_N, OP_T = 1, 2

_lib = None


def build():
    """Compile kron_oracle.c (plain gcc, a couple of seconds)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ko_flop.restype = ctypes.c_uint64
    return _lib


def _u32(a):
    return (ctypes.c_uint32 * len(a))(*[int(v) for v in a])


def _u64(a):
    return (ctypes.c_uint64 * len(a))(*[int(v) for v in a])


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def flop(M, Ps, Qs):
    return int(lib().ko_flop(ctypes.c_uint32(M), ctypes.c_uint32(len(Ps)), _u32(Ps), _u32(Qs)))


def gekmm_sizes(M, Ps, Qs):
    y, t = ctypes.c_size_t(0), ctypes.c_size_t(0)
    e = lib().ko_gekmm_sizes(ctypes.c_uint32(M), ctypes.c_uint32(len(Ps)), _u32(Ps), _u32(Qs),
                             ctypes.byref(y), ctypes.byref(t))
    assert e == 0
    return y.value, t.value


def gekmm_sizes_forward(M, Ps, Qs):
    n = len(Ps)
    y = ctypes.c_size_t(0)
    inter = (ctypes.c_size_t * max(n - 1, 1))()
    e = lib().ko_gekmm_sizes_forward(ctypes.c_uint32(M), ctypes.c_uint32(n), _u32(Ps), _u32(Qs),
                                     ctypes.byref(y), inter)
    assert e == 0
    return y.value, [inter[i] for i in range(n - 1)]


def kron_bruteforce(mmtype, M, Ps, Qs, X, Fs):
    """Defining sum in float64.  X: (M,K) for MKM or (K,M) for KMM; Fs[i]: (P,Q) for MKM or (Q,P) for KMM."""
    X = np.ascontiguousarray(X, dtype=np.float64)
    Fs = [np.ascontiguousarray(f, dtype=np.float64) for f in Fs]
    L = int(np.prod(Qs))
    Z = np.empty((M, L) if mmtype == MKM else (L, M), dtype=np.float64)
    fp = (ctypes.c_void_p * len(Fs))(*[f.ctypes.data for f in Fs])
    lib().ko_kron_bruteforce(ctypes.c_int(mmtype), ctypes.c_uint32(M), ctypes.c_uint32(len(Ps)),
                             _u32(Ps), _u32(Qs), _ptr(X), fp, _ptr(Z))
    return Z


def sliced_multiply(mmtype, M, Ps, Qs, X, Fs, alpha=1.0, beta=0.0, Y=None, opX=OP_N, opFs=OP_N,
                    batch=1, strideX=None, strideF=None, strideZ=None, strideY=None,
                    keep_intermediates=False):
    """Step-wise sliced multiply on flat buffers.

    X, Fs[i], Y are numpy arrays of float32 or float64 (any shape; they are used as flat buffers laid
    out exactly as the C API expects, including batches).  Returns Z as a flat array of batch*M*L
    elements (strideZ defaults to M*L), plus the list of N-1 flat intermediates when asked.
    """
    dt = X.dtype
    assert dt in (np.float32, np.float64)
    fn = lib().ko_sliced_multiply_f32 if dt == np.float32 else lib().ko_sliced_multiply_f64
    n = len(Ps)
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = np.ascontiguousarray(X).reshape(-1)
    Fs = [np.ascontiguousarray(f, dtype=dt).reshape(-1) for f in Fs]
    if Y is not None:
        Y = np.ascontiguousarray(Y, dtype=dt).reshape(-1)
    strideX = M * K if strideX is None else strideX
    strideZ = M * L if strideZ is None else strideZ
    strideY = M * L if strideY is None else strideY
    strideF = [int(Ps[i]) * int(Qs[i]) for i in range(n)] if strideF is None else list(strideF)
    Z = np.zeros(max(strideZ * (batch - 1) + M * L, 1), dtype=dt)
    fp = (ctypes.c_void_p * n)(*[f.ctypes.data for f in Fs])
    inters, ip, istr = [], None, None
    if keep_intermediates and n > 1:
        _, sizes = gekmm_sizes_forward(M, Ps, Qs)
        inters = [np.zeros(sz * batch, dtype=dt) for sz in sizes]
        ip = (ctypes.c_void_p * (n - 1))(*[a.ctypes.data for a in inters])
        istr = _u64(sizes)
    e = fn(ctypes.c_int(mmtype), ctypes.c_uint32(M), ctypes.c_uint32(n), _u32(Ps), _u32(Qs),
           _ptr(X), ctypes.c_int(opX), ctypes.c_uint64(strideX),
           fp, ctypes.c_int(opFs), _u64(strideF),
           _ptr(Z), ctypes.c_uint64(strideZ), ctypes.c_double(alpha), ctypes.c_double(beta),
           _ptr(Y), ctypes.c_uint64(strideY), ctypes.c_uint32(batch), ip, istr)
    assert e == 0, e
    if keep_intermediates:
        return Z, inters
    return Z


def sliced_multiply_fast(M, Ps, Qs, X, Fs, alpha=1.0, beta=0.0, Y=None, out=None):
    """MKM, opX = opF = N, one problem: the vectorised OpenMP variant timed as the CPU baseline."""
    dt = X.dtype
    assert dt in (np.float32, np.float64)
    fn = lib().ko_sliced_multiply_fast_f32 if dt == np.float32 else lib().ko_sliced_multiply_fast_f64
    sc = ctypes.c_float if dt == np.float32 else ctypes.c_double
    n = len(Ps)
    L = int(np.prod(Qs))
    X = np.ascontiguousarray(X).reshape(-1)
    Fs = [np.ascontiguousarray(f, dtype=dt).reshape(-1) for f in Fs]
    Z = np.empty(M * L, dtype=dt) if out is None else out
    fp = (ctypes.c_void_p * n)(*[f.ctypes.data for f in Fs])
    e = fn(ctypes.c_uint32(M), ctypes.c_uint32(n), _u32(Ps), _u32(Qs), _ptr(X), fp, _ptr(Z),
           sc(alpha), sc(beta), _ptr(Y))
    assert e == 0, e
    return Z
