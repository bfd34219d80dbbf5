"""fastkron_amd -- MI355X (gfx950) Kronecker-matrix multiplication behind FastKron's C API.

The product is `lib/libFastKron.so` (C ABI, include/fastkron.h).  This package is the thin Python
side: `capi` holds the ctypes declarations, `FastKron` wraps a handle, and `torch_frontend` (`gemkm`,
`gekmm`, the autograd functions `MKM` / `KMM`) mirrors the PyTorch front end of the reference (reference
pyfastkron/fastkrontorch.py:340-465) for tensors that live in HBM.  PyTorch is used for device memory and streams only; all arithmetic happens in the
library's HIP kernels, and a missing library or a CPU tensor is an error, never a fallback.
"""
import ctypes

from . import capi
from .capi import (BACKEND_HIP, OP_N, OP_T, OPT_NONE, OPT_TUNE, OPT_USE_FUSION, SUCCESS)

__all__ = ["FastKron", "FastKronError", "gemkm", "gekmm", "MKM", "KMM", "capi"]


class FastKronError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        msg = capi.load().fastKronGetErrorString(code)
        super().__init__(f"{where}: fastKronError {code} ({msg.decode() if msg else 'unnamed'})")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


class FastKron:
    """One fastKronHandle bound to the HIP backend and a stream (reference pyfastkron/fastkronhandle.py:5-56)."""

    def __init__(self, stream=None, tune=False, fusion=True):
        import torch
        self.lib = capi.load()
        self.h = ctypes.c_void_p()
        e = self.lib.fastKronInit(ctypes.byref(self.h), BACKEND_HIP)
        if e != SUCCESS:
            raise FastKronError(e, "fastKronInit")
        opts = (OPT_USE_FUSION if fusion else OPT_NONE) | (OPT_TUNE if tune else 0)
        self.lib.fastKronSetOptions(self.h, opts)
        s = stream if stream is not None else torch.cuda.current_stream()
        self._stream = ctypes.c_void_p(s.cuda_stream)
        e = self.lib.fastKronInitHIP(self.h, ctypes.byref(self._stream))
        if e != SUCCESS:
            raise FastKronError(e, "fastKronInitHIP")

    def close(self):
        if self.h:
            self.lib.fastKronDestroy(self.h)
            self.h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_stream(self, stream):
        self._stream = ctypes.c_void_p(stream.cuda_stream)
        e = self.lib.fastKronSetStream(self.h, BACKEND_HIP, ctypes.byref(self._stream))
        if e != SUCCESS:
            raise FastKronError(e, "fastKronSetStream")

    def set_options(self, tune=False, fusion=True):
        self.lib.fastKronSetOptions(self.h, (OPT_USE_FUSION if fusion else OPT_NONE) | (OPT_TUNE if tune else 0))

    def sync_error(self):
        """Error word of the kernels that synchronise their workgroups (0: no wait ran out); cleared by the call."""
        w = ctypes.c_uint32(0)
        e = self.lib.fastKronGetSyncError(self.h, ctypes.byref(w))
        if e != 0:
            raise RuntimeError(f"fastKronGetSyncError: {e}")
        return w.value

    def last_plan(self):
        """[(lo, hi, kernel name), ...] of the most recent call, in launch order (include/fastkron_ext.h)."""
        buf = ctypes.create_string_buffer(4096)
        if self.lib.fastKronGetLastPlan(self.h, buf, 4096) == 0:
            return None
        parts = buf.value.decode().split(";")
        plan = []
        for p in parts[1:]:
            rng, name = p.split(":")
            lo, hi = rng.split("-")
            plan.append((int(lo), int(hi), name))
        return plan

    def set_tuned_db(self, path):
        self.lib.fastKronSetTunedDB(self.h, path.encode() if path else None)

    def sizes(self, M, Ps, Qs):
        y, t = ctypes.c_size_t(), ctypes.c_size_t()
        e = self.lib.gekmmSizes(self.h, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs),
                                ctypes.byref(y), ctypes.byref(t))
        if e != SUCCESS:
            raise FastKronError(e, "gekmmSizes")
        return y.value, t.value

    def sizes_forward(self, M, Ps, Qs):
        y = ctypes.c_size_t()
        inter = (ctypes.c_size_t * max(len(Ps) - 1, 1))()
        e = self.lib.gekmmSizesForward(self.h, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs),
                                       ctypes.byref(y), inter)
        if e != SUCCESS:
            raise FastKronError(e, "gekmmSizesForward")
        return y.value, [inter[i] for i in range(len(Ps) - 1)]

    # ---- raw calls: tensors are used as flat HBM buffers, exactly as the C API sees them ----
    def _prefix(self, dtype):
        import torch
        if dtype == torch.float32:
            return "s", ctypes.c_float
        if dtype == torch.float64:
            return "d", ctypes.c_double
        raise TypeError(f"unsupported dtype {dtype}")

    def xgemkm(self, M, Ps, Qs, X, Fs, Z, alpha=1.0, beta=0.0, Y=None, temp1=None, temp2=None,
               opX=OP_N, opFs=OP_N, backend=BACKEND_HIP):
        pre, sc = self._prefix(X.dtype)
        fn = getattr(self.lib, pre + "gemkm")
        return fn(self.h, backend, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs), _ptr(X), opX,
                  capi.arr_ptr([f.data_ptr() for f in Fs]), opFs, _ptr(Z), sc(alpha), sc(beta),
                  _ptr(Y), _ptr(temp1), _ptr(temp2))

    def xgemkm_static_scratch(self, M, Ps, Qs, X, Fs, Z, alpha=1.0, beta=0.0, Y=None, opX=OP_N, opFs=OP_N,
                              backend=BACKEND_HIP):
        """sgemkm without temporaries: they come from the library's static device array; allocates nothing."""
        return self.lib.sgemkmStaticScratch(self.h, backend, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs), _ptr(X), opX,
                                            capi.arr_ptr([f.data_ptr() for f in Fs]), opFs, _ptr(Z),
                                            ctypes.c_float(alpha), ctypes.c_float(beta), _ptr(Y))

    def xgekmm(self, M, Ps, Qs, X, Fs, Z, alpha=1.0, beta=0.0, Y=None, temp1=None, temp2=None,
               opX=OP_N, opFs=OP_N, backend=BACKEND_HIP):
        pre, sc = self._prefix(X.dtype)
        fn = getattr(self.lib, pre + "gekmm")
        return fn(self.h, backend, len(Ps), capi.arr_u32(Qs), capi.arr_u32(Ps), M,
                  capi.arr_ptr([f.data_ptr() for f in Fs]), opFs, _ptr(X), opX, _ptr(Z), sc(alpha), sc(beta),
                  _ptr(Y), _ptr(temp1), _ptr(temp2))

    def xgemkm_strided_batched(self, M, Ps, Qs, X, strideX, Fs, strideF, Z, strideZ, batch, alpha=1.0,
                               beta=0.0, Y=None, strideY=0, temp1=None, temp2=None, opX=OP_N, opFs=OP_N,
                               backend=BACKEND_HIP):
        pre, sc = self._prefix(X.dtype)
        fn = getattr(self.lib, pre + "gemkmStridedBatched")
        return fn(self.h, backend, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs), _ptr(X), opX, strideX,
                  capi.arr_ptr([f.data_ptr() for f in Fs]), opFs, capi.arr_u64(strideF), _ptr(Z), strideZ,
                  sc(alpha), sc(beta), batch, _ptr(Y), strideY, _ptr(temp1), _ptr(temp2))

    def xgekmm_strided_batched(self, M, Ps, Qs, X, strideX, Fs, strideF, Z, strideZ, batch, alpha=1.0,
                               beta=0.0, Y=None, strideY=0, temp1=None, temp2=None, opX=OP_N, opFs=OP_N,
                               backend=BACKEND_HIP):
        pre, sc = self._prefix(X.dtype)
        fn = getattr(self.lib, pre + "gekmmStridedBatched")
        return fn(self.h, backend, len(Ps), capi.arr_u32(Qs), capi.arr_u32(Ps), M,
                  capi.arr_ptr([f.data_ptr() for f in Fs]), opFs, capi.arr_u64(strideF), _ptr(X), opX, strideX,
                  _ptr(Z), strideZ, sc(alpha), sc(beta), batch, _ptr(Y), strideY, _ptr(temp1), _ptr(temp2))

    def prepared(self, call, *args, **kwargs):
        """Marshal the arguments of one raw call once and return a zero-argument callable that repeats
        it (what a C caller does when it calls the same problem in a loop).  `call` is the name of one
        of the x* methods above, e.g. "xgemkm"."""
        captured = {}
        real = self.lib

        class _Capture:
            def __getattr__(_, name):
                def grab(*a):
                    captured["fn"], captured["args"] = getattr(real, name), a
                    return SUCCESS
                return grab

        self.lib = _Capture()
        try:
            getattr(self, call)(*args, **kwargs)
        finally:
            self.lib = real
        fn, a = captured["fn"], captured["args"]
        return lambda: fn(*a)

    def xforward(self, mmtype, M, Ps, Qs, X, Fs, Z, inters, opX=OP_N, opFs=OP_N, backend=BACKEND_HIP):
        pre, _ = self._prefix(X.dtype)
        ip = capi.arr_ptr([t.data_ptr() for t in inters]) if inters else None
        fp = capi.arr_ptr([f.data_ptr() for f in Fs])
        if mmtype == "mkm":
            return getattr(self.lib, pre + "mkmForward")(self.h, backend, M, len(Ps), capi.arr_u32(Ps),
                                                         capi.arr_u32(Qs), _ptr(X), opX, fp, opFs, _ptr(Z), ip)
        return getattr(self.lib, pre + "kmmForward")(self.h, backend, len(Ps), capi.arr_u32(Qs), capi.arr_u32(Ps),
                                                     M, fp, opFs, _ptr(X), opX, _ptr(Z), ip)


_default = None


def default_handle():
    global _default
    if _default is None:
        _default = FastKron()
    return _default


def __getattr__(name):
    # gemkm / gekmm / MKM / KMM live in torch_frontend; importing them lazily keeps `import fastkron_amd`
    # usable by hosts that only want the ctypes declarations
    if name in ("gemkm", "gekmm", "MKM", "KMM"):
        from . import torch_frontend
        return getattr(torch_frontend, name)
    raise AttributeError(f"module 'fastkron_amd' has no attribute '{name}'")
