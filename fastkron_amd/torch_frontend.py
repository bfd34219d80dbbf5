"""PyTorch front end over libFastKron.so for tensors that live in HBM.

Mirrors the reference's `pyfastkron` interface (reference pyfastkron/fastkrontorch.py:404-465 `gemkm` /
`gekmm`, :340-401 the autograd functions `MKM` / `KMM`, pyfastkron/fastkronbase.py:104-518 the shape,
broadcast and batching rules):

* operands may carry leading batch dimensions, broadcast between X, the factors and Y the NumPy way; the
  innermost batch dimension becomes one strided-batched library call (stride 0 = shared operand), outer
  ones a host loop; a batch of X against shared factors (MKM) is folded into the row count instead;
* a tensor whose last two dimensions are a transposed view of a row-major buffer is passed as that buffer
  with `fastKronOp_T` instead of being copied (reference fastkrontorch.py:66-76);
* 1-D X is a single row (MKM) or column (KMM);
* with gradients required, the forward family of the library keeps every step's output and `backward`
  chains through the saved intermediates (reference fastkrontorch.py:160-217); when only X needs a gradient
  the backward pass is one fused library call with the transposed factors.

PyTorch supplies memory, streams and, in `backward` for factor gradients, the per-step GEMMs (as in the
reference); the forward arithmetic is always the library's HIP kernels.  CPU tensors and dtypes other than
float32 / float64 are errors: there is no fallback path (the reference falls back to a shuffle algorithm
built from `torch.matmul`, fastkronbase.py:478-518).
"""
import ctypes
import math

import torch

from . import capi
from .capi import BACKEND_HIP, OP_N, OP_T, SUCCESS

__all__ = ["gemkm", "gekmm", "MKM", "KMM"]


def _prod(v):
    return int(math.prod(v)) if len(v) else 1


def _operand(t, force_contiguous=False):
    """(op, buffer): `buffer` is contiguous; op T says the last two dims of `t` are the buffer's, swapped."""
    if force_contiguous or t.is_contiguous():
        return OP_N, t.contiguous()
    if t.ndim >= 2 and t.mT.is_contiguous():
        return OP_T, t.mT
    return OP_N, t.contiguous()


def _validate(mm, x, fs, y):
    if not isinstance(x, torch.Tensor):
        raise ValueError("Input 'x' should be a Tensor")
    if not isinstance(fs, (list, tuple)) or len(fs) == 0:
        raise ValueError("Input 'fs' should be a list of Tensor")
    for i, f in enumerate(fs):
        if not isinstance(f, torch.Tensor):
            raise ValueError(f"Input fs[{i}] should be a Tensor")
        if f.ndim < 2:
            raise ValueError(f"Input fs[{i}] should have at least two dimensions")
    if y is not None and not isinstance(y, torch.Tensor):
        raise ValueError("Input 'y' should be a Tensor")
    tensors = [x] + list(fs) + ([y] if y is not None else [])
    devices = {t.device for t in tensors}
    if len(devices) != 1:
        raise RuntimeError(f"Expected all tensors to be on the same device, but found {sorted(str(d) for d in devices)}")
    if not x.is_cuda:
        raise RuntimeError("fastkron_amd runs on HBM-resident tensors only: there is no CPU path")
    if x.dtype not in (torch.float32, torch.float64):
        raise TypeError(f"float32 and float64 only, got {x.dtype}")
    if any(t.dtype != x.dtype for t in tensors):
        raise ValueError(f"Operand types mismatch: {[t.dtype for t in tensors]}")
    for f in fs[1:]:
        if f.shape[:-2] != fs[0].shape[:-2]:
            raise ValueError(f"Batched dims of factors do not match: {fs[0].shape[:-2]} != {f.shape[:-2]}")


class _Problem:
    """Shapes, ops and contiguous buffers of one call; logical shapes are X (.., M, K) for MKM and
    (.., K, M) for KMM, factors (.., P, Q) for MKM and (.., Q, P) for KMM."""

    def __init__(self, mm, x, fs, y):
        self.mm = mm
        self.is_vec = x.ndim == 1
        if self.is_vec:
            x = x.reshape(1, -1) if mm == "mkm" else x.reshape(-1, 1)
        self.opX, self.xb = _operand(x)
        ops = [_operand(f) for f in fs]
        if len({o for o, _ in ops}) > 1:          # mixed storage: one op is passed for all factors
            ops = [_operand(f, force_contiguous=True) for f in fs]
        self.opF = ops[0][0]
        self.fb = [b for _, b in ops]
        if mm == "mkm":
            self.M, self.K = x.shape[-2], x.shape[-1]
            self.Ps, self.Qs = [f.shape[-2] for f in fs], [f.shape[-1] for f in fs]
        else:
            self.K, self.M = x.shape[-2], x.shape[-1]
            self.Ps, self.Qs = [f.shape[-1] for f in fs], [f.shape[-2] for f in fs]
        if self.K != _prod(self.Ps):
            raise ValueError(f"Input operand x has a mismatch with its dimension ('{self.K}') with the rows of the "
                             f"Kronecker product of fs ('{_prod(self.Ps)}')")
        self.L = _prod(self.Qs)
        self.xbatch, self.fbatch = tuple(x.shape[:-2]), tuple(fs[0].shape[:-2])
        try:
            self.zbatch = tuple(torch.broadcast_shapes(self.xbatch, self.fbatch))
        except RuntimeError:
            raise ValueError(f"Shape {self.xbatch} of x and {self.fbatch} of fs are not broadcastable")
        self.zshape = self.zbatch + ((self.M, self.L) if mm == "mkm" else (self.L, self.M))
        self.yb = None
        self.ybatch = ()
        if y is not None:
            if self.is_vec and y.ndim == 1:
                y = y.reshape(1, -1) if mm == "mkm" else y.reshape(-1, 1)
            if tuple(y.shape[-2:]) != self.zshape[-2:]:
                raise ValueError(f"Input operand 'y' shape {tuple(y.shape)} mismatch with output {self.zshape}")
            self.ybatch = tuple(y.shape[:-2])
            try:
                ok = tuple(torch.broadcast_shapes(self.ybatch, self.zbatch)) == self.zbatch
            except RuntimeError:
                ok = False
            if not ok:
                raise ValueError(f"Input operand 'y' shape {tuple(y.shape)} cannot be broadcasted to output {self.zshape}")
            self.yb = y.contiguous()


def _handle():
    from . import default_handle
    h = default_handle()
    h.set_stream(torch.cuda.current_stream())
    return h


def _address(t, elem_offset=0):
    return ctypes.c_void_p(t.data_ptr() + elem_offset * t.element_size())


def _batch_plan(zbatch, shapes):
    """For every index of the outer batch dims of Z: the linear batch index of each operand (broadcast dims
    clamp to 0) with the innermost index at 0, plus the operand's step along the innermost dim (0 or 1)."""
    d = len(zbatch)
    padded = [(1,) * (d - len(s)) + tuple(s) for s in shapes]
    inner = zbatch[-1]
    outer = zbatch[:-1]
    plans = []
    for lin in range(_prod(outer)):
        idx, rem = [], lin
        for n in reversed(outer):
            idx.append(rem % n)
            rem //= n
        idx = list(reversed(idx)) + [0]
        offs = []
        for s in padded:
            o = 0
            for i, n in zip(idx, s):
                o = o * n + (i if n > 1 else 0)
            offs.append(o)
        plans.append(offs)
    steps = [1 if s[-1] > 1 else 0 for s in padded]
    return inner, plans, steps


def _run(mm, x, fs, alpha, beta, y, keep_intermediates):
    """Returns (z, intermediates); intermediates is [] unless keep_intermediates."""
    _validate(mm, x, fs, y)
    if beta != 0.0 and y is None:
        raise ValueError(f"When beta != 0 ({beta}) then y should not be None")
    p = _Problem(mm, x, fs, y)
    h = _handle()
    lib, pre = h.lib, ("s" if x.dtype == torch.float32 else "d")
    N = len(fs)
    Ps, Qs = capi.arr_u32(p.Ps), capi.arr_u32(p.Qs)
    new = lambda n: torch.empty(n, dtype=x.dtype, device=x.device)
    z = torch.empty(p.zshape, dtype=x.dtype, device=x.device)
    nb = _prod(p.zbatch)

    # batch of X against shared factors: more rows of the same problem (MKM, X stored row-major)
    fold = (mm == "mkm" and len(p.zbatch) > 0 and p.fbatch == () and p.opX == OP_N and
            (p.yb is None or p.ybatch == p.zbatch))
    M = p.M * nb if fold else p.M
    if keep_intermediates:
        widths = h.sizes_forward(p.M, p.Ps, p.Qs)[1]          # elements per problem, one per kept step
        inter = [torch.empty(p.zbatch + ((p.M, w // p.M) if mm == "mkm" else (w // p.M, p.M)),
                             dtype=x.dtype, device=x.device) for w in widths]
        t1 = t2 = None
    else:
        inter = []
        te = h.sizes(M, p.Ps, p.Qs)[1]
        inner = 1 if (fold or not p.zbatch) else p.zbatch[-1]
        t1, t2 = new(te * inner), new(te * inner)

    def check(e, where):
        if e != SUCCESS:
            from . import FastKronError
            raise FastKronError(e, where)

    if fold or not p.zbatch:
        fptr = capi.arr_ptr([f.data_ptr() for f in p.fb])
        if keep_intermediates:
            ip = capi.arr_ptr([t.data_ptr() for t in inter]) if inter else None
            if mm == "mkm":
                check(getattr(lib, pre + "mkmForward")(h.h, BACKEND_HIP, M, N, Ps, Qs, _address(p.xb), p.opX, fptr, p.opF,
                                                       _address(z), ip), "mkmForward")
            else:
                check(getattr(lib, pre + "kmmForward")(h.h, BACKEND_HIP, N, Qs, Ps, M, fptr, p.opF, _address(p.xb), p.opX,
                                                       _address(z), ip), "kmmForward")
        else:
            yp = _address(p.yb) if p.yb is not None else None
            if mm == "mkm":
                check(getattr(lib, pre + "gemkm")(h.h, BACKEND_HIP, M, N, Ps, Qs, _address(p.xb), p.opX, fptr, p.opF,
                                                  _address(z), alpha, beta, yp, _address(t1), _address(t2)), "gemkm")
            else:
                check(getattr(lib, pre + "gekmm")(h.h, BACKEND_HIP, N, Qs, Ps, M, fptr, p.opF, _address(p.xb), p.opX,
                                                  _address(z), alpha, beta, yp, _address(t1), _address(t2)), "gekmm")
    else:
        shapes = [p.xbatch, p.fbatch, p.ybatch if p.yb is not None else p.zbatch, p.zbatch]
        inner, plans, steps = _batch_plan(p.zbatch, shapes)
        xblk, zblk = p.M * p.K, p.M * p.L
        fblk = [a * b for a, b in zip(p.Ps, p.Qs)]
        sF = capi.arr_u64([steps[1] * b for b in fblk])
        for xo, fo, yo, zo in plans:
            fptr = capi.arr_ptr([f.data_ptr() + fo * b * f.element_size() for f, b in zip(p.fb, fblk)])
            xp, zp = _address(p.xb, xo * xblk), _address(z, zo * zblk)
            if keep_intermediates:
                ip = capi.arr_ptr([t.data_ptr() + zo * (w) * t.element_size() for t, w in zip(inter, widths)]) if inter else None
                sI = capi.arr_u64(list(widths)) if inter else None
                if mm == "mkm":
                    check(getattr(lib, pre + "mkmForwardStridedBatched")(
                        h.h, BACKEND_HIP, p.M, N, Ps, Qs, xp, p.opX, steps[0] * xblk, fptr, p.opF, sF, zp, zblk, inner,
                        ip, sI), "mkmForwardStridedBatched")
                else:
                    check(getattr(lib, pre + "kmmForwardStridedBatched")(
                        h.h, BACKEND_HIP, N, Qs, Ps, p.M, fptr, p.opF, sF, xp, p.opX, steps[0] * xblk, zp, zblk, inner,
                        ip, sI), "kmmForwardStridedBatched")
            else:
                yp = _address(p.yb, yo * zblk) if p.yb is not None else None
                sY = steps[2] * zblk if p.yb is not None else 0
                if mm == "mkm":
                    check(getattr(lib, pre + "gemkmStridedBatched")(
                        h.h, BACKEND_HIP, p.M, N, Ps, Qs, xp, p.opX, steps[0] * xblk, fptr, p.opF, sF, zp, zblk,
                        alpha, beta, inner, yp, sY, _address(t1), _address(t2)), "gemkmStridedBatched")
                else:
                    check(getattr(lib, pre + "gekmmStridedBatched")(
                        h.h, BACKEND_HIP, N, Qs, Ps, p.M, fptr, p.opF, sF, xp, p.opX, steps[0] * xblk, zp, zblk,
                        alpha, beta, inner, yp, sY, _address(t1), _address(t2)), "gekmmStridedBatched")
    if p.is_vec:
        z = z.reshape(z.shape[:-2] + (-1,))
    return z, inter


def _sum_to(g, shape):
    """Reduce a gradient over the dimensions that were broadcast in the forward pass."""
    return g.sum_to_size(shape) if tuple(g.shape) != tuple(shape) else g


def _mkm_backward(grad_z, x, fs, inter, need_x, need_f):
    """Gradients of Z = X (F_0 (x) ... (x) F_{N-1}) (logical MKM shapes).  inter[j] is the input of the step of
    factor j (the output of the step of factor j+1); the input of the last factor's step is X itself.
    Step of factor i maps rows (m, s) of its input, reshaped (M*S, P_i), through F_i and stores column q at
    q*S + s; its backward therefore un-shuffles the output gradient to (M*S, Q_i) first."""
    inputs = list(inter) + [x]
    M = grad_z.shape[-2]
    g = grad_z
    grad_fs = []
    for i, f in enumerate(fs):
        P, Q = f.shape[-2], f.shape[-1]
        S = g.shape[-1] // Q
        a = g.reshape(g.shape[:-2] + (M, Q, S)).transpose(-1, -2).reshape(g.shape[:-2] + (M * S, Q))
        if need_f[i]:
            inp = inputs[i]
            inp = inp.reshape(inp.shape[:-2] + (M * S, P))
            grad_fs.append(_sum_to(inp.mT @ a, f.shape))
        else:
            grad_fs.append(None)
        if i + 1 < len(fs) or need_x:
            g = (a @ f.mT).reshape(a.shape[:-2] + (M, S * P))
    return (_sum_to(g, x.shape) if need_x else None), grad_fs


class MKM(torch.autograd.Function):
    """Z = X (F_0 (x) ... (x) F_{N-1}) with gradients (reference fastkrontorch.py:340-357)."""

    @staticmethod
    def forward(ctx, x, *fs):
        need_f = any(f.requires_grad for f in fs)
        z, inter = _run("mkm", x, fs, 1.0, 0.0, None, keep_intermediates=need_f)
        ctx.save_for_backward(x, *fs, *inter)
        ctx.nf, ctx.kept = len(fs), need_f
        return z

    @staticmethod
    def backward(ctx, grad_z):
        x, fs, inter = ctx.saved_tensors[0], ctx.saved_tensors[1:ctx.nf + 1], ctx.saved_tensors[ctx.nf + 1:]
        need_x, need_f = ctx.needs_input_grad[0], ctx.needs_input_grad[1:ctx.nf + 1]
        if not any(need_f):
            # dX = dZ (F_0^T (x) ... (x) F_{N-1}^T): one fused library call on the transposed views
            gx = _run("mkm", grad_z, [f.mT for f in fs], 1.0, 0.0, None, False)[0] if need_x else None
            return (_sum_to(gx, x.shape) if gx is not None else None,) + (None,) * ctx.nf
        xv = x.reshape(1, -1) if x.ndim == 1 else x
        gz = grad_z.reshape(1, -1) if grad_z.ndim == 1 else grad_z
        gx, gfs = _mkm_backward(gz, xv, fs, inter, need_x, need_f)
        if gx is not None and x.ndim == 1:
            gx = gx.reshape(x.shape)
        return (gx,) + tuple(gfs)


class KMM(torch.autograd.Function):
    """Z = (F_0 (x) ... (x) F_{N-1}) X with gradients (reference fastkrontorch.py:360-378); the arguments
    are (x, *fs) as in the reference."""

    @staticmethod
    def forward(ctx, x, *fs):
        need_f = any(f.requires_grad for f in fs)
        z, inter = _run("kmm", x, fs, 1.0, 0.0, None, keep_intermediates=need_f)
        ctx.save_for_backward(x, *fs, *inter)
        ctx.nf = len(fs)
        return z

    @staticmethod
    def backward(ctx, grad_z):
        x, fs, inter = ctx.saved_tensors[0], ctx.saved_tensors[1:ctx.nf + 1], ctx.saved_tensors[ctx.nf + 1:]
        need_x, need_f = ctx.needs_input_grad[0], ctx.needs_input_grad[1:ctx.nf + 1]
        if not any(need_f):
            # dX = (F_0^T (x) ... (x) F_{N-1}^T) dZ
            gx = _run("kmm", grad_z, [f.mT for f in fs], 1.0, 0.0, None, False)[0] if need_x else None
            return (_sum_to(gx, x.shape) if gx is not None else None,) + (None,) * ctx.nf
        # Z^T = X^T (F_0^T (x) ...): the MKM rule on the transposed tensors
        xv = x.reshape(-1, 1) if x.ndim == 1 else x
        gz = grad_z.reshape(-1, 1) if grad_z.ndim == 1 else grad_z
        gx, gfs = _mkm_backward(gz.mT, xv.mT, [f.mT for f in fs], [t.mT for t in inter], need_x, need_f)
        if gx is not None:
            gx = gx.mT.reshape(x.shape)
        return (gx,) + tuple(g.mT if g is not None else None for g in gfs)


def _wants_grad(x, fs):
    return torch.is_grad_enabled() and (x.requires_grad or any(f.requires_grad for f in fs))


def _no_epilogue_with_grad(alpha, beta, y):
    if alpha != 1:
        raise ValueError(f"When requires_grad is True alpha should be 1 but is {alpha}")
    if beta != 0:
        raise ValueError(f"When requires_grad is True beta should be 0 but is {beta}")
    if y is not None:
        raise ValueError("When requires_grad is True y should be None")


def gemkm(x, fs, alpha=1.0, beta=0.0, y=None):
    """Z = alpha * X (F_0 (x) ... (x) F_{N-1}) + beta * Y.  X is (.., M, prod P) or a vector of prod P elements,
    fs[i] is (.., P_i, Q_i), Y broadcastable to Z (reference fastkrontorch.py:404-434)."""
    _validate("mkm", x, fs, y)
    if _wants_grad(x, fs):
        _no_epilogue_with_grad(alpha, beta, y)
        return MKM.apply(x, *fs)
    return _run("mkm", x, fs, float(alpha), float(beta), y, False)[0]


def gekmm(fs, x, alpha=1.0, beta=0.0, y=None):
    """Z = alpha * (F_0 (x) ... (x) F_{N-1}) X + beta * Y.  X is (.., prod P, M) or a vector, fs[i] is
    (.., Q_i, P_i) (reference fastkrontorch.py:437-465)."""
    _validate("kmm", x, fs, y)
    if _wants_grad(x, fs):
        _no_epilogue_with_grad(alpha, beta, y)
        return KMM.apply(x, *fs)
    return _run("kmm", x, fs, float(alpha), float(beta), y, False)[0]
