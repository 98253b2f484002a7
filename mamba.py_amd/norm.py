"""RMSNorm on the gfx950 kernel: y = x * rsqrt(mean(x^2, -1) + eps) [* weight]
(mambapy/mamba.py:416-433), one pass forward and one backward instead of five elementwise
kernels each way."""
import ctypes

import torch

from . import _lib
from .scan import _f32c, _io_dtype, _ptr, _require_gpu, _stream


def rmsnorm_supported(x) -> bool:
    """Shapes the kernel takes: float32 / bfloat16, last dim a multiple of 4 / 8 and at most
    2048 / 4096."""
    if x.dtype == torch.float32:
        return x.shape[-1] % 4 == 0 and x.shape[-1] <= 2048
    if x.dtype == torch.bfloat16:
        return x.shape[-1] % 8 == 0 and x.shape[-1] <= 4096
    return False


def _norm_backward(ctx, x, w, dy, dsum):
    lib = _lib.load()
    d = x.shape[-1]
    rows = x.numel() // d
    dy = dy.to(x.dtype).contiguous()
    if dsum is not None:
        dsum = dsum.to(x.dtype).contiguous()
    dx = torch.empty_like(x)
    dw = ws = None
    nbytes = 0
    if w is not None:
        dw = torch.empty(d, dtype=torch.float32, device=x.device)
        nbytes = lib.mpa_rmsnorm_bwd_workspace_bytes(rows, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.mpa_rmsnorm_bwd(_ptr(x), _ptr(w), _ptr(dy), _ptr(dsum), _ptr(dx), _ptr(dw), rows, d,
                                 ctx.eps, _io_dtype(x), _ptr(ws), nbytes, _stream(x.device))
    _lib.check(rc, "mpa_rmsnorm_bwd")
    return dx, None if dw is None else dw.to(ctx.wdtype)


class RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        _require_gpu(x, weight)
        lib = _lib.load()
        io = _io_dtype(x)
        d = x.shape[-1]
        x_ = x.detach().contiguous()
        rows = x_.numel() // d
        w_ = _f32c(weight)
        y = torch.empty_like(x_)
        with torch.cuda.device(x.device):
            rc = lib.mpa_rmsnorm_fwd(_ptr(x_), None, _ptr(w_), _ptr(y), None, None, rows, d, eps, io,
                                     _stream(x.device))
        _lib.check(rc, "mpa_rmsnorm_fwd")
        ctx.save_for_backward(x_, w_)
        ctx.eps = eps
        ctx.wdtype = None if weight is None else weight.dtype
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dx, dw = _norm_backward(ctx, x, w, dy, None)
        return dx, dw, None


class AddRMSNormFn(torch.autograd.Function):
    """(x, residual) -> (rmsnorm(x + residual), x + residual) in one pass each way."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps):
        _require_gpu(x, residual, weight)
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise RuntimeError("residual must have the shape and dtype of x")
        lib = _lib.load()
        io = _io_dtype(x)
        d = x.shape[-1]
        x_, r_ = x.detach().contiguous(), residual.detach().contiguous()
        rows = x_.numel() // d
        w_ = _f32c(weight)
        y, total = torch.empty_like(x_), torch.empty_like(x_)
        with torch.cuda.device(x.device):
            rc = lib.mpa_rmsnorm_fwd(_ptr(x_), _ptr(r_), _ptr(w_), _ptr(y), _ptr(total), None, rows, d, eps,
                                     io, _stream(x.device))
        _lib.check(rc, "mpa_rmsnorm_fwd")
        ctx.save_for_backward(total, w_)
        ctx.eps = eps
        ctx.wdtype = None if weight is None else weight.dtype
        return y, total

    @staticmethod
    def backward(ctx, dy, dtotal):
        total, w = ctx.saved_tensors
        if dy is None:
            dy = torch.zeros_like(total)
        g, dw = _norm_backward(ctx, total, w, dy, dtotal)
        return g, g, dw, None


def add_rmsnorm_fn(x, residual, weight=None, eps: float = 1e-5):
    """The residual add of the layer stack folded into the norm that reads its result
    (mambapy/mamba.py:106-112).  Returns (rmsnorm(x + residual) [* weight], x + residual)."""
    return AddRMSNormFn.apply(x, residual, weight, float(eps))


def rmsnorm_fn(x, weight=None, eps: float = 1e-5):
    """x : (..., d);  weight : (d) or None.  Returns a contiguous tensor of x's shape."""
    return RMSNormFn.apply(x, weight, float(eps))
