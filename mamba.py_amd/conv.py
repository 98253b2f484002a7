"""Causal depthwise convolution along time (+ bias, + SiLU) on the gfx950 kernel.

`causal_conv1d_fn(x, weight, bias)` is what MambaBlock.forward computes with
    conv1d(x.transpose(1, 2))[:, :, :L].transpose(1, 2) followed by silu
(mambapy/mamba.py:217-221), on the (B, L, ED) tensor directly: any strides are read in place,
the result is a new (B, L, ED) tensor with unit stride along ED.
"""
import ctypes

import torch

from . import _lib
from .scan import _f32c, _io_dtype, _ptr, _require_gpu, _stream


def _conv_shape(x, y_like, g_like, K, silu):
    s = _lib.ConvShape()
    s.batch, s.seqlen, s.dim = x.shape
    s.kernel = K
    s.io_dtype = _io_dtype(x)
    s.flags = _lib.MPA_CONV_SILU if silu else 0
    s.x_sb, s.x_sl, s.x_sd = x.stride()
    s.y_sb, s.y_sl, s.y_sd = y_like.stride()
    s.g_sb, s.g_sl, s.g_sd = g_like.stride()
    return s


class CausalConv1dFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, window, silu, return_window):
        _require_gpu(x, weight, bias, window)
        lib = _lib.load()
        if x.dim() != 3:
            raise RuntimeError("x must be (B, L, ED)")
        Bsz, L, ED = x.shape
        K = weight.shape[-1]
        if weight.numel() != ED * K:
            raise RuntimeError(f"weight must be (ED, 1, K) or (ED, K), got {tuple(weight.shape)}")
        if window is not None and window.shape != (Bsz, ED, K - 1):
            raise RuntimeError("window must be (B, ED, K-1)")
        x_ = x.detach()
        w_ = _f32c(weight).view(ED, K)
        b_ = _f32c(bias)
        win_ = None if window is None else window.detach().to(x.dtype).contiguous()
        y = torch.empty((Bsz, L, ED), dtype=x.dtype, device=x.device)
        wout = torch.empty((Bsz, ED, K - 1), dtype=x.dtype, device=x.device) if return_window else None
        shape = _conv_shape(x_, y, y, K, silu)
        with torch.cuda.device(x.device):
            rc = lib.mpa_conv1d_fwd(ctypes.byref(shape), _ptr(x_), _ptr(w_), _ptr(b_), _ptr(win_),
                                    _ptr(y), _ptr(wout), _stream(x.device))
        _lib.check(rc, "mpa_conv1d_fwd")
        ctx.save_for_backward(x_, w_, b_, win_)
        ctx.silu = silu
        ctx.meta = (weight.shape, weight.dtype, None if bias is None else bias.dtype)
        if return_window:
            ctx.mark_non_differentiable(wout)
            return y, wout
        return y

    @staticmethod
    def backward(ctx, dy, *unused):
        lib = _lib.load()
        x, w, b, win = ctx.saved_tensors
        Bsz, L, ED = x.shape
        K = w.shape[-1]
        dy = dy.to(x.dtype)
        dx = torch.empty((Bsz, L, ED), dtype=x.dtype, device=x.device)
        dw = torch.empty((ED, K), dtype=torch.float32, device=x.device)
        db = torch.empty((ED,), dtype=torch.float32, device=x.device) if b is not None else None
        shape = _conv_shape(x, dy, dx, K, ctx.silu)
        nbytes = lib.mpa_conv1d_bwd_workspace_bytes(ctypes.byref(shape))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        with torch.cuda.device(x.device):
            rc = lib.mpa_conv1d_bwd(ctypes.byref(shape), _ptr(x), _ptr(w), _ptr(b), _ptr(win), _ptr(dy),
                                    _ptr(dx), _ptr(dw), _ptr(db), _ptr(ws), nbytes, _stream(x.device))
        _lib.check(rc, "mpa_conv1d_bwd")
        wshape, wdtype, bdtype = ctx.meta
        return (dx, dw.view(wshape).to(wdtype), None if db is None else db.to(bdtype), None, None, None)


def causal_conv1d_update(x, window, weight, bias=None, silu=True):
    """One decode step of the convolution (mambapy/mamba.py:366-369, 379) in one kernel:
    x : (B, ED) newest input (any row stride);  window : (B, ED, K-1) contiguous rolling cache of
    the previous inputs, UPDATED IN PLACE (oldest dropped, x appended).  Returns
    silu(conv) as (B, ED).  No autograd: decoding runs under torch.no_grad()."""
    _require_gpu(x, window, weight, bias)
    lib = _lib.load()
    Bsz, ED = x.shape
    K = weight.shape[-1]
    if window.shape != (Bsz, ED, K - 1) or window.dtype != x.dtype or not window.is_contiguous():
        raise RuntimeError("window must be a contiguous (B, ED, K-1) tensor of x's dtype")
    x_ = x.detach().unsqueeze(1)
    w_ = _f32c(weight).view(ED, K)
    b_ = _f32c(bias)
    y = torch.empty((Bsz, 1, ED), dtype=x.dtype, device=x.device)
    shape = _conv_shape(x_, y, y, K, silu)
    with torch.cuda.device(x.device):
        rc = lib.mpa_conv1d_fwd(ctypes.byref(shape), _ptr(x_), _ptr(w_), _ptr(b_), _ptr(window), _ptr(y),
                                _ptr(window), _stream(x.device))
    _lib.check(rc, "mpa_conv1d_fwd")
    return y[:, 0]


def causal_conv1d_fn(x, weight, bias=None, window=None, silu=True, return_window=False):
    """x : (B, L, ED) (any strides);  weight : (ED, 1, K) or (ED, K), K in 2..4;  bias : (ED).
    window : optional (B, ED, K-1) inputs before step 0 (zeros if None).
    Returns silu(conv(x)) as (B, L, ED) [, the last K-1 inputs as (B, ED, K-1)]."""
    return CausalConv1dFn.apply(x, weight, bias, window, bool(silu), bool(return_window))
