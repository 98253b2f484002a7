"""Host side of the selective-scan hot path: the reference's operator surface
(`pscan`, `selective_scan`, `ssm_step`) bound to the gfx950 kernels through the C ABI.

Mirrors, by name and argument meaning:
  pscan(A, X)                                   mambapy/pscan.py:151-226
  selective_scan(x, delta, A, B, C, D)          mambapy/mamba.py:274-295
  selective_scan_fn(..., z=, delta_bias=, delta_softplus=)   the fused call of mamba.py:259-260
  ssm_step(x, delta, A, B, C, D, h)             mambapy/mamba.py:400-412
PyTorch supplies device memory, streams and the autograd graph; all arithmetic runs in
libmambapy_amd.so.  Tensors must live on a ROCm device: there is no CPU path.
"""
import contextlib
import ctypes
import os

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.MPA_F32, torch.bfloat16: _lib.MPA_BF16}


def _io_dtype(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}: the kernels take float32 or bfloat16 "
                        "tensors (state and accumulation are float32 in both cases)") from None


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mambapy_amd ops need tensors on a ROCm device "
                               "(there is no CPU implementation in this package)")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _f32c(t):
    return None if t is None else t.detach().to(torch.float32).contiguous()


def _rows_unit_stride(t):
    """(B, L, N) tensor whose last stride is 1 (slices of a projection qualify)."""
    return t if t.stride(-1) == 1 else t.contiguous()


class LaunchPlan:
    """Overrides of the decomposition the library would choose from the shape (None / False =
    let it choose).  The library itself reads no environment: the MPA_* variables below are
    read here, once, when the module is imported, and travel to the kernels inside the shape
    struct of every call.

        MPA_FWD_NS / MPA_BWD_NS       states of d_state per lane (a power of two)
        MPA_FWD_NSEG / MPA_BWD_NSEG   segments a sequence is cut into (1 = never cut)
        MPA_PSCAN_CHUNKS              pieces the generic scan cuts a sequence into (1 = never cut)
        MPA_BWD_GENERAL=1             general backward kernel even where the fast one applies
        MPA_GROUP_CHANNELS            64 or 48 channels of a batch row per workgroup
    """
    _FIELDS = ("fwd_states_per_lane", "bwd_states_per_lane", "fwd_segments", "bwd_segments",
               "bwd_general", "expire_waits", "pscan_chunks", "group_channels")

    def __init__(self):
        env = lambda k: int(os.environ[k]) if os.environ.get(k, "").strip() else None
        self.fwd_states_per_lane = env("MPA_FWD_NS")
        self.bwd_states_per_lane = env("MPA_BWD_NS")
        self.fwd_segments = env("MPA_FWD_NSEG")
        self.bwd_segments = env("MPA_BWD_NSEG")
        self.pscan_chunks = env("MPA_PSCAN_CHUNKS")
        self.bwd_general = os.environ.get("MPA_BWD_GENERAL", "") == "1"
        self.expire_waits = False  # test hook (MPA_PLAN_EXPIRE_WAITS)
        self.group_channels = env("MPA_GROUP_CHANNELS")  # 64 or 48 channels per workgroup (None: the library picks)

    def fill(self, shape, backward):
        shape.plan_states_per_lane = (self.bwd_states_per_lane if backward else self.fwd_states_per_lane) or 0
        shape.plan_segments = (self.bwd_segments if backward else self.fwd_segments) or 0
        shape.plan_flags = (_lib.MPA_PLAN_BWD_GENERAL if self.bwd_general else 0) | \
                           (_lib.MPA_PLAN_EXPIRE_WAITS if self.expire_waits else 0) | \
                           {None: 0, 64: _lib.MPA_PLAN_GROUP_64, 48: _lib.MPA_PLAN_GROUP_48}[self.group_channels]


plan = LaunchPlan()


@contextlib.contextmanager
def plan_override(**kw):
    """with plan_override(fwd_segments=4, bwd_states_per_lane=2): ...  (tuning and tests)"""
    for k in kw:
        if k not in LaunchPlan._FIELDS:
            raise TypeError(f"unknown plan field {k!r}")
    old = {k: getattr(plan, k) for k in kw}
    for k, v in kw.items():
        setattr(plan, k, v)
    try:
        yield plan
    finally:
        for k, v in old.items():
            setattr(plan, k, v)


def _sscan_shape(x, delta, Bm, y_like, g_like, dbc_like, N, flags, z=None, backward=False):
    """Shape struct of one call.  delta may be float32 next to bfloat16 tensors (the reference's call
    under autocast, mambapy/mamba.py:264-265): the library then reads it, and writes ddelta, as float32."""
    s = _lib.SscanShape()
    s.batch, s.seqlen, s.dim = x.shape
    s.dstate = N
    s.io_dtype = _io_dtype(x)
    s.flags = flags
    s.u_sb, s.u_sl, s.u_sd = x.stride()
    if z is not None:
        s.z_sb, s.z_sl, s.z_sd = z.stride()
    s.d_sb, s.d_sl, s.d_sd = delta.stride()
    s.delta_dtype = _lib.MPA_DELTA_F32 if (delta.dtype == torch.float32 and x.dtype != torch.float32) else 0
    s.y_sb, s.y_sl, s.y_sd = y_like.stride()
    s.g_sb, s.g_sl, s.g_sd = g_like.stride()
    s.bc_sb, s.bc_sl = Bm.stride(0), Bm.stride(1)
    s.dbc_sb, s.dbc_sl = dbc_like.stride(0), dbc_like.stride(1)
    plan.fill(s, backward)
    return s


class SelectiveScanFn(torch.autograd.Function):
    """Fused discretise -> scan -> readout with a hand-written backward kernel."""

    @staticmethod
    def forward(ctx, x, delta, A, B, C, D, z, delta_bias, delta_softplus, h0, return_last_state,
                need_grad=True, reverse=False):
        _require_gpu(x, delta, A, B, C, D, z, delta_bias, h0)
        lib = _lib.load()
        dt = x.dtype
        _io_dtype(x)
        Bsz, L, ED = x.shape
        N = A.shape[-1]
        if delta.shape != x.shape or A.shape != (ED, N) or B.shape != (Bsz, L, N) \
                or C.shape != (Bsz, L, N) or D.shape != (ED,):
            raise RuntimeError(
                f"shape mismatch: x{tuple(x.shape)} delta{tuple(delta.shape)} A{tuple(A.shape)} "
                f"B{tuple(B.shape)} C{tuple(C.shape)} D{tuple(D.shape)}")
        if z is not None and z.shape != x.shape:
            raise RuntimeError("z must have the shape of x")
        if delta_bias is not None and not delta_softplus:
            raise RuntimeError("delta_bias needs delta_softplus=True")
        if h0 is not None and h0.requires_grad and need_grad:
            raise RuntimeError("selective_scan_fn: no gradient is computed for h0; pass h0.detach()")
        x_ = x.detach()
        # float32 delta next to bfloat16 x, B, C is what the reference passes under autocast (softplus
        # promotes to float32): it is read as it is, unrounded and without a copy (the general
        # backward kernel, which only a pinned plan selects, has no such path)
        if delta.dtype == torch.float32 and dt == torch.bfloat16 and not plan.bwd_general:
            delta_ = delta.detach()
        else:
            delta_ = delta.detach().to(dt)
        B_ = _rows_unit_stride(B.detach().to(dt))
        C_ = _rows_unit_stride(C.detach().to(dt))
        if C_.stride() != B_.stride():
            B_, C_ = B_.contiguous(), C_.contiguous()
        z_ = None if z is None else z.detach().to(dt)
        A_, D_, bias_, h0_ = _f32c(A), _f32c(D), _f32c(delta_bias), _f32c(h0)
        y = torch.empty((Bsz, L, ED), dtype=dt, device=x.device)
        # need_grad: checkpoints (and the pre-gate output) are written only for a backward pass;
        # without them the library is also free to cut a long sequence into parallel segments
        flags = (_lib.MPA_SSCAN_DELTA_SOFTPLUS if delta_softplus else 0) | \
                (_lib.MPA_SSCAN_REVERSE if reverse else 0)
        shape = _sscan_shape(x_, delta_, B_, y, y, B_, N, flags, z_)
        ckpt = y_pre = None
        if need_grad:
            ckpt = torch.empty(lib.mpa_sscan_ckpt_elems(ctypes.byref(shape)), dtype=torch.float32,
                               device=x.device)
            if z_ is not None:
                y_pre = torch.empty_like(y)  # output before the gate, read again by the backward
        h_last = torch.empty((Bsz, ED, N), dtype=torch.float32, device=x.device) \
            if return_last_state else None
        nbytes = lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(shape), 1 if need_grad else 0)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        with torch.cuda.device(x.device):
            rc = lib.mpa_sscan_fwd(ctypes.byref(shape), _ptr(x_), _ptr(delta_), _ptr(A_), _ptr(B_),
                                   _ptr(C_), _ptr(D_), _ptr(z_), _ptr(bias_), _ptr(h0_), _ptr(y),
                                   _ptr(y_pre), _ptr(ckpt), _ptr(h_last), _ptr(ws), nbytes,
                                   _stream(x.device))
        _lib.check(rc, "mpa_sscan_fwd")
        ctx.save_for_backward(x_, delta_, A_, B_, C_, D_, z_, bias_, h0_, ckpt, y_pre)
        ctx.flags = flags
        ctx.in_dtypes = (x.dtype, delta.dtype, A.dtype, B.dtype, C.dtype, D.dtype,
                         None if z is None else z.dtype,
                         None if delta_bias is None else delta_bias.dtype)
        if return_last_state:
            ctx.mark_non_differentiable(h_last)
            return y, h_last
        return y

    @staticmethod
    def backward(ctx, dy, *unused):
        lib = _lib.load()
        x, delta, A, B, C, D, z, bias, h0, ckpt, y_pre = ctx.saved_tensors
        if ckpt is None:
            raise RuntimeError("backward called on a selective scan that saved no checkpoints")
        dt = x.dtype
        Bsz, L, ED = x.shape
        N = A.shape[-1]
        dy = dy.to(dt)
        if y_pre is not None and dy.stride() != y_pre.stride():
            dy = dy.contiguous()  # the saved pre-gate output is addressed with dy's strides
        dx = torch.empty((Bsz, L, ED), dtype=dt, device=x.device)
        ddelta = torch.empty((Bsz, L, ED), dtype=delta.dtype, device=x.device)   # float32 with a float32 delta
        dz = torch.empty_like(dx) if z is not None else None
        dA = torch.empty((ED, N), dtype=torch.float32, device=x.device)
        dD = torch.empty((ED,), dtype=torch.float32, device=x.device)
        dB = torch.empty((Bsz, L, N), dtype=dt, device=x.device)
        dC = torch.empty_like(dB)
        dbias = torch.empty((ED,), dtype=torch.float32, device=x.device) if bias is not None else None
        shape = _sscan_shape(x, delta, B, dy, dx, dB, N, ctx.flags, z, backward=True)
        nbytes = lib.mpa_sscan_bwd_workspace_bytes(ctypes.byref(shape))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        with torch.cuda.device(x.device):
            rc = lib.mpa_sscan_bwd(ctypes.byref(shape), _ptr(x), _ptr(delta), _ptr(A), _ptr(B),
                                   _ptr(C), _ptr(D), _ptr(z), _ptr(bias), _ptr(h0), _ptr(dy),
                                   _ptr(y_pre), _ptr(ckpt), _ptr(dx), _ptr(ddelta), _ptr(dA), _ptr(dB), _ptr(dC),
                                   _ptr(dD), _ptr(dz), _ptr(dbias), _ptr(ws), nbytes,
                                   _stream(x.device))
        _lib.check(rc, "mpa_sscan_bwd")
        tx, td, tA, tB, tC, tD, tz, tb = ctx.in_dtypes
        return (dx.to(tx), ddelta.to(td), dA.to(tA), dB.to(tB), dC.to(tC), dD.to(tD),
                None if dz is None else dz.to(tz), None if dbias is None else dbias.to(tb),
                None, None, None, None, None)


def selective_scan_fn(x, delta, A, B, C, D, z=None, delta_bias=None, delta_softplus=False,
                      h0=None, return_last_state=False, reverse=False):
    """y = selective scan of (x, delta, A, B, C, D), optionally with softplus(delta + bias)
    and the gate y*silu(z) folded in (the fused form the reference reaches through
    `use_cuda`, mambapy/mamba.py:252-261), in this package's (B, L, ED) layout.

    x, delta, z : (B, L, ED);  A : (ED, N);  B, C : (B, L, N);  D, delta_bias : (ED);
    h0 : optional (B, ED, N) initial state.  Returns y (B, L, ED) [, last state (B, ED, N)].
    reverse=True runs the recurrence from the last step to the first: the same result as
    flipping x, delta, z, B, C along time, scanning and flipping y back (the backward direction
    of the reference's bidirectional block, mambapy/vim.py:228-261), without the copies; h0 is
    then the state before step L-1 and the last state the one after step 0.
    """
    # grad mode is off inside Function.forward and parameters keep requires_grad under no_grad,
    # so whether a backward can follow is decided here
    need_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (x, delta, A, B, C, D, z, delta_bias))
    return SelectiveScanFn.apply(x, delta, A, B, C, D, z, delta_bias, bool(delta_softplus), h0,
                                 bool(return_last_state), need_grad, bool(reverse))


def selective_scan(x, delta, A, B, C, D):
    """Drop-in for MambaBlock.selective_scan / selective_scan_seq
    (mambapy/mamba.py:274-327): same arguments, same result, differentiable."""
    return selective_scan_fn(x, delta, A, B, C, D)


# ------------------------------------------------------------------------------------------
# generic scan
# ------------------------------------------------------------------------------------------

def _pscan_shape(A, X, H, gA=None, gX=None, reverse=False):
    s = _lib.PscanShape()
    s.batch, s.seqlen, s.dim, s.dstate = X.shape
    s.io_dtype = _io_dtype(X)
    s.reverse = 1 if reverse else 0
    s.plan_chunks = plan.pscan_chunks or 0
    for name, t in (("a_st", A), ("x_st", X), ("h_st", H), ("ga_st", gA), ("gx_st", gX)):
        if t is not None:
            getattr(s, name)[:] = list(t.stride())
    return s


class PScan(torch.autograd.Function):
    """H[t] = A[t]*H[t-1] + X[t] along dim 1 of (B, L, D, N) tensors; returns a new tensor
    and never modifies its inputs (mambapy/pscan.py:151-224).  Any L: no padding."""

    @staticmethod
    def forward(ctx, A_in, X_in, reverse=False):
        _require_gpu(A_in, X_in)
        if A_in.shape != X_in.shape or X_in.dim() != 4:
            raise RuntimeError(f"pscan expects two (B, L, D, N) tensors, got {tuple(A_in.shape)} "
                               f"and {tuple(X_in.shape)}")
        lib = _lib.load()
        dt = torch.promote_types(A_in.dtype, X_in.dtype)
        if dt not in _DTYPES:
            raise TypeError(f"unsupported dtype {dt}")
        A = A_in.detach().to(dt)
        X = X_in.detach().to(dt)
        H = torch.empty(X.shape, dtype=dt, device=X.device)
        shape = _pscan_shape(A, X, H, reverse=reverse)
        nbytes = lib.mpa_pscan_workspace_bytes(ctypes.byref(shape))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=X.device)
        with torch.cuda.device(X.device):
            rc = lib.mpa_pscan_fwd(ctypes.byref(shape), _ptr(A), _ptr(X), _ptr(H), _ptr(ws), nbytes,
                                   _stream(X.device))
        _lib.check(rc, "mpa_pscan_fwd")
        ctx.save_for_backward(A, H)
        ctx.in_dtypes = (A_in.dtype, X_in.dtype)
        ctx.reverse = bool(reverse)
        return H

    @staticmethod
    def backward(ctx, grad_output_in):
        lib = _lib.load()
        A, H = ctx.saved_tensors
        G = grad_output_in.to(H.dtype)
        gA = torch.empty_like(H)
        gX = torch.empty_like(H)
        shape = _pscan_shape(A, G, H, gA, gX, reverse=ctx.reverse)
        nbytes = lib.mpa_pscan_workspace_bytes(ctypes.byref(shape))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=H.device)
        with torch.cuda.device(H.device):
            rc = lib.mpa_pscan_bwd(ctypes.byref(shape), _ptr(A), _ptr(H), _ptr(G), _ptr(gA), _ptr(gX),
                                   _ptr(ws), nbytes, _stream(H.device))
        _lib.check(rc, "mpa_pscan_bwd")
        return gA.to(ctx.in_dtypes[0]), gX.to(ctx.in_dtypes[1]), None


pscan = PScan.apply


def pscan_rev(A, X):
    """H[t] = A[t]*H[t+1] + X[t], H[L] = 0: the scan of mambapy/pscan.py:94-149
    (PScan.pscan_rev, `flip . pscan . flip`) as a differentiable call of its own."""
    return PScan.apply(A, X, True)


# ------------------------------------------------------------------------------------------
# decode step
# ------------------------------------------------------------------------------------------

def ssm_step(x, delta, A, B, C, D, h=None, z=None, delta_bias=None, delta_softplus=False,
             inplace=False):
    """One token: h' = exp(delta*A)*h + delta*B*x, y = C.h' + D*x (mambapy/mamba.py:400-412).

    x, delta, z : (B, ED);  A : (ED, N);  B, C : (B, N);  D, delta_bias : (ED);
    h : (B, ED, N) float32 or None (zeros).  Returns (y, h').  By default h' is a new tensor
    and h is left untouched, as in the reference; inplace=True updates h itself.
    No autograd: decoding runs under torch.no_grad().
    """
    _require_gpu(x, delta, A, B, C, D, h, z, delta_bias)
    lib = _lib.load()
    dt = x.dtype
    io = _io_dtype(x)
    Bsz, ED = x.shape
    N = A.shape[-1]
    x_ = x.detach().contiguous()
    delta_ = delta.detach().to(dt).contiguous()
    z_ = None if z is None else _rows_unit_stride(z.detach().to(dt))   # a half of in_proj's output
    B_ = _rows_unit_stride(B.detach().to(dt))
    C_ = _rows_unit_stride(C.detach().to(dt))
    if B_.stride(0) != C_.stride(0):
        B_, C_ = B_.contiguous(), C_.contiguous()
    A_, D_, bias_ = _f32c(A), _f32c(D), _f32c(delta_bias)
    if h is not None:
        if h.dtype != torch.float32 or not h.is_contiguous() or h.shape != (Bsz, ED, N):
            if inplace:
                raise RuntimeError("in-place step needs a contiguous float32 (B, ED, N) state")
            h = h.detach().to(torch.float32).contiguous()
    if inplace and h is None:
        raise RuntimeError("in-place step needs an existing state tensor")
    h_out = h if inplace else torch.empty((Bsz, ED, N), dtype=torch.float32, device=x.device)
    y = torch.empty((Bsz, ED), dtype=dt, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.mpa_ssm_step(_ptr(x_), _ptr(delta_), _ptr(A_), _ptr(B_), _ptr(C_), _ptr(D_),
                              _ptr(z_), _ptr(bias_), _ptr(h), _ptr(h_out), _ptr(y), Bsz, ED, N,
                              B_.stride(0), 0 if z_ is None else z_.stride(0), io,
                              1 if delta_softplus else 0, _stream(x.device))
    _lib.check(rc, "mpa_ssm_step")
    return y, h_out
