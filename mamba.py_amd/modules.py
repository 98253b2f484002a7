"""Callers of the selective-scan hot path, restated on top of the gfx950 kernels.

These classes mirror the reference's public surface (constructor arguments, method names,
tensor shapes and `state_dict` keys) so that a model built or trained with mambapy loads
here and the other way round:
    MambaConfig, MambaBlock, ResidualBlock, Mamba, RMSNorm      mambapy/mamba.py:31-433
They are the harness around the kernels, not the product: projections, the depthwise
convolution and the norms stay on PyTorch-ROCm library calls; the scan, its backward and the
decode-step state update run in libmambapy_amd.so.
"""
import math
from dataclasses import dataclass
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from .conv import causal_conv1d_fn, causal_conv1d_update
from .norm import add_rmsnorm_fn, rmsnorm_fn, rmsnorm_supported
from .scan import selective_scan, selective_scan_fn, ssm_step


@dataclass
class MambaConfig:
    """Same fields and derived values as mambapy/mamba.py:31-67 (d_inner = expand_factor *
    d_model, dt_rank = ceil(d_model / 16) when 'auto').  `pscan` / `use_cuda` are accepted for
    compatibility; both select the fused HIP scan here.  `fused_softplus` folds
    softplus(delta + dt_proj.bias) into the scan kernel (the reference does so only on its
    `use_cuda` path, mamba.py:259-260)."""
    d_model: int
    n_layers: int
    dt_rank: Union[int, str] = "auto"
    d_state: int = 16
    expand_factor: int = 2
    d_conv: int = 4

    dt_min: float = 0.001
    dt_max: float = 0.1
    dt_init: str = "random"
    dt_scale: float = 1.0
    dt_init_floor: float = 1e-4

    rms_norm_eps: float = 1e-5
    base_std: float = 0.02

    bias: bool = False
    conv_bias: bool = True
    inner_layernorms: bool = False

    mup: bool = False
    mup_base_width: float = 128

    pscan: bool = True
    use_cuda: bool = False
    fused_softplus: bool = True

    def __post_init__(self):
        self.d_inner = self.expand_factor * self.d_model
        if self.dt_rank == "auto":
            self.dt_rank = math.ceil(self.d_model / 16)
        if self.mup:
            self.mup_width_mult = self.d_model / self.mup_base_width


# x_proj / dt_proj run on zero-padded copies of their weights where that gives the GEMM library better
# tile shapes (see MambaBlock._padded_projections); False runs them on the parameters as they are
PAD_PROJECTIONS = True


def _frozen_f32(owner, key, p, fn=None):
    """float32 form of a small parameter (optionally fn(parameter)) for the kernels that take
    float32 constants.  Inside autograd the parameter itself is returned and the conversion is
    part of the graph.  Outside it (decode, prefill) the converted value is kept in one
    persistent buffer per (module, key) that is refreshed in place when the parameter has
    changed: a forward pass then spends no kernels on these conversions and a captured HIP graph
    keeps reading the same memory."""
    if p is None:
        return None
    if torch.is_grad_enabled() and p.requires_grad:
        return p if fn is None else fn(p)
    if fn is None and p.dtype == torch.float32:
        return p
    cache = owner.__dict__.setdefault("_f32_cache", {})
    tag = (p._version, p.data_ptr(), p.device, p.dtype)
    hit = cache.get(key)
    if hit is None or hit[0] != tag:
        with torch.no_grad():
            fresh = p.detach().float() if fn is None else fn(p.detach())
            if hit is not None and hit[1].shape == fresh.shape and hit[1].device == fresh.device \
                    and hit[1].dtype == fresh.dtype:
                hit[1].copy_(fresh)
                fresh = hit[1]
        cache[key] = (tag, fresh)
    return cache[key][1]


class RMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) [* weight]  (mambapy/mamba.py:416-433; no gain under muP)."""

    def __init__(self, d_model: int, eps: float = 1e-5, use_mup: bool = False):
        super().__init__()
        self.eps = eps
        self.use_mup = use_mup
        if not use_mup:
            self.weight = nn.Parameter(torch.ones(d_model))

    def _w(self):
        return None if self.use_mup else _frozen_f32(self, "weight", self.weight)

    def forward(self, x):
        if x.is_cuda and rmsnorm_supported(x):
            return rmsnorm_fn(x, self._w(), self.eps)
        y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps)
        return y if self.use_mup else y * self.weight

    def add_norm(self, x, residual):
        """(norm(x + residual), x + residual); the add rides in the norm kernel when it can."""
        if residual is None:
            return self(x), x
        if x.is_cuda and rmsnorm_supported(x) and residual.dtype == x.dtype:
            return add_rmsnorm_fn(x, residual, self._w(), self.eps)
        total = x + residual
        return self(total), total


class MambaBlock(nn.Module):
    """The mixer of mambapy/mamba.py:127-414 with the scan replaced by the HIP kernels.

    Parameters (state_dict keys): in_proj.weight, conv1d.weight (ED,1,d_conv), conv1d.bias,
    x_proj.weight, dt_proj.weight, dt_proj.bias, A_log (ED,N), D (ED), out_proj.weight.
    """

    def __init__(self, config: MambaConfig):
        super().__init__()
        self.config = config
        ED, N, R = config.d_inner, config.d_state, config.dt_rank
        self.in_proj = nn.Linear(config.d_model, 2 * ED, bias=config.bias)
        self.conv1d = nn.Conv1d(ED, ED, kernel_size=config.d_conv, groups=ED,
                                padding=config.d_conv - 1, bias=config.conv_bias)
        self.x_proj = nn.Linear(ED, R + 2 * N, bias=False)
        self.dt_proj = nn.Linear(R, ED, bias=True)
        self.out_proj = nn.Linear(ED, config.d_model, bias=config.bias)

        # initial values as in mamba.py:147-172: dt_proj.weight uniform or constant,
        # dt_proj.bias = inverse softplus of a log-uniform step in [dt_min, dt_max],
        # A = -(1..N) per channel stored as log (S4D-real), D = 1
        bound = R ** -0.5 * config.dt_scale
        if config.dt_init == "constant":
            nn.init.constant_(self.dt_proj.weight, bound)
        elif config.dt_init == "random":
            nn.init.uniform_(self.dt_proj.weight, -bound, bound)
        else:
            raise NotImplementedError(f"dt_init={config.dt_init!r}")
        lo, hi = math.log(config.dt_min), math.log(config.dt_max)
        dt = torch.exp(torch.rand(ED) * (hi - lo) + lo).clamp(min=config.dt_init_floor)
        with torch.no_grad():
            self.dt_proj.bias.copy_(dt + torch.log(-torch.expm1(-dt)))
        self.A_log = nn.Parameter(torch.log(torch.arange(1, N + 1, dtype=torch.float32)).repeat(ED, 1))
        self.A_log._no_weight_decay = True
        self.D = nn.Parameter(torch.ones(ED))
        self.D._no_weight_decay = True

        if config.inner_layernorms:
            self.dt_layernorm = RMSNorm(R, config.rms_norm_eps, config.mup)
            self.B_layernorm = RMSNorm(N, config.rms_norm_eps, config.mup)
            self.C_layernorm = RMSNorm(N, config.rms_norm_eps, config.mup)
        else:
            self.dt_layernorm = self.B_layernorm = self.C_layernorm = None

    # -- helpers -------------------------------------------------------------------------
    def _split_projection(self, dbc):
        R, N = self.config.dt_rank, self.config.d_state
        dlow, Bm, C = torch.split(dbc, [R, N, N], dim=-1)
        if self.dt_layernorm is not None:
            dlow, Bm, C = self.dt_layernorm(dlow), self.B_layernorm(Bm), self.C_layernorm(C)
        return dlow, Bm, C

    def _A(self):
        """A = -exp(A_log) in float32 (mambapy/mamba.py:239)."""
        return _frozen_f32(self, "A", self.A_log, lambda t: -torch.exp(t.float()))

    def _D(self):
        return _frozen_f32(self, "D", self.D)

    def _dt_bias(self):
        return _frozen_f32(self, "dt_bias", self.dt_proj.bias)

    def _padded_projections(self):
        """x_proj and dt_proj weights in the shape the GEMM library serves best, or None when the
        layer's own shapes already are.  The low-rank width R = dt_rank (48 at d_model 768) is the K of
        dt_proj and R + 2N (80) the N of x_proj; both land on generic tiles.  With R rounded up to a
        multiple of 64 by zero columns, and the rows of x_proj regrouped as [delta rows | zeros up to
        the rounded width | B rows | C rows | zeros up to a multiple of 64], the two products cost
        21 + 26 us instead of 25 + 38 us at (8 x 4096) x 1536 in bfloat16, and the low-rank input of
        dt_proj is a view of the x_proj output as before.  The parameters keep the reference's shapes
        (state_dict keys x_proj.weight (R + 2N, ED), dt_proj.weight (ED, R)); the padded forms are
        derived from them (inside autograd as part of the graph, outside it cached)."""
        R, N = self.config.dt_rank, self.config.d_state
        Rp = -(-R // 64) * 64
        if Rp == R or self.dt_layernorm is not None or not PAD_PROJECTIONS:
            return None
        rows = -(-(Rp + 2 * N) // 64) * 64

        def pad_x(w):
            out = w.new_zeros(rows, w.shape[1])
            out[:R] = w[:R]
            out[Rp:Rp + 2 * N] = w[R:]
            return out

        def pad_dt(w):
            return F.pad(w, (0, Rp - R))
        return (_frozen_f32(self, "x_proj_padded", self.x_proj.weight, pad_x),
                _frozen_f32(self, "dt_proj_padded", self.dt_proj.weight, pad_dt), Rp)

    def _conv_wb(self):
        return (_frozen_f32(self, "conv_w", self.conv1d.weight), _frozen_f32(self, "conv_b", self.conv1d.bias))

    # -- training / prefill ---------------------------------------------------------------
    def forward(self, x, cache: Optional[Tuple] = None, return_cache: bool = False):
        """x : (B, L, D) -> (B, L, D).  With return_cache=True also returns the decode cache
        (h (B,ED,N) float32, inputs (B,ED,d_conv-1)) after the last position, so that
        generation can continue with step() instead of re-running the sequence.  `cache` (the
        same pair, from an earlier call or from step(); h may be None) is what the sequence
        continues from: the state before position 0 and the inputs before it.  No gradient
        flows into the cache."""
        L = x.shape[1]
        xz = self.in_proj(x)
        xin, z = xz.chunk(2, dim=-1)
        K = self.config.d_conv
        h_in, win_in = cache if cache is not None else (None, None)
        window = None
        if 2 <= K <= 4:
            # causal depthwise convolution + bias + silu in one kernel, reading the x half of
            # the projection in place (no transposes) and returning the decode window
            cw, cb = self._conv_wb()
            if return_cache:
                xs, window = causal_conv1d_fn(xin, cw, cb, window=win_in, return_window=True)
            else:
                xs = causal_conv1d_fn(xin, cw, cb, window=win_in)
        else:
            pre = xin.transpose(1, 2)                        # (B, ED, L)
            if win_in is not None:
                full = torch.cat([win_in.detach().to(pre.dtype), pre], dim=2)
                xc = F.conv1d(full, self.conv1d.weight, self.conv1d.bias, groups=self.config.d_inner)
            else:
                full = F.pad(pre, (K - 1, 0))
                xc = self.conv1d(pre)[:, :, :L]
            xs = F.silu(xc).transpose(1, 2)                  # (B, L, ED), unit stride along L
            if return_cache:
                window = full[:, :, full.shape[2] - (K - 1):].detach().contiguous()
        h0 = None if h_in is None else h_in.detach()
        # the gate y * silu(z) is applied inside the scan kernel (z is read in place)
        if return_cache:
            y, h_last = self.ssm(xs, z, return_last_state=True, h0=h0)
        else:
            y = self.ssm(xs, z, h0=h0)
        out = self.out_proj(y)
        if not return_cache:
            return out
        return out, (h_last, window)

    def ssm(self, x, z=None, return_last_state: bool = False, h0=None):
        """(B, L, ED) -> (B, L, ED): projections to (delta, B, C), then the fused scan
        (mambapy/mamba.py:236-272); with z the result is already gated, y * silu(z), as on the
        reference's fused path (mamba.py:259-260, 225-227)."""
        A, D = self._A(), self._D()
        padded = self._padded_projections() if x.is_cuda else None
        if padded is None:
            dlow, Bm, C = self._split_projection(self.x_proj(x))
            # (B, L, ED) with unit stride along ED, the layout of x: the reference forms the transposed
            # product (mamba.py:247) only because its fused backend wants (B, ED, L)
            delta = F.linear(dlow, self.dt_proj.weight)
        else:
            wx, wdt, Rp = padded
            N = self.config.d_state
            dbc = F.linear(x, wx)
            Bm, C = dbc[..., Rp:Rp + N], dbc[..., Rp + N:Rp + 2 * N]
            delta = F.linear(dbc[..., :Rp], wdt)     # the zero columns meet the zero rows
        if self.config.fused_softplus:
            return selective_scan_fn(x, delta, A, Bm, C, D, z=z, delta_bias=self._dt_bias(),
                                     delta_softplus=True, h0=h0, return_last_state=return_last_state)
        delta = F.softplus(delta + self.dt_proj.bias)
        return selective_scan_fn(x, delta, A, Bm, C, D, z=z, h0=h0, return_last_state=return_last_state)

    def selective_scan(self, x, delta, A, B, C, D):
        """Same call as MambaBlock.selective_scan (mambapy/mamba.py:274-295)."""
        return selective_scan(x, delta, A, B, C, D)

    def selective_scan_seq(self, x, delta, A, B, C, D):
        """The reference keeps a sequential twin (mamba.py:297-327); both names run the same
        kernel here."""
        return selective_scan(x, delta, A, B, C, D)

    # -- decode -----------------------------------------------------------------------------
    def step(self, x, cache):
        """x : (B, D), cache = (h (B,ED,N) or None, inputs (B,ED,d_conv-1)) ->
        (y (B, D), new cache); mambapy/mamba.py:351-382.  The old cache tuple stays valid."""
        h, inputs = cache
        xz = self.in_proj(x)
        xin, z = xz.chunk(2, dim=1)
        if 2 <= self.config.d_conv <= 4 and not torch.is_grad_enabled():
            # convolution over (cache, newest input) + bias + silu and the new cache: one kernel
            xs, window = causal_conv1d_fn(xin.unsqueeze(1), *self._conv_wb(), window=inputs, return_window=True)
            xs = xs[:, 0]
        else:
            full = torch.cat([inputs, xin.unsqueeze(2)], dim=2)          # (B, ED, d_conv)
            xc = (full * self.conv1d.weight[:, 0, :]).sum(-1)
            if self.conv1d.bias is not None:
                xc = xc + self.conv1d.bias
            xs, window = F.silu(xc), full[:, :, 1:]
        y, h = self.ssm_step(xs, h, z=z)
        out = self.out_proj(y)
        return out, (h, window)

    def ssm_step(self, x, h, z=None, inplace: bool = False):
        """x : (B, ED), h : (B, ED, N) or None -> (y, h'); mambapy/mamba.py:384-414.  With z
        the gate y*silu(z) is applied inside the kernel; inplace=True updates h itself."""
        dlow, Bm, C = self._split_projection(self.x_proj(x))
        raw = F.linear(dlow, self.dt_proj.weight)                        # bias added in-kernel
        y, h_new = ssm_step(x, raw, self._A(), Bm, C, self._D(), h, z=z,
                            delta_bias=self._dt_bias(), delta_softplus=True, inplace=inplace)
        return y, h_new

    def step_(self, x, h, window):
        """In-place decode step for loops that must not allocate new cache tensors (HIP graph
        replay): x (B, D); h (B, ED, N) float32 and window (B, ED, d_conv-1) are updated in
        place.  Same arithmetic as step()."""
        xz = self.in_proj(x)
        xin, z = xz.chunk(2, dim=1)
        if 2 <= self.config.d_conv <= 4 and window.is_contiguous() and window.dtype == xin.dtype:
            xs = causal_conv1d_update(xin, window, *self._conv_wb())
        else:
            full = torch.cat([window, xin.unsqueeze(2)], dim=2)          # (B, ED, d_conv)
            xc = (full * self.conv1d.weight[:, 0, :]).sum(-1)
            if self.conv1d.bias is not None:
                xc = xc + self.conv1d.bias
            xs = F.silu(xc)
            window.copy_(full[:, :, 1:])
        y, _ = self.ssm_step(xs, h, z=z, inplace=True)
        return self.out_proj(y)


class ResidualBlock(nn.Module):
    """mixer(norm(x)) + x  (mambapy/mamba.py:99-125); keys: mixer.*, norm.weight."""

    def __init__(self, config: MambaConfig):
        super().__init__()
        self.mixer = MambaBlock(config)
        self.norm = RMSNorm(config.d_model, config.rms_norm_eps, config.mup)

    def forward(self, x, cache: Optional[Tuple] = None, return_cache: bool = False):
        if return_cache:
            y, cache = self.mixer(self.norm(x), cache=cache, return_cache=True)
            return y + x, cache
        return self.mixer(self.norm(x), cache=cache) + x

    def step(self, x, cache):
        y, cache = self.mixer.step(self.norm(x), cache)
        return y + x, cache

    def step_(self, x, h, window):
        return self.mixer.step_(self.norm(x), h, window) + x


class Mamba(nn.Module):
    """Stack of residual blocks (mambapy/mamba.py:69-97); keys: layers.{i}.*"""

    def __init__(self, config: MambaConfig):
        super().__init__()
        self.config = config
        self.layers = nn.ModuleList([ResidualBlock(config) for _ in range(config.n_layers)])

    def forward(self, x, caches=None, return_caches: bool = False):
        """x : (B, L, D) -> (B, L, D) [, caches].  `caches` (one (h, inputs) pair per layer, as
        returned by an earlier call with return_caches=True, by step() or by empty_caches()) makes
        the call continue that sequence."""
        # Same arithmetic as x = layer(x) for every layer, in another order of kernels: the add
        # that ends layer i is done by the norm kernel that starts layer i+1 (pre-norm
        # residual stream: `hidden` is the last mixer output, `residual` the running sum).
        hidden, residual = x, None
        new_caches = []
        for i, layer in enumerate(self.layers):
            normed, residual = layer.norm.add_norm(hidden, residual)
            cache = None if caches is None else caches[i]
            if return_caches:
                hidden, c = layer.mixer(normed, cache=cache, return_cache=True)
                new_caches.append(c)
            else:
                hidden = layer.mixer(normed, cache=cache)
        x = hidden + residual if self.layers else x
        return (x, new_caches) if return_caches else x

    def step(self, x, caches):
        hidden, residual = x, None
        for i, layer in enumerate(self.layers):
            normed, residual = layer.norm.add_norm(hidden, residual)
            hidden, caches[i] = layer.mixer.step(normed, caches[i])
        return (hidden + residual if self.layers else x), caches

    def step_(self, x, caches):
        """In-place variant of step(): every (h, window) pair of `caches` is updated in place
        (h must be a float32 tensor, not None)."""
        hidden, residual = x, None
        for layer, (h, window) in zip(self.layers, caches):
            normed, residual = layer.norm.add_norm(hidden, residual)
            hidden = layer.mixer.step_(normed, h, window)
        return hidden + residual if self.layers else x

    def empty_caches(self, batch: int, device=None, dtype=None):
        """Fresh decode caches: h = None (zero state), zero conv window (mamba.py:344-346)."""
        cfg = self.config
        p = self.layers[0].mixer.in_proj.weight
        device = device or p.device
        dtype = dtype or p.dtype
        return [(None, torch.zeros(batch, cfg.d_inner, cfg.d_conv - 1, device=device, dtype=dtype))
                for _ in self.layers]
