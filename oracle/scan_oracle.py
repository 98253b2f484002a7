"""CPU oracle for the selective-scan hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it is the checker used by
tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.  The
product path is the HIP library and fails loudly when that library is missing.

Every function restates, in this build's own code, an algorithm of the reference and
names the lines it follows.  What pins each function (see tests/test_oracle.py):

  linear_recurrence      definition H[t] = A[t]*H[t-1] + X[t], H[-1] = 0
                         (mambapy/pscan.py:41-44).  Pinned by the reference's literal
                         cumulative-sum vectors (docs/pscan.ipynb cells 5/8/11,
                         docs/tests.ipynb cell 1), by the closed form
                         (1-a^(t+1))/(1-a), by the brute-force double sum on tiny
                         inputs and by chunk-split consistency.
  blelloch_scan[_rev]    up-sweep / down-sweep tree of mambapy/pscan.py:36-92 and its
                         mirror image :94-149.  Pinned by the up-sweep-only vector of
                         docs/pscan.ipynb cell 43, by equality with linear_recurrence
                         and by rev == flip . fwd . flip (pscan.py:99-101).
  BlellochPScan          forward/backward of mambapy/pscan.py:151-224 (padding to a
                         power of two, shifted-A reverse scan, gradA[t]=H[t-1]*gradX[t]).
                         Pinned against fp64 autograd through linear_recurrence.
  selective_scan_ref     mambapy/mamba.py:274-327 (discretise, scan, readout).  Pinned
                         by the special cases delta=0, C=0, A=0 (closed forms) and by
                         the brute-force sum; its gradients are plain torch autograd
                         (checked with torch.autograd.gradcheck).
  ssm_step_ref           mambapy/mamba.py:400-412.  Pinned by "L steps == one scan".
  conv_window_step_ref   mambapy/mamba.py:366-367, 379.  Pinned against
                         torch.nn.functional.conv1d with left zero padding.
  causal_conv1d_ref      mambapy/mamba.py:217-221.  Pinned against the definition written
                         as explicit loops on small cases and against nn.Conv1d with
                         padding=K-1 truncated to L (the reference's own expression).
  rmsnorm_ref            mambapy/mamba.py:427-433.  Pinned by a hand-computed vector
                         ([3,4] -> [3,4]/sqrt(12.5)), by explicit loops, by unit mean
                         square of the output rows at eps=0 and by invariance to a
                         rescaling of the input row at eps=0.

Floating-point rounding of torch's own elementwise kernels is not pinned by any
reference fixture ("parity unpinned" at the torch boundary; irrelevant at the
tolerances used: these are IEEE elementwise operations).
"""

import math

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------
# scan primitive
# --------------------------------------------------------------------------------------

def next_pow2(length: int) -> int:
    """Smallest power of two >= length (mambapy/pscan.py:13-18)."""
    p = 1
    while p < length:
        p *= 2
    return p


def linear_recurrence(A: torch.Tensor, X: torch.Tensor, h0: torch.Tensor = None) -> torch.Tensor:
    """H[:, t] = A[:, t] * H[:, t-1] + X[:, t] over dim 1, H[:, -1] = h0 (zero by default).

    The definition the reference's scan computes (mambapy/pscan.py:41-44) and that its
    own sequential loop spells out (mambapy/mamba.py:314-321).  Differentiable by
    plain autograd.  A, X : (B, L, ...).
    """
    h = torch.zeros_like(X[:, 0]) if h0 is None else h0
    out = []
    for t in range(X.shape[1]):
        h = A[:, t] * h + X[:, t]
        out.append(h)
    return torch.stack(out, dim=1)


def linear_recurrence_bruteforce(A: torch.Tensor, X: torch.Tensor) -> torch.Tensor:
    """H[t] = sum_{s<=t} (prod_{r=s+1..t} A[r]) * X[s]; O(L^2), tiny inputs only."""
    L = X.shape[1]
    H = torch.zeros_like(X)
    for t in range(L):
        for s in range(t + 1):
            w = torch.ones_like(X[:, 0])
            for r in range(s + 1, t + 1):
                w = w * A[:, r]
            H[:, t] += w * X[:, s]
    return H


def blelloch_upsweep_(A: torch.Tensor, X: torch.Tensor, reverse: bool = False) -> None:
    """In-place reduction tree over dim 1 (length a power of two).

    Level with stride s combines node pairs (left, right) that are s apart:
    X_r += A_r * X_l ; A_r *= A_l (mambapy/pscan.py:54-75), or the mirror image for the
    reverse scan (:111-132).  After the call the last (first, if reverse) element holds
    the full combination; the other tree nodes hold partial results.
    """
    L = X.shape[1]
    s = 1
    while s < L:
        if not reverse:
            dst, src = slice(2 * s - 1, L, 2 * s), slice(s - 1, L, 2 * s)
        else:
            dst, src = slice(0, L, 2 * s), slice(s, L, 2 * s)
        X[:, dst] += A[:, dst] * X[:, src]
        A[:, dst] *= A[:, src]
        s *= 2


def blelloch_downsweep_(A: torch.Tensor, X: torch.Tensor, reverse: bool = False) -> None:
    """In-place distribution phase (mambapy/pscan.py:78-92; mirror image :135-149).

    At stride s the nodes at odd multiples of s (3s-1, 5s-1, ...) receive the prefix
    that ends s positions before them.
    """
    L = X.shape[1]
    s = L // 4
    while s >= 1:
        if not reverse:
            dst, src = slice(3 * s - 1, L, 2 * s), slice(2 * s - 1, L - s, 2 * s)
        else:
            dst, src = slice(s, L - 2 * s, 2 * s), slice(2 * s, L - s, 2 * s)
        X[:, dst] += A[:, dst] * X[:, src]
        A[:, dst] *= A[:, src]
        s //= 2


def blelloch_scan_(A: torch.Tensor, X: torch.Tensor, reverse: bool = False) -> None:
    """In-place Blelloch scan of (B, L, D, N) tensors along dim 1, L a power of two.

    Forward: X[t] <- A[t] X[t-1] + X[t].  Reverse: X[t] <- X[t] + A[t] X[t+1].
    A is destroyed (holds partial products), as in mambapy/pscan.py:36-149.
    """
    L = X.shape[1]
    assert L == next_pow2(L), "length must be a power of two (mambapy/pscan.py:46)"
    blelloch_upsweep_(A, X, reverse)
    blelloch_downsweep_(A, X, reverse)


def pad_pow2(T: torch.Tensor) -> torch.Tensor:
    """Zero-pad dim 1 of (B, L, D, N) to the next power of two; always returns a copy
    (mambapy/pscan.py:20-33, 168-174)."""
    L = T.shape[1]
    P = next_pow2(L)
    if P == L:
        return T.clone()
    return F.pad(T, (0, 0, 0, 0, 0, P - L))


class BlellochPScan(torch.autograd.Function):
    """CPU restatement of the reference's differentiable scan (mambapy/pscan.py:151-224).

    forward : H = scan(A, X) on padded copies, returns H[:, :L].
    backward: gradX = reverse scan of the incoming gradient with A shifted one step to
              the left (zero at the end, :216); gradA[t] = H[t-1] * gradX[t], gradA[0] = 0
              (:221-222).
    """

    @staticmethod
    def forward(ctx, A_in, X_in):
        L = X_in.shape[1]
        A = pad_pow2(A_in)
        H = pad_pow2(X_in)
        blelloch_scan_(A, H)
        ctx.save_for_backward(A_in, H)
        ctx.L = L
        return H[:, :L].clone()

    @staticmethod
    def backward(ctx, grad_out):
        A_in, H = ctx.saved_tensors
        L = ctx.L
        G = pad_pow2(grad_out)
        A_shift = torch.zeros_like(H)
        A_shift[:, : L - 1] = A_in[:, 1:L]
        blelloch_scan_(A_shift, G, reverse=True)
        gradA = torch.zeros_like(H)
        gradA[:, 1:] = H[:, :-1] * G[:, 1:]
        return gradA[:, :L], G[:, :L]


def pscan_blelloch(A: torch.Tensor, X: torch.Tensor) -> torch.Tensor:
    """Differentiable Blelloch scan with the call shape of `pscan` (mambapy/pscan.py:226)."""
    return BlellochPScan.apply(A, X)


# --------------------------------------------------------------------------------------
# selective scan
# --------------------------------------------------------------------------------------

def discretise(x, delta, A, B):
    """deltaA = exp(delta * A) (zero-order hold) and BX = delta * B * x (Euler), both
    (B, L, ED, N) (mambapy/mamba.py:284-287)."""
    deltaA = torch.exp(delta.unsqueeze(-1) * A)
    BX = delta.unsqueeze(-1) * B.unsqueeze(2) * x.unsqueeze(-1)
    return deltaA, BX


def selective_scan_ref(x, delta, A, B, C, D, h0=None, return_last_state=False):
    """y = C . h + D x with h_t = exp(delta_t A) h_{t-1} + delta_t B_t x_t
    (mambapy/mamba.py:297-327, the reference's own sequential ground truth).

    x, delta : (B, L, ED); A : (ED, N); B, C : (B, L, N); D : (ED).  Run it in float64.
    """
    deltaA, BX = discretise(x, delta, A, B)
    hs = linear_recurrence(deltaA, BX, h0)
    y = (hs * C.unsqueeze(2)).sum(-1) + D * x
    if return_last_state:
        return y, hs[:, -1]
    return y


def selective_scan_blelloch(x, delta, A, B, C, D):
    """The reference's parallel-scan path (mambapy/mamba.py:274-295) on the CPU:
    materialised (B, L, ED, N) tensors, Blelloch scan, batched readout.  This is the
    "port" that bench.py times as cpu_baseline."""
    deltaA, BX = discretise(x, delta, A, B)
    hs = pscan_blelloch(deltaA, BX)
    y = (hs @ C.unsqueeze(-1)).squeeze(3)
    return y + D * x


def selective_scan_bruteforce(x, delta, A, B, C, D):
    """y[b,t,d] = sum_n C[b,t,n] sum_{s<=t} exp(A[d,n] sum_{r=s+1..t} delta[b,r,d])
    * delta[b,s,d] B[b,s,n] x[b,s,d] + D[d] x[b,t,d].  Closed-form product of the
    decays (prod exp = exp sum); tiny inputs only."""
    Bs, L, ED = x.shape
    y = torch.zeros_like(x)
    for t in range(L):
        for s in range(t + 1):
            dsum = delta[:, s + 1 : t + 1].sum(1)                       # (B, ED)
            w = torch.exp(dsum.unsqueeze(-1) * A)                       # (B, ED, N)
            contrib = w * (delta[:, s] * x[:, s]).unsqueeze(-1) * B[:, s].unsqueeze(1)
            y[:, t] += (contrib * C[:, t].unsqueeze(1)).sum(-1)
        y[:, t] += D * x[:, t]
    return y


def selective_scan_grads_autograd(x, delta, A, B, C, D, dy, chunk=None):
    """fp64 forward + gradients by plain autograd through selective_scan_ref.

    Inputs of any float dtype are promoted to float64 first.  `chunk` splits the channel
    dimension (channels are independent; dB and dC are summed over chunks) to bound
    memory.  Returns dict(y, dx, ddelta, dA, dB, dC, dD) in float64.
    """
    f64 = lambda t: t.detach().to(torch.float64)
    x, delta, A, B, C, D, dy = map(f64, (x, delta, A, B, C, D, dy))
    ED = x.shape[2]
    chunk = ED if chunk is None else chunk
    out = dict(y=torch.empty_like(x), dx=torch.empty_like(x), ddelta=torch.empty_like(x),
               dA=torch.empty_like(A), dB=torch.zeros_like(B), dC=torch.zeros_like(C),
               dD=torch.empty_like(D))
    for lo in range(0, ED, chunk):
        sl = slice(lo, min(lo + chunk, ED))
        xs = x[:, :, sl].clone().requires_grad_()
        ds = delta[:, :, sl].clone().requires_grad_()
        As = A[sl].clone().requires_grad_()
        Ds = D[sl].clone().requires_grad_()
        Bs = B.clone().requires_grad_()
        Cs = C.clone().requires_grad_()
        y = selective_scan_ref(xs, ds, As, Bs, Cs, Ds)
        y.backward(dy[:, :, sl])
        out["y"][:, :, sl] = y.detach()
        out["dx"][:, :, sl] = xs.grad
        out["ddelta"][:, :, sl] = ds.grad
        out["dA"][sl] = As.grad
        out["dD"][sl] = Ds.grad
        out["dB"] += Bs.grad
        out["dC"] += Cs.grad
    return out


# --------------------------------------------------------------------------------------
# decode step
# --------------------------------------------------------------------------------------

def ssm_step_ref(x, delta, A, B, C, D, h=None):
    """One token of the recurrence (mambapy/mamba.py:400-412), delta already softplus'ed.

    x, delta : (B, ED); A : (ED, N); B, C : (B, N); D : (ED); h : (B, ED, N) or None (= 0).
    Returns (y (B, ED), h_new (B, ED, N)); h is not modified.
    """
    deltaA = torch.exp(delta.unsqueeze(-1) * A)
    BX = delta.unsqueeze(-1) * B.unsqueeze(1) * x.unsqueeze(-1)
    if h is None:
        h = torch.zeros_like(BX)
    h_new = deltaA * h + BX
    y = (h_new * C.unsqueeze(1)).sum(-1) + D * x
    return y, h_new


def conv_window_step_ref(window, x_new, weight, bias):
    """Depthwise causal conv for one new token with a rolling window of the last
    d_conv-1 pre-conv inputs (mambapy/mamba.py:366-367, 379).

    window : (B, ED, K-1); x_new : (B, ED); weight : (ED, 1, K); bias : (ED) or None.
    Returns (conv_out (B, ED), new_window (B, ED, K-1)).
    """
    full = torch.cat([window, x_new.unsqueeze(2)], dim=2)               # (B, ED, K)
    out = (full * weight[:, 0, :].unsqueeze(0)).sum(-1)
    if bias is not None:
        out = out + bias
    return out, full[:, :, 1:].clone()


def causal_conv1d_ref(x, weight, bias=None, window=None, silu=True):
    """Depthwise causal convolution along time as MambaBlock.forward applies it
    (mambapy/mamba.py:217-221): conv1d(x^T, padding=K-1)[:, :, :L]^T, then silu (:221).

    x : (B, L, ED); weight : (ED, 1, K); bias : (ED) or None; window : optional (B, ED, K-1)
    inputs that precede step 0 (the reference pads with zeros; the decode cache of
    mamba.py:344-346 is the non-zero case).  Returns (B, L, ED).
    """
    K = weight.shape[-1]
    xt = x.transpose(1, 2)                                            # (B, ED, L)
    left = window if window is not None else xt.new_zeros(xt.shape[0], xt.shape[1], K - 1)
    y = F.conv1d(torch.cat([left.to(xt.dtype), xt], dim=2), weight, bias, groups=xt.shape[1])
    y = y.transpose(1, 2)
    return F.silu(y) if silu else y


def rmsnorm_ref(x, weight=None, eps=1e-5):
    """x * rsqrt(mean(x^2, last axis) + eps) [* weight]  (mambapy/mamba.py:427-433;
    no weight under muP, :421-424)."""
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def softplus_ref(v):
    """log(1 + exp(v)), overflow-safe (torch.nn.functional.softplus, mamba.py:265, 398)."""
    return torch.where(v > 20, v, torch.log1p(torch.exp(torch.clamp(v, max=20))))


# --------------------------------------------------------------------------------------
# seeded synthetic inputs: the recipe lives in the neutral module synthetic_inputs.py (the
# benchmark and smoke() take their inputs from there, not from the checker); re-exported
# here because every parity test draws its inputs through this module
# --------------------------------------------------------------------------------------
import os as _os
import sys as _sys

_sys.path.insert(0, _os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))))
from synthetic_inputs import make_inputs  # noqa: E402,F401
