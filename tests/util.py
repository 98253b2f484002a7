"""Shared helpers of the parity tests."""
import torch


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max |got - ref| / max |ref| per tensor: the error measure of every parity test
    (element-wise relative error is meaningless next to zeros)."""
    ref = ref.detach().double().cpu()
    got = got.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


# tolerances stated by the task: float32 I/O 1e-4, bfloat16 I/O (float32 state) 2e-2
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}

GRAD_KEYS = ("dx", "ddelta", "dA", "dB", "dC", "dD")


def run_gpu_fwd_bwd(pkg, inp, dev, **kw):
    """Forward + backward of the fused scan on the GPU; returns dict like the oracles."""
    names = ("x", "delta", "A", "B", "C", "D")
    args = [inp[k].to(dev).requires_grad_() for k in names]
    y = pkg.selective_scan_fn(*args, **kw)
    y.backward(inp["dy"].to(dev))
    torch.cuda.synchronize()
    out = dict(y=y.detach())
    for k, a in zip(GRAD_KEYS, args):
        out[k] = a.grad
    return out
