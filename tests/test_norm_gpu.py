"""GPU parity of the RMSNorm kernel against the float64 oracle (mambapy/mamba.py:427-433)."""
import pytest
import torch

from oracle import scan_oracle as so
from util import TOL, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,dtype,with_w", [
    ((2, 37, 768), torch.float32, True), ((3, 5, 64), torch.float32, True), ((1, 1, 8), torch.bfloat16, True),
    ((2, 129, 2560), torch.bfloat16, True), ((4, 33, 2048), torch.float32, False), ((7, 4096), torch.bfloat16, True),
    ((5, 3, 4), torch.float32, True),
])
def test_rmsnorm_forward_backward(pkg, dev, shape, dtype, with_w):
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 1.5 + 0.3).to(dtype)
    w = (torch.randn(shape[-1], generator=g) * 0.5 + 1.0).to(dtype) if with_w else None
    dy = torch.randn(*shape, generator=g).to(dtype)
    eps = 1e-5
    xr = x.double().requires_grad_()
    wr = None if w is None else w.double().requires_grad_()
    yr = so.rmsnorm_ref(xr, wr, eps)
    yr.backward(dy.double())
    xg = x.to(dev).requires_grad_()
    wg = None if w is None else w.to(dev).requires_grad_()
    y = pkg.rmsnorm_fn(xg, wg, eps)
    y.backward(dy.to(dev))
    tol = TOL[dtype]
    assert rel_err(y, yr) <= tol
    assert rel_err(xg.grad, xr.grad) <= tol
    if w is not None:
        assert rel_err(wg.grad, wr.grad) <= tol


def test_rmsnorm_module_uses_kernel_and_matches(pkg, dev):
    torch.manual_seed(3)
    norm = pkg.RMSNorm(96).to(dev)
    with torch.no_grad():
        norm.weight.mul_(torch.rand(96, device=dev) + 0.5)
    x = torch.randn(4, 10, 96, device=dev)
    want = so.rmsnorm_ref(x.double(), norm.weight.double(), norm.eps)
    assert rel_err(norm(x), want) <= TOL[torch.float32]
    # an unsupported width falls back to the same formula on PyTorch kernels
    norm2 = pkg.RMSNorm(10).to(dev)
    x2 = torch.randn(3, 10, device=dev)
    assert rel_err(norm2(x2), so.rmsnorm_ref(x2.double(), norm2.weight.double(), norm2.eps)) <= TOL[torch.float32]


@pytest.mark.parametrize("shape,dtype,with_w", [
    ((2, 37, 768), torch.float32, True), ((3, 5, 64), torch.bfloat16, True), ((19, 2048), torch.float32, False),
    ((2, 70, 1536), torch.bfloat16, True),
])
def test_add_rmsnorm_forward_backward(pkg, dev, shape, dtype, with_w):
    # (norm(x + r), x + r) with both outputs used downstream: the gradient of x and of r is the
    # gradient through the norm plus the one that reaches the sum directly
    g = torch.Generator().manual_seed(7 + sum(shape))
    x = (torch.randn(*shape, generator=g) * 1.5).to(dtype)
    r = (torch.randn(*shape, generator=g) + 0.2).to(dtype)
    w = (torch.randn(shape[-1], generator=g) * 0.5 + 1.0).to(dtype) if with_w else None
    dy = torch.randn(*shape, generator=g).to(dtype)
    dt = torch.randn(*shape, generator=g).to(dtype)
    xr, rr = x.double().requires_grad_(), r.double().requires_grad_()
    wr = None if w is None else w.double().requires_grad_()
    # the kernel rounds the sum to the I/O type before it normalises it (as a separate add would)
    tr = xr + rr
    tr_q = tr + (tr.detach().to(dtype).double() - tr.detach())
    yr = so.rmsnorm_ref(tr_q, wr, 1e-5)
    (yr * dy.double()).sum().add((tr_q * dt.double()).sum()).backward()
    xg, rg = x.to(dev).requires_grad_(), r.to(dev).requires_grad_()
    wg = None if w is None else w.to(dev).requires_grad_()
    y, total = pkg.add_rmsnorm_fn(xg, rg, wg, 1e-5)
    torch.autograd.backward([y, total], [dy.to(dev), dt.to(dev)])
    tol = TOL[dtype]
    assert torch.equal(total.cpu(), (x.double() + r.double()).to(dtype))   # one rounding of the exact sum
    assert rel_err(y, yr) <= tol
    assert rel_err(xg.grad, xr.grad) <= tol and rel_err(rg.grad, rr.grad) <= tol
    if w is not None:
        assert rel_err(wg.grad, wr.grad) <= tol
    # only the normalised output used: no gradient reaches the sum directly
    xg2, rg2 = x.to(dev).requires_grad_(), r.to(dev).requires_grad_()
    y2, _ = pkg.add_rmsnorm_fn(xg2, rg2, None if w is None else w.to(dev), 1e-5)
    y2.backward(dy.to(dev))
    xr2 = (x.double() + r.double()).to(dtype).double().requires_grad_()
    so.rmsnorm_ref(xr2, None if w is None else w.double(), 1e-5).backward(dy.double())
    assert rel_err(xg2.grad, xr2.grad) <= tol and torch.equal(xg2.grad, rg2.grad)


@pytest.mark.parametrize("seed", range(16))
def test_rmsnorm_random_sweep(pkg, dev, seed):
    # seeded sweep over row counts (around the rows-per-wave and waves-per-block boundaries) and
    # every supported width class (1, 2, 4, 8 vectors per lane), with and without the residual
    import random
    rnd = random.Random(300 + seed)
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    vec = 4 if dtype == torch.float32 else 8
    d = vec * rnd.choice([1, 3, 16, 64, 65, 96, 128, 200, 256, 300, 512])
    rows = rnd.choice([1, 2, 7, 8, 9, 63, 64, 65, 257, 1000, 4097, 9000])
    with_res, with_w = rnd.random() < 0.5, rnd.random() < 0.8
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, d, generator=g) * 1.3).to(dtype)
    r = torch.randn(rows, d, generator=g).to(dtype)
    w = (torch.randn(d, generator=g) * 0.5 + 1.0) if with_w else None
    dy = torch.randn(rows, d, generator=g).to(dtype)
    dt = torch.randn(rows, d, generator=g).to(dtype)
    xr, rr = x.double().requires_grad_(), r.double().requires_grad_()
    wr = None if w is None else w.double().requires_grad_()
    tr = xr + rr if with_res else xr
    tq = tr + (tr.detach().to(dtype).double() - tr.detach()) if with_res else tr
    yr = so.rmsnorm_ref(tq, wr, 1e-5)
    loss = (yr * dy.double()).sum() + ((tq * dt.double()).sum() if with_res else 0.0)
    loss.backward()
    xg, rg = x.to(dev).requires_grad_(), r.to(dev).requires_grad_()
    wg = None if w is None else w.to(dev).requires_grad_()
    if with_res:
        y, total = pkg.add_rmsnorm_fn(xg, rg, wg, 1e-5)
        torch.autograd.backward([y, total], [dy.to(dev), dt.to(dev)])
    else:
        y = pkg.rmsnorm_fn(xg, wg, 1e-5)
        y.backward(dy.to(dev))
    tol = TOL[dtype]
    what = f"rows {rows} d {d} {dtype} res={with_res} w={with_w}"
    assert rel_err(y, yr) <= tol, what
    assert rel_err(xg.grad, xr.grad) <= tol, what
    if with_res:
        assert rel_err(rg.grad, rr.grad) <= tol, what
    if with_w:
        assert rel_err(wg.grad, wr.grad) <= tol, what


def test_add_rmsnorm_configs4_layer_shape_bf16(pkg, dev):
    # the norm of configs[4] at full size: (8, 4096, 768) bf16 with the residual add, forward and backward
    g = torch.Generator().manual_seed(1004)
    shape, dtype = (8, 4096, 768), torch.bfloat16
    x, r, dy, dt = (torch.randn(*shape, generator=g).to(dtype) for _ in range(4))
    w = torch.randn(768, generator=g) * 0.2 + 1.0
    xr, rr, wr = x.double().requires_grad_(), r.double().requires_grad_(), w.double().requires_grad_()
    tr = xr + rr
    tq = tr + (tr.detach().to(dtype).double() - tr.detach())
    yr = so.rmsnorm_ref(tq, wr, 1e-5)
    ((yr * dy.double()).sum() + (tq * dt.double()).sum()).backward()
    xg, rg, wg = x.to(dev).requires_grad_(), r.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    y, total = pkg.add_rmsnorm_fn(xg, rg, wg, 1e-5)
    torch.autograd.backward([y, total], [dy.to(dev), dt.to(dev)])
    tol = TOL[dtype]
    assert rel_err(y, yr) <= tol and rel_err(xg.grad, xr.grad) <= tol and rel_err(wg.grad, wr.grad) <= tol
    assert torch.equal(xg.grad, rg.grad)
