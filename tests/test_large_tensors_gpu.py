"""Tensors beyond 4 GiB: element offsets above 2^31 and byte offsets above 2^32.

A card with 288 GB holds (B, L, ED) tensors far larger than a 32-bit offset reaches; the kernels
address every tile as a 64-bit base plus 32-bit offsets inside the tile.  The checks are
size-independent properties: channels are independent, so three groups of 64 channels of the big
call (the first, one in the middle, the last: the highest addresses) must equal, bit for bit, calls
on small contiguous copies of those channels with the same segment plan; the sums over channels
(dB, dC) are checked by masking dy to those groups, and one small call is checked against the
float64 C oracle so that the chain ends at the reference's arithmetic."""
import pytest
import torch

from oracle import c_oracle
from util import rel_err

pytestmark = pytest.mark.gpu

GROUPS = (0, 2048, 4032)


def _fwd_bwd(pkg, x, delta, A, Bm, C, D, dy):
    leaves = [t.detach().requires_grad_() for t in (x, delta, A, Bm, C, D)]
    y = pkg.selective_scan_fn(*leaves)
    y.backward(dy)
    return [y.detach()] + [t.grad for t in leaves]   # y, dx, ddelta, dA, dB, dC, dD


def test_fused_scan_beyond_4_gib(pkg, dev):
    Bs, L, ED, N = 1, 280_003, 4096, 16          # 4.59e9 bytes per (B, L, ED) float32 tensor
    g = torch.Generator(device=dev).manual_seed(4100)
    x = torch.randn(Bs, L, ED, device=dev, generator=g)
    delta = torch.rand(Bs, L, ED, device=dev, generator=g) * 0.1 + 1e-3
    dy = torch.randn(Bs, L, ED, device=dev, generator=g)
    Bm, C = torch.randn(Bs, L, N, device=dev, generator=g), torch.randn(Bs, L, N, device=dev, generator=g)
    A = -torch.arange(1, N + 1, dtype=torch.float32, device=dev).repeat(ED, 1) * (
        0.5 + torch.rand(ED, 1, device=dev, generator=g))
    D = torch.randn(ED, device=dev, generator=g)
    assert x.numel() * x.element_size() > 1 << 32

    with pkg.plan_override(fwd_segments=4, bwd_segments=4):
        big = _fwd_bwd(pkg, x, delta, A, Bm, C, D, dy)
        small = {}
        for d0 in GROUPS:
            sl = slice(d0, d0 + 64)
            small[d0] = _fwd_bwd(pkg, x[:, :, sl].contiguous(), delta[:, :, sl].contiguous(), A[sl].contiguous(),
                                 Bm, C, D[sl].contiguous(), dy[:, :, sl].contiguous())
        for d0 in GROUPS:
            sl = slice(d0, d0 + 64)
            y, dx, dd, dA, _, _, dD = small[d0]
            assert torch.equal(big[0][:, :, sl], y), d0
            assert torch.equal(big[1][:, :, sl], dx), d0
            assert torch.equal(big[2][:, :, sl], dd), d0
            assert torch.equal(big[3][sl], dA), d0
            assert torch.equal(big[6][sl], dD), d0
        # dB, dC: with dy zero outside the three groups the other channels add exact zeros
        dym = torch.zeros_like(dy)
        for d0 in GROUPS:
            dym[:, :, d0:d0 + 64] = dy[:, :, d0:d0 + 64]
        masked = _fwd_bwd(pkg, x, delta, A, Bm, C, D, dym)
        for i in (4, 5):
            want = sum(small[d0][i].double() for d0 in GROUPS)
            assert rel_err(masked[i], want) <= 1e-6, i
        del masked, dym

        # the same values in (B, ED, L) memory, the layout a MambaBlock's convolution leaves: the
        # channel stride is L, the last group starts 4.5e9 bytes into the tensor
        tm = lambda t: t.transpose(1, 2).contiguous().transpose(1, 2)
        with torch.no_grad():
            y_t = pkg.selective_scan_fn(tm(x), tm(delta), A, Bm, C, D)
        assert torch.equal(y_t, big[0])
        del y_t

    # anchor: the last group's small call against the float64 C oracle
    sl = slice(GROUPS[-1], GROUPS[-1] + 64)
    inp = dict(x=x[:, :, sl].cpu(), delta=delta[:, :, sl].cpu(), A=A[sl].cpu(), B=Bm.cpu(), C=C.cpu(),
               D=D[sl].cpu(), dy=dy[:, :, sl].cpu())
    ref = c_oracle.sscan_fwd_bwd(**inp)
    names = ("y", "dx", "ddelta", "dA", "dB", "dC", "dD")
    for k, got in zip(names, small[GROUPS[-1]]):
        assert rel_err(got, ref[k]) <= 1e-4, k


def test_generic_scan_beyond_4_gib(pkg, dev):
    """pscan(A, X) on (1, 280 003, 256, 16) float32 operands (4.59e9 bytes each): lanes are
    independent, so slices of channels equal calls on small contiguous copies cut into the same
    pieces; one slice against the float64 recurrence."""
    from oracle import scan_oracle as so
    Bs, L, Dm, N = 1, 280_003, 256, 16
    g = torch.Generator(device=dev).manual_seed(4200)
    A = torch.rand(Bs, L, Dm, N, device=dev, generator=g) * 0.9 + 0.05
    X = torch.randn(Bs, L, Dm, N, device=dev, generator=g)
    G = torch.randn(Bs, L, Dm, N, device=dev, generator=g)
    assert A.numel() * A.element_size() > 1 << 32

    def run(a, x, gr):
        a, x = a.detach().requires_grad_(), x.detach().requires_grad_()
        h = pkg.pscan(a, x)
        h.backward(gr)
        return h.detach(), a.grad, x.grad

    with pkg.plan_override(pscan_chunks=64):
        big = run(A, X, G)
        for d0 in (0, 128, 252):
            sl = slice(d0, d0 + 4)
            small = run(A[:, :, sl].contiguous(), X[:, :, sl].contiguous(), G[:, :, sl].contiguous())
            for b_, s_ in zip(big, small):
                assert torch.equal(b_[:, :, sl], s_), d0
    # anchor: the last slice's first 20 000 steps against the float64 recurrence
    a64, x64 = A[:, :20000, 252:].double().cpu(), X[:, :20000, 252:].double().cpu()
    assert rel_err(big[0][:, :20000, 252:], so.linear_recurrence(a64, x64)) <= 1e-5
