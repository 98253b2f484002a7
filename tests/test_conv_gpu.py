"""GPU parity of the causal depthwise conv1d (+bias, +SiLU) kernel against the oracle
(mambapy/mamba.py:217-221, 366-369, 379)."""
import pytest
import torch

from oracle import scan_oracle as so
from util import TOL, rel_err

pytestmark = pytest.mark.gpu


def _case(pkg, dev, Bsz, L, ED, K, dtype, seed, strided=False, window=False, silu=True, bias=True):
    g = torch.Generator().manual_seed(seed)
    if strided:  # the x half of an in_proj output: row stride 2*ED
        xz = torch.randn(Bsz, L, 2 * ED, generator=g).to(dtype)
        x = xz[:, :, :ED]
    else:
        x = torch.randn(Bsz, L, ED, generator=g).to(dtype)
    w = (torch.randn(ED, 1, K, generator=g) * 0.5).to(dtype)
    b = (torch.randn(ED, generator=g) * 0.3).to(dtype) if bias else None
    win = torch.randn(Bsz, ED, K - 1, generator=g).to(dtype) if window else None
    dy = torch.randn(Bsz, L, ED, generator=g).to(dtype)

    xr, wr = x.double().requires_grad_(), w.double().requires_grad_()
    br = None if b is None else b.double().requires_grad_()
    yr = so.causal_conv1d_ref(xr, wr, br, None if win is None else win.double(), silu=silu)
    yr.backward(dy.double())
    ref = dict(y=yr, dx=xr.grad, dw=wr.grad)
    if br is not None:
        ref["db"] = br.grad

    if strided:
        xzg = xz.to(dev).requires_grad_()
        xg = xzg[:, :, :ED]
    else:
        xg = x.to(dev).requires_grad_()
    wg = w.to(dev).requires_grad_()
    bg = None if b is None else b.to(dev).requires_grad_()
    y, wout = pkg.causal_conv1d_fn(xg, wg, bg, window=None if win is None else win.to(dev),
                                   silu=silu, return_window=True)
    y.backward(dy.to(dev))
    got = dict(y=y, dx=(xzg.grad[:, :, :ED] if strided else xg.grad), dw=wg.grad)
    if bg is not None:
        got["db"] = bg.grad
    # the window to continue decoding from: the last K-1 inputs (mamba.py:379)
    full = x.transpose(1, 2) if win is None else torch.cat([win, x.transpose(1, 2)], dim=2)
    if full.shape[2] < K - 1:
        full = torch.nn.functional.pad(full, (K - 1 - full.shape[2], 0))
    assert torch.equal(wout.cpu(), full[:, :, full.shape[2] - (K - 1):].contiguous())
    if strided:
        assert torch.count_nonzero(xzg.grad[:, :, ED:]) == 0
    return got, ref


@pytest.mark.parametrize("Bsz,L,ED,K", [(2, 64, 64, 4), (1, 1, 3, 4), (3, 70, 130, 4), (2, 200, 257, 3),
                                         (2, 2, 70, 4), (1, 129, 64, 2)])
def test_conv_fp32_shapes(pkg, dev, Bsz, L, ED, K):
    got, ref = _case(pkg, dev, Bsz, L, ED, K, torch.float32, 400 + L + ED)
    for k in ref:
        assert rel_err(got[k], ref[k]) <= TOL[torch.float32], k


def test_conv_strided_input_window_no_bias_no_silu(pkg, dev):
    got, ref = _case(pkg, dev, 2, 100, 96, 4, torch.float32, 431, strided=True, window=True)
    for k in ref:
        assert rel_err(got[k], ref[k]) <= TOL[torch.float32], k
    got, ref = _case(pkg, dev, 2, 50, 64, 4, torch.float32, 432, silu=False, bias=False)
    for k in ref:
        assert rel_err(got[k], ref[k]) <= TOL[torch.float32], k


def test_conv_bf16(pkg, dev):
    got, ref = _case(pkg, dev, 2, 300, 192, 4, torch.bfloat16, 441, strided=True)
    for k in ref:
        assert rel_err(got[k], ref[k]) <= TOL[torch.bfloat16], k


def test_conv_matches_step_by_step_decode(pkg, dev):
    # prefill with the kernel, then one token at a time with the rolling window of the oracle
    g = torch.Generator().manual_seed(451)
    Bsz, L, ED, K = 2, 20, 64, 4
    x = torch.randn(Bsz, L + 5, ED, generator=g)
    w, b = torch.randn(ED, 1, K, generator=g) * 0.5, torch.randn(ED, generator=g) * 0.3
    y_all = so.causal_conv1d_ref(x.double(), w.double(), b.double(), silu=False)
    y, win = pkg.causal_conv1d_fn(x[:, :L].to(dev), w.to(dev), b.to(dev), silu=False, return_window=True)
    assert rel_err(y, y_all[:, :L]) <= TOL[torch.float32]
    win = win.cpu().double()
    for t in range(L, L + 5):
        out, win = so.conv_window_step_ref(win, x[:, t].double(), w.double(), b.double())
        assert rel_err(out, y_all[:, t]) <= 1e-12


def test_conv_full_size_c4_layer_properties(pkg, dev):
    # configs[4] layer shape (B=8, L=3000, ED=1536), bf16: linearity of the pre-activation in x
    # and agreement of two segments (second one started from the first one's window) with one pass
    g = torch.Generator().manual_seed(461)
    Bsz, L, ED, K = 8, 3000, 1536, 4
    x = torch.randn(Bsz, L, ED, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(ED, 1, K, generator=g) * 0.5).to(dev)
    b = (torch.randn(ED, generator=g) * 0.3).to(dev)
    with torch.no_grad():
        y = pkg.causal_conv1d_fn(x, w, b)
        y1, win = pkg.causal_conv1d_fn(x[:, :1700], w, b, return_window=True)
        y2 = pkg.causal_conv1d_fn(x[:, 1700:], w, b, window=win)
        assert torch.equal(torch.cat([y1, y2], dim=1), y)
        p1 = pkg.causal_conv1d_fn(x, w, None, silu=False).float()
        p2 = pkg.causal_conv1d_fn((2 * x.float()).to(torch.bfloat16), w, None, silu=False).float()
        assert rel_err(p2, 2 * p1) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("K,dtype", [(4, torch.float32), (3, torch.float32), (2, torch.bfloat16), (4, torch.bfloat16)])
def test_decode_update_rolls_the_window_in_place(pkg, dev, K, dtype):
    # mambapy/mamba.py:366-369, 379: conv over (cache, newest input), then the cache drops its oldest
    g = torch.Generator().manual_seed(40 + K)
    Bsz, ED = 3, 200
    w = torch.randn(ED, 1, K, generator=g)
    b = torch.randn(ED, generator=g)
    window = torch.randn(Bsz, ED, K - 1, generator=g).to(dtype)
    xz = torch.randn(Bsz, 2 * ED, generator=g).to(dtype)       # x is the first half of a wider row
    win_dev = window.to(dev)
    ref_win = window.double()
    for _ in range(3):
        x = xz[:, :ED]
        want, ref_win = so.conv_window_step_ref(ref_win, x.double(), w.double(), b.double())
        want = want * torch.sigmoid(want)
        got = pkg.causal_conv1d_update(xz.to(dev)[:, :ED], win_dev, w.to(dev), b.to(dev))
        assert rel_err(got, want) <= TOL[dtype]
        assert torch.equal(win_dev.cpu().double(), ref_win)    # the cache holds inputs, bit for bit
        xz = xz.roll(1, 0) * 0.5 + 0.1


@pytest.mark.parametrize("seed", range(24))
def test_conv_random_sweep(pkg, dev, seed):
    # seeded sweep: ragged lengths around the 64/128-step spans, channel counts around the
    # wave width, every tap count, strided input, decode window, with and without silu / bias
    import random
    rnd = random.Random(77 + seed)
    Bsz = rnd.randint(1, 3)
    L = rnd.choice([1, 2, 3, 5, 63, 64, 65, 127, 128, 129, 191, 200, 257, 300])
    ED = rnd.choice([1, 5, 63, 64, 65, 128, 200, 256, 257])
    K = rnd.choice([2, 3, 4])
    dtype = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
    got, ref = _case(pkg, dev, Bsz, L, ED, K, dtype, 5000 + seed, strided=rnd.random() < 0.5,
                     window=rnd.random() < 0.5, silu=rnd.random() < 0.7, bias=rnd.random() < 0.8)
    for k in ref:
        assert rel_err(got[k], ref[k]) <= TOL[dtype], f"B{Bsz} L{L} ED{ED} K{K} {dtype}: {k}"
