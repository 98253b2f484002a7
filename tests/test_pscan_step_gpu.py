"""GPU parity of the generic scan (mpa_pscan_fwd/bwd) and of the decode step (mpa_ssm_step)."""
import pytest
import torch

from oracle import scan_oracle as so
from util import TOL, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("Bs,L,D,N", [(1, 1, 1, 1), (2, 4, 3, 16), (2, 64, 32, 16), (3, 100, 7, 5),
                                      (1, 3000, 16, 16), (2, 17, 130, 16)])
def test_pscan_forward_backward_fp32(pkg, dev, Bs, L, D, N):
    g = torch.Generator().manual_seed(L + D)
    A = torch.rand(Bs, L, D, N, generator=g) * 0.98 + 0.01
    X = torch.randn(Bs, L, D, N, generator=g)
    G = torch.randn(Bs, L, D, N, generator=g)
    A64, X64 = A.double().requires_grad_(), X.double().requires_grad_()
    Href = so.linear_recurrence(A64, X64)
    gA_ref, gX_ref = torch.autograd.grad(Href, (A64, X64), G.double())
    Ag, Xg = A.to(dev).requires_grad_(), X.to(dev).requires_grad_()
    H = pkg.pscan(Ag, Xg)
    H.backward(G.to(dev))
    assert rel_err(H, Href) <= TOL[torch.float32]
    assert rel_err(Ag.grad, gA_ref) <= TOL[torch.float32]
    assert rel_err(Xg.grad, gX_ref) <= TOL[torch.float32]
    assert torch.all(Ag.grad[:, 0] == 0)  # mambapy/pscan.py:221-222


def test_pscan_reference_golden_vectors(pkg, dev):
    # docs/pscan.ipynb cells 5/8/11 and docs/tests.ipynb cell 1 (A == 1: cumulative sums)
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.json")) as f:
        golden = json.load(f)
    for key in ("cumsum_1234", "padded_scan"):
        X = torch.tensor(golden[key]["X"], dtype=torch.float32, device=dev).reshape(1, -1, 1, 1)
        assert pkg.pscan(torch.ones_like(X), X).flatten().tolist() == golden[key]["H"]


def test_pscan_inputs_untouched_and_strided_views(pkg, dev):
    # the reference clones its inputs (pscan.py:167-174); inside MambaBlock the tensors are
    # (B,ED,L,N) memory viewed as (B,L,ED,N)
    g = torch.Generator().manual_seed(0)
    A = (torch.rand(2, 8, 50, 16, generator=g) * 0.9).to(dev).transpose(1, 2)
    X = torch.randn(2, 8, 50, 16, generator=g).to(dev).transpose(1, 2)
    A0, X0 = A.clone(), X.clone()
    H = pkg.pscan(A, X)
    assert torch.equal(A, A0) and torch.equal(X, X0)
    assert rel_err(H, so.linear_recurrence(A.double().cpu(), X.double().cpu())) <= TOL[torch.float32]


def test_pscan_bf16(pkg, dev):
    g = torch.Generator().manual_seed(1)
    A = (torch.rand(2, 200, 24, 16, generator=g) * 0.9).bfloat16()
    X = torch.randn(2, 200, 24, 16, generator=g).bfloat16()
    H = pkg.pscan(A.to(dev), X.to(dev))
    assert H.dtype == torch.bfloat16
    assert rel_err(H, so.linear_recurrence(A.double(), X.double())) <= TOL[torch.bfloat16]


def test_selective_scan_through_pscan_equals_fused(pkg, dev):
    # the reference composes discretise -> pscan -> readout (mamba.py:284-293); the same
    # composition through the generic kernel must agree with the fused kernel
    inp = so.make_inputs(2, 70, 48, 16, seed=3)
    g = {k: v.to(dev) for k, v in inp.items()}
    dA = torch.exp(g["delta"].unsqueeze(-1) * g["A"])
    BX = g["delta"].unsqueeze(-1) * g["B"].unsqueeze(2) * g["x"].unsqueeze(-1)
    hs = pkg.pscan(dA, BX)
    y1 = (hs @ g["C"].unsqueeze(-1)).squeeze(3) + g["D"] * g["x"]
    y2 = pkg.selective_scan(g["x"], g["delta"], g["A"], g["B"], g["C"], g["D"])
    assert rel_err(y1, y2) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_steps_reproduce_scan(pkg, dev, dtype):
    # L decode steps from h = None equal one scan over L (mamba.py:344-346)
    inp = so.make_inputs(3, 40, 100, 16, seed=13, dtype=dtype)
    names = ("x", "delta", "A", "B", "C", "D")
    yr, hr = so.selective_scan_ref(*[inp[k].double() for k in names], return_last_state=True)
    g = {k: v.to(dev) for k, v in inp.items()}
    h, ys = None, []
    for t in range(40):
        y, h = pkg.ssm_step(g["x"][:, t], g["delta"][:, t], g["A"], g["B"][:, t], g["C"][:, t], g["D"], h)
        ys.append(y)
    assert rel_err(torch.stack(ys, 1), yr) <= TOL[dtype]
    assert rel_err(h, hr) <= TOL[torch.float32]


def test_step_semantics_new_state_inplace_gate_softplus(pkg, dev):
    Bs, ED, N = 4, 70, 16
    g = torch.Generator().manual_seed(5)
    x, raw, z = (torch.randn(Bs, ED, generator=g) for _ in range(3))
    Bm, C = torch.randn(Bs, N, generator=g), torch.randn(Bs, N, generator=g)
    A = -torch.rand(ED, N, generator=g) * 4
    D, bias = torch.randn(ED, generator=g), torch.randn(ED, generator=g)
    h = torch.randn(Bs, ED, N, generator=g)
    delta = so.softplus_ref((raw + bias).double())
    yr, hr = so.ssm_step_ref(x.double(), delta, A.double(), Bm.double(), C.double(), D.double(), h.double())
    yr = yr * (z.double() * torch.sigmoid(z.double()))
    hg = h.to(dev)
    h_before = hg.clone()
    y, h_new = pkg.ssm_step(x.to(dev), raw.to(dev), A.to(dev), Bm.to(dev), C.to(dev), D.to(dev), hg,
                            z=z.to(dev), delta_bias=bias.to(dev), delta_softplus=True)
    assert torch.equal(hg, h_before) and h_new.data_ptr() != hg.data_ptr()  # old cache stays valid
    assert rel_err(y, yr) <= TOL[torch.float32] and rel_err(h_new, hr) <= TOL[torch.float32]
    y2, h2 = pkg.ssm_step(x.to(dev), raw.to(dev), A.to(dev), Bm.to(dev), C.to(dev), D.to(dev), hg,
                          z=z.to(dev), delta_bias=bias.to(dev), delta_softplus=True, inplace=True)
    assert h2.data_ptr() == hg.data_ptr() and torch.equal(h2, h_new) and torch.equal(y2, y)


def test_step_config3_shape(pkg, dev):
    # configs[3]: mamba-2.8b decode, batch 64, ED=5120, N=16, float32 state
    Bs, ED, N = 64, 5120, 16
    g = torch.Generator().manual_seed(7)
    inp = so.make_inputs(Bs, 1, ED, N, seed=1003)
    h = torch.randn(Bs, ED, N, generator=g)
    x, dl, Bm, C = inp["x"][:, 0], inp["delta"][:, 0], inp["B"][:, 0], inp["C"][:, 0]
    yr, hr = so.ssm_step_ref(x.double(), dl.double(), inp["A"].double(), Bm.double(), C.double(),
                             inp["D"].double(), h.double())
    y, hn = pkg.ssm_step(x.to(dev), dl.to(dev), inp["A"].to(dev), Bm.to(dev), C.to(dev),
                         inp["D"].to(dev), h.to(dev))
    assert rel_err(y, yr) <= TOL[torch.float32] and rel_err(hn, hr) <= TOL[torch.float32]


def test_config3_256_steps_equal_one_scan_with_carried_state(pkg, dev):
    # configs[3] at full size: 256 in-place decode steps from a random state (batch 64, ED=5120,
    # N=16) must give what one scan over the same 256 positions with that initial state gives
    # (mambapy/mamba.py:344-346), outputs and final state
    Bs, T, ED, N = 64, 256, 5120, 16
    inp = so.make_inputs(Bs, T, ED, N, seed=1003)
    g = torch.Generator().manual_seed(8)
    h0 = torch.randn(Bs, ED, N, generator=g)
    d = {k: v.to(dev) for k, v in inp.items()}
    with torch.no_grad():
        y_scan, h_scan = pkg.selective_scan_fn(d["x"], d["delta"], d["A"], d["B"], d["C"], d["D"],
                                               h0=h0.to(dev), return_last_state=True)
        h = h0.to(dev).clone()
        ys = []
        for t in range(T):
            y, _ = pkg.ssm_step(d["x"][:, t], d["delta"][:, t], d["A"], d["B"][:, t], d["C"][:, t], d["D"], h,
                                inplace=True)
            ys.append(y)
    assert rel_err(torch.stack(ys, 1), y_scan.double()) <= TOL[torch.float32]
    assert rel_err(h, h_scan.double()) <= TOL[torch.float32]


@pytest.mark.parametrize("seed", range(24))
def test_step_random_sweep(pkg, dev, seed):
    # seeded sweep of the decode step: every d_state class of the kernel (4*Q lanes-per-row form, the
    # one-lane-per-row forms), B / C / z as slices of wider rows, gate + softplus + bias, fresh and
    # carried state, fp32 and bf16 vectors
    import random
    rnd = random.Random(900 + seed)
    Bs, ED = rnd.choice([1, 2, 5, 64]), rnd.choice([1, 7, 64, 65, 130, 256])
    N = rnd.choice([1, 2, 3, 4, 8, 12, 16, 16, 16, 24, 32, 64])
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    gated, with_h = rnd.random() < 0.6, rnd.random() < 0.7
    g = torch.Generator().manual_seed(seed)
    xz = torch.randn(Bs, 2 * ED, generator=g).to(dtype)            # z is the second half of a wider row
    x, z = torch.randn(Bs, ED, generator=g).to(dtype), xz[:, ED:]
    raw = (torch.randn(Bs, ED, generator=g) * 0.5 - 3.0).to(dtype)
    dbc = torch.randn(Bs, 5 + 2 * N, generator=g).to(dtype)        # B and C as slices of one projection
    Bm, C = dbc[:, 5:5 + N], dbc[:, 5 + N:]
    A = -torch.rand(ED, N, generator=g) * 4
    D, bias = torch.randn(ED, generator=g), torch.randn(ED, generator=g) * 0.3
    h = torch.randn(Bs, ED, N, generator=g) if with_h else None
    delta = so.softplus_ref(raw.double() + bias.double()) if gated else raw.double().abs() * 0.05
    yr, hr = so.ssm_step_ref(x.double(), delta, A.double(), Bm.double(), C.double(), D.double(),
                             None if h is None else h.double())
    if gated:
        yr = yr * (z.double() * torch.sigmoid(z.double()))
        y, hn = pkg.ssm_step(x.to(dev), raw.to(dev), A.to(dev), dbc.to(dev)[:, 5:5 + N], dbc.to(dev)[:, 5 + N:],
                             D.to(dev), None if h is None else h.to(dev), z=xz.to(dev)[:, ED:],
                             delta_bias=bias.to(dev), delta_softplus=True)
    else:
        dl = (raw.double().abs() * 0.05).to(dtype)
        yr, hr = so.ssm_step_ref(x.double(), dl.double(), A.double(), Bm.double(), C.double(), D.double(),
                                 None if h is None else h.double())
        y, hn = pkg.ssm_step(x.to(dev), dl.to(dev), A.to(dev), dbc.to(dev)[:, 5:5 + N], dbc.to(dev)[:, 5 + N:],
                             D.to(dev), None if h is None else h.to(dev))
    what = f"B{Bs} ED{ED} N{N} {dtype} gated={gated} h={with_h}"
    assert rel_err(y, yr) <= TOL[dtype], what
    assert rel_err(hn, hr) <= TOL[torch.float32], what
