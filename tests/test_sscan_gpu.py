"""GPU parity of the fused selective scan (mpa_sscan_fwd / mpa_sscan_bwd through the C ABI)
against the float64 oracles, on the seeded inputs of the benchmark configurations."""
import pytest
import torch

from oracle import c_oracle, scan_oracle as so
from util import GRAD_KEYS, TOL, rel_err, run_gpu_fwd_bwd

pytestmark = pytest.mark.gpu


def _check(got, ref, tol, what):
    for k in ("y",) + GRAD_KEYS:
        e = rel_err(got[k], ref[k])
        assert e <= tol, f"{what}: {k} rel err {e:.3e} > {tol}"


def test_config0_fp32_vs_autograd_oracle(pkg, dev):
    # configs[0]: B=2, L=64, ED=32, N=16, float32
    inp = so.make_inputs(2, 64, 32, 16, seed=1000)
    ref = so.selective_scan_grads_autograd(**inp)
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.float32], "config0")


@pytest.mark.parametrize("Bs,L,ED,N", [
    (1, 1, 1, 16), (1, 7, 5, 16), (2, 17, 64, 16), (3, 100, 96, 16), (2, 33, 130, 8),
    (1, 250, 70, 4), (2, 48, 64, 32), (1, 40, 65, 64), (2, 31, 33, 1), (1, 129, 64, 24),
])
def test_ragged_shapes_fp32(pkg, dev, Bs, L, ED, N):
    inp = so.make_inputs(Bs, L, ED, N, seed=11 * L + ED + N)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.float32], f"B{Bs} L{L} ED{ED} N{N}")


@pytest.mark.parametrize("ns", [1, 2, 4])
def test_every_state_split_agrees(pkg, dev, ns):
    # the wave decomposition (states per lane) is a tuning choice; every choice must agree
    inp = so.make_inputs(2, 200, 160, 16, seed=5)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    with pkg.plan_override(fwd_states_per_lane=ns, bwd_states_per_lane=ns):
        got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.float32], f"ns={ns}")


@pytest.mark.parametrize("ns", [8, 16])
def test_forward_wide_lanes(pkg, dev, ns):
    inp = so.make_inputs(2, 200, 160, 16, seed=6)
    ref = c_oracle.sscan_fwd(*[inp[k] for k in ("x", "delta", "A", "B", "C", "D")])
    with torch.no_grad(), pkg.plan_override(fwd_states_per_lane=ns):
        y = pkg.selective_scan(*[inp[k].to(dev) for k in ("x", "delta", "A", "B", "C", "D")])
    assert rel_err(y, ref) <= TOL[torch.float32]


def test_bf16_io_fp32_state(pkg, dev):
    inp = so.make_inputs(2, 300, 192, 16, seed=21, dtype=torch.bfloat16)
    ref = c_oracle.sscan_fwd_bwd(**inp)  # oracle consumes the bf16-rounded values
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    assert got["y"].dtype == torch.bfloat16 and got["dx"].dtype == torch.bfloat16
    _check(got, ref, TOL[torch.bfloat16], "bf16")


def test_time_contiguous_views_and_sliced_BC(pkg, dev):
    # the layouts MambaBlock.forward produces: x, delta are (B,ED,L) memory viewed as
    # (B,L,ED); B and C are slices of one (B,L,dt_rank+2N) projection
    Bs, L, ED, N, R = 2, 77, 100, 16, 7
    inp = so.make_inputs(Bs, L, ED, N, seed=31)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    x = inp["x"].to(dev).transpose(1, 2).contiguous().transpose(1, 2).requires_grad_()
    delta = inp["delta"].to(dev).transpose(1, 2).contiguous().transpose(1, 2).requires_grad_()
    assert x.stride() == (ED * L, 1, L)
    proj = torch.zeros(Bs, L, R + 2 * N, device=dev)
    proj[..., R:R + N] = inp["B"].to(dev)
    proj[..., R + N:] = inp["C"].to(dev)
    proj.requires_grad_()
    _, Bm, C = torch.split(proj, [R, N, N], dim=-1)
    A = inp["A"].to(dev).requires_grad_()
    D = inp["D"].to(dev).requires_grad_()
    y = pkg.selective_scan(x, delta, A, Bm, C, D)
    y.backward(inp["dy"].to(dev))
    got = dict(y=y, dx=x.grad, ddelta=delta.grad, dA=A.grad, dD=D.grad,
               dB=proj.grad[..., R:R + N], dC=proj.grad[..., R + N:])
    _check(got, ref, TOL[torch.float32], "strided")


def test_special_cases_closed_form(pkg, dev):
    # delta = 0 or C = 0  =>  y = D*x ;  A = 0  =>  y_t = sum_{s<=t} delta_s x_s (B_s.C_t) + D x_t
    inp = so.make_inputs(2, 50, 64, 16, seed=41)
    g = {k: v.to(dev) for k, v in inp.items()}
    with torch.no_grad():
        y = pkg.selective_scan(g["x"], torch.zeros_like(g["delta"]), g["A"], g["B"], g["C"], g["D"])
        assert rel_err(y, inp["D"] * inp["x"]) <= 1e-6
        y = pkg.selective_scan(g["x"], g["delta"], g["A"], g["B"], torch.zeros_like(g["C"]), g["D"])
        assert rel_err(y, inp["D"] * inp["x"]) <= 1e-6
        y = pkg.selective_scan(g["x"], g["delta"], torch.zeros_like(g["A"]), g["B"], g["C"], g["D"])
    u = (inp["delta"] * inp["x"]).double()
    G = torch.einsum("btn,bsn->bts", inp["C"].double(), inp["B"].double()).tril()
    ref = torch.einsum("bts,bsd->btd", G, u) + inp["D"].double() * inp["x"].double()
    assert rel_err(y, ref) <= TOL[torch.float32]


def test_reference_test_distribution_randn_A_and_delta(pkg, dev):
    # tests/compare_seq_pscan.py:24-29 of the reference draws every input, delta and A
    # included, from N(0,1) (so exp(delta*A) may exceed 1), Bs,L,ED,N = 2,64,64,16
    g = torch.Generator().manual_seed(3)
    Bs, L, ED, N = 2, 64, 64, 16
    inp = dict(x=torch.randn(Bs, L, ED, generator=g), delta=torch.randn(Bs, L, ED, generator=g),
               A=torch.randn(ED, N, generator=g), B=torch.randn(Bs, L, N, generator=g),
               C=torch.randn(Bs, L, N, generator=g), D=torch.randn(ED, generator=g),
               dy=torch.randn(Bs, L, ED, generator=g))
    ref = c_oracle.sscan_fwd_bwd(**inp)
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.float32], "randn A/delta")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sum_backward_convention_of_the_reference_tests(pkg, dev, dtype):
    # tests/compare_mambapy_cuda.py:49-53 of the reference backpropagates y.sum(): the upstream
    # gradient is an expanded (stride-0) tensor of ones
    inp = so.make_inputs(2, 300, 192, 16, seed=77, dtype=dtype)
    inp["dy"] = torch.ones_like(inp["x"])
    ref = c_oracle.sscan_fwd_bwd(**inp)
    names = ("x", "delta", "A", "B", "C", "D")
    args = [inp[k].to(dev).requires_grad_() for k in names]
    y = pkg.selective_scan(*args)
    y.sum().backward()
    got = dict(y=y.detach(), **{k: a.grad for k, a in zip(GRAD_KEYS, args)})
    _check(got, ref, TOL[dtype], "y.sum().backward()")


def test_gate_softplus_bias_h0_and_last_state(pkg, dev):
    Bs, L, ED, N = 2, 90, 80, 16
    inp = so.make_inputs(Bs, L, ED, N, seed=51)
    g = torch.Generator().manual_seed(52)
    z = torch.randn(Bs, L, ED, generator=g)
    raw = torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0
    bias = torch.randn(ED, generator=g) * 0.3
    h0 = torch.randn(Bs, ED, N, generator=g)
    f64 = lambda t: t.double().requires_grad_()
    x, r, A, Bm, C, D, zz, bb = map(f64, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    delta = so.softplus_ref(r + bb)
    yr, hl = so.selective_scan_ref(x, delta, A, Bm, C, D, h0=h0.double(), return_last_state=True)
    yr = yr * (zz * torch.sigmoid(zz))
    yr.backward(inp["dy"].double())
    ref = dict(y=yr, dx=x.grad, ddelta=r.grad, dA=A.grad, dB=Bm.grad, dC=C.grad, dD=D.grad,
               dz=zz.grad, dbias=bb.grad, hl=hl)
    t = lambda v: v.to(dev).requires_grad_()
    gx, gr, gA, gB, gC, gD, gz, gb = map(t, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    y, h_last = pkg.selective_scan_fn(gx, gr, gA, gB, gC, gD, z=gz, delta_bias=gb,
                                      delta_softplus=True, h0=h0.to(dev), return_last_state=True)
    y.backward(inp["dy"].to(dev))
    got = dict(y=y, dx=gx.grad, ddelta=gr.grad, dA=gA.grad, dB=gB.grad, dC=gC.grad, dD=gD.grad,
               dz=gz.grad, dbias=gb.grad, hl=h_last)
    for k in ref:
        e = rel_err(got[k], ref[k])
        assert e <= TOL[torch.float32], f"{k}: {e:.3e}"



def _gated_case(pkg, dev, Bs, L, ED, N, dtype, seed, tmajor=False):
    inp = so.make_inputs(Bs, L, ED, N, seed=seed, dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1)
    z = torch.randn(Bs, L, ED, generator=g).to(dtype)
    f64 = lambda t: t.double().requires_grad_()
    names = ("x", "delta", "A", "B", "C", "D")
    ref_in = [f64(inp[k]) for k in names] + [f64(z)]
    yr = so.selective_scan_ref(*ref_in[:6]) * (ref_in[6] * torch.sigmoid(ref_in[6]))
    yr.backward(inp["dy"].double())
    ref = dict(y=yr, dz=ref_in[6].grad, **{k: a.grad for k, a in zip(GRAD_KEYS, ref_in)})

    def to_dev(t):
        t = t.to(dev)
        if tmajor and t.dim() == 3 and t.shape[-1] == ED:
            t = t.transpose(1, 2).contiguous().transpose(1, 2)  # (B, ED, L) memory
        return t.requires_grad_()

    gin = [to_dev(inp[k]) for k in names] + [to_dev(z)]
    y = pkg.selective_scan_fn(*gin[:6], z=gin[6])
    y.backward(inp["dy"].to(dev))
    got = dict(y=y, dz=gin[6].grad, **{k: a.grad for k, a in zip(GRAD_KEYS, gin)})
    return got, ref


@pytest.mark.parametrize("Bs,L,ED,N", [(2, 64, 64, 16), (1, 37, 70, 16), (3, 129, 200, 12)])
def test_gated_backward_fast_path_fp32(pkg, dev, Bs, L, ED, N):
    got, ref = _gated_case(pkg, dev, Bs, L, ED, N, torch.float32, 300 + L)
    for k in ref:
        e = rel_err(got[k], ref[k])
        assert e <= TOL[torch.float32], f"{k}: {e:.3e}"


def test_gated_backward_bf16_and_time_contiguous(pkg, dev):
    got, ref = _gated_case(pkg, dev, 2, 100, 96, 16, torch.bfloat16, 311, tmajor=True)
    for k in ref:
        e = rel_err(got[k], ref[k])
        assert e <= TOL[torch.bfloat16], f"{k}: {e:.3e}"


def test_gated_backward_fast_equals_general_kernel(pkg, dev):
    # the two backward kernels (saved pre-gate output vs recomputed one) must agree
    a, _ = _gated_case(pkg, dev, 2, 80, 128, 16, torch.float32, 321)
    with pkg.plan_override(bwd_general=True):
        b, _ = _gated_case(pkg, dev, 2, 80, 128, 16, torch.float32, 321)
    for k in a:
        assert rel_err(a[k], b[k]) <= 2e-6, k



def test_time_outermost_memory_and_ragged_tail(pkg, dev):
    # (L, B, ED) memory viewed as (B, L, ED): the time stride is the largest one, so a ragged
    # last tile of ANY batch row would run off the allocation if loads were not windowed;
    # also a batch-expanded (stride 0) delta
    Bs, L, ED, N = 3, 21, 70, 16
    inp = so.make_inputs(Bs, L, ED, N, seed=91)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    names = ("x", "delta", "A", "B", "C", "D")

    def lbe(t):  # same values, time-outermost memory
        return t.to(dev).permute(1, 0, 2).contiguous().permute(1, 0, 2).requires_grad_()

    args = [lbe(inp[k]) if k in ("x", "delta", "B", "C") else inp[k].to(dev).requires_grad_() for k in names]
    assert args[0].stride() == (ED, Bs * ED, 1)
    y = pkg.selective_scan_fn(*args)
    y.backward(lbe(inp["dy"]).detach())
    got = dict(y=y, **{k: a.grad for k, a in zip(GRAD_KEYS, args)})
    _check(got, ref, TOL[torch.float32], "time-outermost")

    d1 = inp["delta"][:1]
    with torch.no_grad():
        y_exp = pkg.selective_scan_fn(inp["x"].to(dev), d1.to(dev).expand(Bs, L, ED), inp["A"].to(dev),
                                      inp["B"].to(dev), inp["C"].to(dev), inp["D"].to(dev))
    ref_exp = c_oracle.sscan_fwd(inp["x"], d1.expand(Bs, L, ED).contiguous(), inp["A"], inp["B"], inp["C"], inp["D"])
    assert rel_err(y_exp, ref_exp) <= TOL[torch.float32]


def _inference_case(pkg, dev, Bs, L, ED, N, dtype, seed, gated):
    """forward without gradients (no checkpoints): y and the last state"""
    inp = so.make_inputs(Bs, L, ED, N, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    h0 = torch.randn(Bs, ED, N, generator=g)
    z = torch.randn(Bs, L, ED, generator=g) if gated else None
    raw = torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0
    bias = torch.randn(ED, generator=g) * 0.3
    q = lambda t: t.to(dtype)
    d64 = lambda t: q(t).double()
    delta = so.softplus_ref(d64(raw) + bias.double()) if gated else d64(inp["delta"])
    yr, hl = so.selective_scan_ref(d64(inp["x"]), delta, inp["A"].double(), d64(inp["B"]), d64(inp["C"]),
                                   inp["D"].double(), h0=h0.double(), return_last_state=True)
    if gated:
        yr = yr * (d64(z) * torch.sigmoid(d64(z)))
    with torch.no_grad():
        dv = lambda t: q(t).to(dev)
        if gated:
            y, hg = pkg.selective_scan_fn(dv(inp["x"]), dv(raw), inp["A"].to(dev), dv(inp["B"]), dv(inp["C"]),
                                          inp["D"].to(dev), z=dv(z), delta_bias=bias.to(dev), delta_softplus=True,
                                          h0=h0.to(dev), return_last_state=True)
        else:
            y, hg = pkg.selective_scan_fn(dv(inp["x"]), dv(inp["delta"]), inp["A"].to(dev), dv(inp["B"]),
                                          dv(inp["C"]), inp["D"].to(dev), h0=h0.to(dev), return_last_state=True)
    return y, hg, yr, hl


@pytest.mark.parametrize("Bs,L,ED,N,nseg,gated", [
    (1, 160, 64, 16, 3, False), (2, 100, 70, 16, 4, True), (1, 37, 130, 8, 2, False),
    (1, 1000, 96, 16, 7, True), (3, 64, 64, 4, 4, False), (1, 16, 64, 16, 5, False), (1, 33, 5, 16, 64, True),
])
def test_segmented_forward_matches_oracle_and_single_pass(pkg, dev, Bs, L, ED, N, nseg, gated):
    # inference form (no checkpoints) with the sequence cut into segments that run side by side
    with pkg.plan_override(fwd_segments=nseg):
        y, hg, yr, hl = _inference_case(pkg, dev, Bs, L, ED, N, torch.float32, 300 + L, gated)
    assert rel_err(y, yr) <= TOL[torch.float32]
    assert rel_err(hg, hl) <= TOL[torch.float32]
    with pkg.plan_override(fwd_segments=1):
        y1, h1, _, _ = _inference_case(pkg, dev, Bs, L, ED, N, torch.float32, 300 + L, gated)
    assert rel_err(y, y1.double()) <= 1e-5 and rel_err(hg, h1.double()) <= 1e-5


def test_segmented_forward_is_picked_for_a_single_long_sequence(pkg, dev):
    # batch 1, 24 channel groups, 4096 steps in bf16: the library cuts the sequence by itself
    y, hg, yr, hl = _inference_case(pkg, dev, 1, 4096, 1536, 16, torch.bfloat16, 77, True)
    assert rel_err(y, yr) <= TOL[torch.bfloat16]
    assert rel_err(hg, hl) <= TOL[torch.float32]
    big = torch.empty(1, 4096, 1536, dtype=torch.bfloat16, device=dev)
    bc = torch.empty(1, 4096, 16, dtype=torch.bfloat16, device=dev)
    shape = pkg.scan._sscan_shape(big, big, bc, big, big, bc, 16, 0)
    import ctypes
    need = pkg._lib.load().mpa_sscan_fwd_workspace_bytes(ctypes.byref(shape), 0)
    assert need > 2 * 10 * 1536 * 16 * 4  # room for the states of 10 segments


def test_bitwise_reproducible(pkg, dev):
    inp = so.make_inputs(2, 130, 200, 16, seed=61)
    a = run_gpu_fwd_bwd(pkg, inp, dev)
    b = run_gpu_fwd_bwd(pkg, inp, dev)
    for k in a:
        assert torch.equal(a[k], b[k]), k


def test_chunk_split_consistency_with_carried_state(pkg, dev):
    # scan of a concatenation == scan of the second half started from the first half's state
    inp = so.make_inputs(2, 120, 64, 16, seed=71)
    g = {k: v.to(dev) for k, v in inp.items()}
    with torch.no_grad():
        y_full, h_full = pkg.selective_scan_fn(g["x"], g["delta"], g["A"], g["B"], g["C"], g["D"],
                                               return_last_state=True)
        cut = 53
        y1, h1 = pkg.selective_scan_fn(g["x"][:, :cut], g["delta"][:, :cut], g["A"], g["B"][:, :cut],
                                       g["C"][:, :cut], g["D"], return_last_state=True)
        y2, h2 = pkg.selective_scan_fn(g["x"][:, cut:], g["delta"][:, cut:], g["A"], g["B"][:, cut:],
                                       g["C"][:, cut:], g["D"], h0=h1, return_last_state=True)
    assert rel_err(torch.cat([y1, y2], 1), y_full) <= 1e-6
    assert rel_err(h2, h_full) <= 1e-6


def test_long_sequence_fp32_and_segmented_inference(pkg, dev):
    # 50 000 steps, far beyond the benchmark shapes (the reference materialises (B, L, ED, N)
    # tensors and pads L to a power of two, pscan.py:165-174): forward + backward
    # against the float64 C oracle, then the same forward without gradients, which the library
    # cuts into parallel segments by itself (one batch row, two channel groups)
    inp = so.make_inputs(1, 50000, 96, 16, seed=4242)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.float32], "L=50000")
    with torch.no_grad():
        y = pkg.selective_scan_fn(*[inp[k].to(dev) for k in ("x", "delta", "A", "B", "C", "D")])
    assert rel_err(y, ref["y"]) <= TOL[torch.float32]
    # zero-length and zero-batch inputs are rejected, not undefined
    for shape in ((1, 0, 8), (0, 4, 8)):
        x = torch.zeros(*shape, device=dev)
        bc = torch.zeros(shape[0], shape[1], 16, device=dev)
        with pytest.raises(RuntimeError):
            pkg.selective_scan(x, x, inp["A"][:8].to(dev), bc, bc, inp["D"][:8].to(dev))


def test_config1_full_size_fp32(pkg, dev):
    # configs[1]: B=8, L=2048, ED=1536, N=16 float32, against the float64 C oracle
    inp = so.make_inputs(8, 2048, 1536, 16, seed=1001)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.float32], "config1")


def test_config2_full_size_bf16(pkg, dev):
    # configs[2], the headline shape: B=4, L=4096, ED=4096, N=16, bf16 I/O, float32 state
    inp = so.make_inputs(4, 4096, 4096, 16, seed=1002, dtype=torch.bfloat16)
    ref = c_oracle.sscan_fwd_bwd(**inp)
    got = run_gpu_fwd_bwd(pkg, inp, dev)
    _check(got, ref, TOL[torch.bfloat16], "config2")


def test_errors_are_reported_not_undefined(pkg, dev):
    inp = so.make_inputs(1, 8, 8, 16, seed=81)
    g = {k: v.to(dev) for k, v in inp.items()}
    with pytest.raises(RuntimeError):
        pkg.selective_scan(g["x"], g["delta"][:, :4], g["A"], g["B"], g["C"], g["D"])
    with pytest.raises(TypeError):
        pkg.selective_scan(g["x"].double(), g["delta"].double(), g["A"], g["B"].double(),
                           g["C"].double(), g["D"])
    with pytest.raises(RuntimeError):
        pkg.selective_scan(inp["x"], inp["delta"], inp["A"], inp["B"], inp["C"], inp["D"])  # CPU


@pytest.mark.parametrize("seed", range(40))
def test_random_shapes_layouts_and_options(pkg, dev, seed):
    # seeded sweep over ragged shapes, both memory layouts, fp32 / bf16, gate + softplus + bias, initial
    # state: forward, last state and every gradient against the float64 definition
    _random_case(pkg, dev, seed, wide=False)


@pytest.mark.parametrize("seed", range(100, 116))
def test_random_wide_state_directions_and_segments(pkg, dev, seed):
    # the same sweep at d_state 40 ... 256 (passes over blocks of states), in either direction and with
    # the sequence cut into segments
    _random_case(pkg, dev, seed, wide=True)


def _random_case(pkg, dev, seed, wide):
    import contextlib
    import random
    rnd = random.Random(1234 + seed)
    Bs, L = rnd.randint(1, 3), rnd.choice([1, 2, 15, 16, 17, 31, 33, 47, 64, 65, 100, 129, 200])
    ED = rnd.choice([1, 3, 31, 63, 64, 65, 96, 128, 130, 200])
    N = rnd.choice([1, 2, 4, 7, 8, 12, 15, 16, 16, 16, 16, 24, 32, 64])
    dtype = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
    gated, tmajor, with_h0 = rnd.random() < 0.5, rnd.random() < 0.4, rnd.random() < 0.5
    reverse, nseg = False, None
    if wide:
        N = rnd.choice([40, 65, 80, 96, 128, 130, 200, 256])
        ED = rnd.choice([3, 31, 64, 65, 96])
        L = rnd.choice([1, 17, 33, 64, 100, 129])
        reverse, nseg = rnd.random() < 0.5, rnd.choice([None, None, 2, 3])
    inp = so.make_inputs(Bs, L, ED, N, seed=9000 + seed, dtype=dtype)
    g = torch.Generator().manual_seed(9100 + seed)
    z = torch.randn(Bs, L, ED, generator=g).to(dtype)
    raw = (torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0).to(dtype)
    bias = torch.randn(ED, generator=g) * 0.3
    h0 = torch.randn(Bs, ED, N, generator=g) if with_h0 else None
    f64 = lambda t: t.double().requires_grad_()
    x, dl, A, Bm, C, D = map(f64, (inp["x"], raw if gated else inp["delta"], inp["A"], inp["B"], inp["C"], inp["D"]))
    zz, bb = f64(z), f64(bias)
    delta = so.softplus_ref(dl + bb) if gated else dl
    fl = (lambda t: t.flip(1)) if reverse else (lambda t: t)
    yr, hl = so.selective_scan_ref(fl(x), fl(delta), A, fl(Bm), fl(C), D, h0=None if h0 is None else h0.double(),
                                   return_last_state=True)
    yr = fl(yr)
    if gated:
        yr = yr * (zz * torch.sigmoid(zz))
    yr.backward(inp["dy"].double())
    ref = dict(y=yr, hl=hl, dx=x.grad, ddelta=dl.grad, dA=A.grad, dB=Bm.grad, dC=C.grad, dD=D.grad)
    if gated:
        ref.update(dz=zz.grad, dbias=bb.grad)

    def lay(t):  # (B, L, ED) values in (B, ED, L) memory, the layout MambaBlock.forward produces
        t = t.to(dev)
        return t.transpose(1, 2).contiguous().transpose(1, 2) if tmajor else t
    gx = lay(inp["x"]).requires_grad_()
    gd = lay(raw if gated else inp["delta"]).requires_grad_()
    gz = lay(z).requires_grad_()
    gA, gB, gC, gD, gb = (t.to(dev).requires_grad_() for t in (inp["A"], inp["B"], inp["C"], inp["D"], bias))
    kw = dict(z=gz, delta_bias=gb, delta_softplus=True) if gated else {}
    plan = pkg.plan_override(fwd_segments=nseg, bwd_segments=nseg) if nseg else contextlib.nullcontext()
    with plan:
        y, hg = pkg.selective_scan_fn(gx, gd, gA, gB, gC, gD, h0=None if h0 is None else h0.to(dev),
                                      return_last_state=True, reverse=reverse, **kw)
        y.backward(inp["dy"].to(dev))
    got = dict(y=y, hl=hg, dx=gx.grad, ddelta=gd.grad, dA=gA.grad, dB=gB.grad, dC=gC.grad, dD=gD.grad)
    if gated:
        got.update(dz=gz.grad, dbias=gb.grad)
    tol = TOL[dtype]
    what = f"B{Bs} L{L} ED{ED} N{N} {dtype} gated={gated} tmajor={tmajor} h0={with_h0} reverse={reverse} nseg={nseg}"
    for k in ref:
        scale = ref[k].abs().max().item()
        if scale == 0.0:
            assert got[k].abs().max().item() == 0.0, f"{what}: {k}"
            continue
        e = rel_err(got[k], ref[k])
        assert e <= (TOL[torch.float32] if k == "hl" and dtype == torch.float32 else tol), f"{what}: {k} rel err {e:.3e}"


def test_config2_shape_gated_softplus_bf16_channel_slice(pkg, dev):
    # The fused form a Mamba layer actually calls (gate + softplus + bias) at the headline shape,
    # B=4, L=4096, ED=4096, N=16, bf16 I/O.  Channels are independent, so y, dx, ddelta, dz and
    # the per-channel gradients dA, dD, dbias of a 16-channel slice of the full-size run must
    # match the float64 oracle run on that slice alone (dB/dC sum over all channels and are
    # covered at full size by the ungated test above).
    Bs, L, ED, N, S = 4, 4096, 4096, 16, 16
    dt = torch.bfloat16
    inp = so.make_inputs(Bs, L, ED, N, seed=1002, dtype=dt)
    g = torch.Generator().manual_seed(2002)
    z = torch.randn(Bs, L, ED, generator=g).to(dt)
    raw = (torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0).to(dt)
    bias = torch.randn(ED, generator=g) * 0.3
    t = lambda v: v.to(dev).requires_grad_()
    gx, gr, gA, gB, gC, gD, gz, gb = map(t, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    y = pkg.selective_scan_fn(gx, gr, gA, gB, gC, gD, z=gz, delta_bias=gb, delta_softplus=True)
    y.backward(inp["dy"].to(dev))
    sl = slice(1016, 1016 + S)  # a slice that straddles two 64-channel groups (boundary at 1024)
    f64 = lambda v: v.double().requires_grad_()
    x, r, A, Dd, zz, bb = map(f64, (inp["x"][..., sl], raw[..., sl], inp["A"][sl], inp["D"][sl], z[..., sl], bias[sl]))
    Bm, C = inp["B"].double(), inp["C"].double()
    yr = so.selective_scan_ref(x, so.softplus_ref(r + bb), A, Bm, C, Dd)
    yr = yr * (zz * torch.sigmoid(zz))
    yr.backward(inp["dy"][..., sl].double())
    tol = TOL[dt]
    assert rel_err(y[..., sl], yr) <= tol
    assert rel_err(gx.grad[..., sl], x.grad) <= tol
    assert rel_err(gr.grad[..., sl], r.grad) <= tol
    assert rel_err(gz.grad[..., sl], zz.grad) <= tol
    assert rel_err(gA.grad[sl], A.grad) <= tol
    assert rel_err(gD.grad[sl], Dd.grad) <= tol
    assert rel_err(gb.grad[sl], bb.grad) <= tol


def _gated_reference_from_c_oracle(inp, raw, z, bias):
    """Gate + softplus + bias around the float64 C oracle by the chain rule: the oracle runs the plain
    scan on delta = softplus(raw + bias) with the upstream gradient dy * silu(z); dz, d raw and d bias
    follow element-wise in float64.  Everything a fused call returns, at any size the C oracle handles."""
    rd, zd, dyd = raw.double(), z.double(), inp["dy"].double()
    pre = rd + bias.double()
    delta = so.softplus_ref(pre)
    sg = torch.sigmoid(zd)
    silu = zd * sg
    ref = c_oracle.sscan_fwd_bwd(inp["x"], delta, inp["A"], inp["B"], inp["C"], inp["D"], dyd * silu)
    y_pre = ref["y"]
    out = dict(ref)
    out["y"] = y_pre * silu
    out["dz"] = dyd * y_pre * (sg * (1 + zd * (1 - sg)))
    out["ddelta"] = ref["ddelta"] * torch.sigmoid(pre)      # d softplus(v)/dv = sigmoid(v)
    out["dbias"] = out["ddelta"].sum(dim=(0, 1))
    return out


def test_gated_reference_composition_is_the_autograd_oracle():
    # pins the helper above (no GPU work): on a small case it equals plain float64 autograd through the
    # definition with gate and softplus written out
    inp = so.make_inputs(2, 37, 20, 16, seed=71)
    g = torch.Generator().manual_seed(72)
    z = torch.randn(2, 37, 20, generator=g)
    raw = torch.randn(2, 37, 20, generator=g) * 0.5 - 4.0
    bias = torch.randn(20, generator=g) * 0.3
    ref = _gated_reference_from_c_oracle(inp, raw, z, bias)
    f64 = lambda v: v.double().requires_grad_()
    x, r, A, Bm, C, D, zz, bb = map(f64, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    y = so.selective_scan_ref(x, so.softplus_ref(r + bb), A, Bm, C, D) * (zz * torch.sigmoid(zz))
    y.backward(inp["dy"].double())
    want = dict(y=y, dx=x.grad, ddelta=r.grad, dA=A.grad, dB=Bm.grad, dC=C.grad, dD=D.grad, dz=zz.grad, dbias=bb.grad)
    for k, v in want.items():
        assert rel_err(ref[k], v) <= 1e-6, k      # (the C oracle takes its inputs as float32)


def test_config2_full_size_gated_softplus_bf16(pkg, dev):
    # configs[2] in the fused form a Mamba layer calls (gate, softplus, bias inside the kernels), bf16
    # I/O, EVERY output at full size against the float64 C oracle: dB and dC are sums over all 4096
    # channels and a channel slice cannot check them
    Bs, L, ED, N = 4, 4096, 4096, 16
    dt = torch.bfloat16
    inp = so.make_inputs(Bs, L, ED, N, seed=1002, dtype=dt)
    g = torch.Generator().manual_seed(2002)
    z = torch.randn(Bs, L, ED, generator=g).to(dt)
    raw = (torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0).to(dt)
    bias = torch.randn(ED, generator=g) * 0.3
    ref = _gated_reference_from_c_oracle(inp, raw, z, bias)
    t = lambda v: v.to(dev).requires_grad_()
    gx, gr, gA, gB, gC, gD, gz, gb = map(t, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    y = pkg.selective_scan_fn(gx, gr, gA, gB, gC, gD, z=gz, delta_bias=gb, delta_softplus=True)
    y.backward(inp["dy"].to(dev))
    got = dict(y=y, dx=gx.grad, ddelta=gr.grad, dA=gA.grad, dB=gB.grad, dC=gC.grad, dD=gD.grad, dz=gz.grad,
               dbias=gb.grad)
    for k in ref:
        e = rel_err(got[k], ref[k])
        assert e <= TOL[dt], f"gated config2: {k} rel err {e:.3e}"


def test_config4_scan_shape_full_size_gated_bf16(pkg, dev):
    # the scan of one layer of configs[4] (B=8, L=4096, ED=1536, N=16, gate + softplus + bias, bf16):
    # 192 workgroups of 64 channels would leave a quarter of the chip idle, so the forward runs as 256
    # workgroups of 48 channels; every output at full size against the float64 C oracle
    Bs, L, ED, N = 8, 4096, 1536, 16
    dt = torch.bfloat16
    inp = so.make_inputs(Bs, L, ED, N, seed=1004, dtype=dt)
    g = torch.Generator().manual_seed(2004)
    z = torch.randn(Bs, L, ED, generator=g).to(dt)
    raw = (torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0).to(dt)
    bias = torch.randn(ED, generator=g) * 0.3
    ref = _gated_reference_from_c_oracle(inp, raw, z, bias)
    t = lambda v: v.to(dev).requires_grad_()
    gx, gr, gA, gB, gC, gD, gz, gb = map(t, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    y = pkg.selective_scan_fn(gx, gr, gA, gB, gC, gD, z=gz, delta_bias=gb, delta_softplus=True)
    y.backward(inp["dy"].to(dev))
    got = dict(y=y, dx=gx.grad, ddelta=gr.grad, dA=gA.grad, dB=gB.grad, dC=gC.grad, dD=gD.grad, dz=gz.grad,
               dbias=gb.grad)
    for k in ref:
        e = rel_err(got[k], ref[k])
        assert e <= TOL[dt], f"gated config4 scan: {k} rel err {e:.3e}"


# ---------------------------------------------------------------------------------------------
# float32 delta next to bfloat16 tensors (the reference's call under torch.autocast)
# ---------------------------------------------------------------------------------------------

def _mixed_inputs(Bs, L, ED, N, seed):
    """x, B, C, dy rounded to bfloat16, delta kept in float32: what MambaBlock.selective_scan receives
    under autocast (softplus output is float32, mambapy/mamba.py:264-265)."""
    inp = so.make_inputs(Bs, L, ED, N, seed=seed)
    for k in ("x", "B", "C", "dy"):
        inp[k] = inp[k].to(torch.bfloat16)
    return inp


@pytest.mark.parametrize("tmajor", [False, True])
@pytest.mark.parametrize("Bs,L,ED,N", [(2, 300, 192, 16), (1, 77, 100, 16), (2, 64, 70, 40)])
def test_bf16_tensors_with_float32_delta(pkg, dev, Bs, L, ED, N, tmajor):
    inp = _mixed_inputs(Bs, L, ED, N, seed=4000 + L)
    ref = c_oracle.sscan_fwd_bwd(**inp)          # on the UNROUNDED delta

    def lay(v):
        v = v.to(dev)
        return (v.transpose(1, 2).contiguous().transpose(1, 2) if tmajor else v).requires_grad_()
    gx, gd = lay(inp["x"]), lay(inp["delta"])
    gA, gB, gC, gD = (inp[k].to(dev).requires_grad_() for k in ("A", "B", "C", "D"))
    y = pkg.selective_scan_fn(gx, gd, gA, gB, gC, gD)
    y.backward(inp["dy"].to(dev))
    assert y.dtype == torch.bfloat16 and gd.grad.dtype == torch.float32 and gx.grad.dtype == torch.bfloat16
    got = dict(y=y, dx=gx.grad, ddelta=gd.grad, dA=gA.grad, dB=gB.grad, dC=gC.grad, dD=gD.grad)
    for k in ref:
        # ddelta, dA and dD leave the kernels as float32: the float32 bar applies to them
        tol = TOL[torch.float32] if k in ("ddelta", "dA", "dD") else TOL[torch.bfloat16]
        e = rel_err(got[k], ref[k])
        assert e <= tol, f"{k} rel err {e:.3e} > {tol}"
    # and the unrounded delta is what was used: with delta rounded to bfloat16 the float32 outputs
    # are further from this oracle than the bar above
    rounded = dict(inp, delta=inp["delta"].to(torch.bfloat16))
    far = run_gpu_fwd_bwd(pkg, rounded, dev)
    assert rel_err(far["dA"], ref["dA"]) > 10 * rel_err(got["dA"], ref["dA"])


def test_float32_delta_gated_reverse_and_cut(pkg, dev):
    # the same with softplus + bias + gate inside the kernels, the walk reversed and the sequence cut
    Bs, L, ED, N = 2, 200, 130, 16
    inp = _mixed_inputs(Bs, L, ED, N, seed=4100)
    g = torch.Generator().manual_seed(4101)
    z = torch.randn(Bs, L, ED, generator=g).to(torch.bfloat16)
    raw = torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0       # float32
    bias = torch.randn(ED, generator=g) * 0.3
    fl = lambda v: v.flip(1)
    finp = {k: (fl(v) if v.dim() == 3 else v) for k, v in inp.items()}
    ref = _gated_reference_from_c_oracle(finp, fl(raw), fl(z), bias)
    ref = {k: (fl(v) if v.dim() == 3 else v) for k, v in ref.items()}
    t = lambda v: v.to(dev).requires_grad_()
    gx, gr, gA, gB, gC, gD, gz, gb = map(t, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], z, bias))
    with pkg.plan_override(fwd_segments=3, bwd_segments=3):
        y = pkg.selective_scan_fn(gx, gr, gA, gB, gC, gD, z=gz, delta_bias=gb, delta_softplus=True, reverse=True)
        y.backward(inp["dy"].to(dev))
    assert gr.grad.dtype == torch.float32
    got = dict(y=y, dx=gx.grad, ddelta=gr.grad, dA=gA.grad, dB=gB.grad, dC=gC.grad, dD=gD.grad, dz=gz.grad,
               dbias=gb.grad)
    for k in ref:
        tol = TOL[torch.float32] if k in ("ddelta", "dA", "dD", "dbias") else TOL[torch.bfloat16]
        e = rel_err(got[k], ref[k])
        assert e <= tol, f"{k} rel err {e:.3e} > {tol}"


@pytest.mark.parametrize("Bs,L,ED,N,dtype,gated", [
    (2, 100, 48, 16, torch.float32, False), (1, 33, 47, 16, torch.float32, True), (2, 200, 150, 12, torch.bfloat16, True),
    (3, 64, 200, 16, torch.bfloat16, False), (1, 17, 1, 3, torch.float32, False),
])
def test_forward_group_sizes_agree_bit_for_bit(pkg, dev, Bs, L, ED, N, dtype, gated):
    # Workgroups of 64 or of 48 channels are two mappings of lanes to (channel, state group) for the same
    # arithmetic in the same order: outputs, checkpoints (through the backward) and last states are equal
    # bit for bit, and both match the oracle.
    inp = so.make_inputs(Bs, L, ED, N, seed=5000 + ED, dtype=dtype)
    g = torch.Generator().manual_seed(5001)
    z = torch.randn(Bs, L, ED, generator=g).to(dtype)
    raw = (torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0).to(dtype)
    bias = torch.randn(ED, generator=g) * 0.3
    h0 = torch.randn(Bs, ED, N, generator=g)
    outs = []
    for ch in (64, 48):
        t = lambda v: v.to(dev).requires_grad_()
        gx, gd, gA, gB, gC, gD, gz, gb = map(t, (inp["x"], raw if gated else inp["delta"], inp["A"], inp["B"], inp["C"],
                                               inp["D"], z, bias))
        kw = dict(z=gz, delta_bias=gb, delta_softplus=True) if gated else {}
        with pkg.plan_override(group_channels=ch):
            y, hl = pkg.selective_scan_fn(gx, gd, gA, gB, gC, gD, h0=h0.to(dev), return_last_state=True, **kw)
            y.backward(inp["dy"].to(dev))
        outs.append((y.detach(), hl, gx.grad, gd.grad, gA.grad, gB.grad, gC.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    if not gated:
        ref, hr = c_oracle.sscan_fwd(*[inp[k] for k in ("x", "delta", "A", "B", "C", "D")], h0=h0, return_last_state=True)
        assert rel_err(outs[1][0], ref) <= TOL[dtype] and rel_err(outs[1][1], hr) <= TOL[dtype]
