"""Stream order and re-entrancy of the entry points.

The reference's operator holds no global state and runs on PyTorch's current stream; its
backward is called from the autograd engine's own thread (mambapy/pscan.py:151-224 is a
`torch.autograd.Function`).  The library must therefore launch on the stream it is handed,
wait for nothing itself, and give the same bits when several host threads call it at once.
All streams here have the default priority."""
import threading

import pytest
import torch

from oracle import scan_oracle as so
from util import GRAD_KEYS, TOL, rel_err, run_gpu_fwd_bwd

pytestmark = pytest.mark.gpu


def _late_copy(src, stream_work):
    """A copy of `src` that is written at the END of a long chain of work queued on the current
    stream: whoever reads it on another stream, or before the chain has run, sees other bytes."""
    out = torch.full_like(src, float("nan"))
    acc = stream_work
    for _ in range(60):
        acc = (acc @ stream_work).clamp_(-1.0, 1.0)
    out.copy_(src + 0.0 * acc.sum().to(src.dtype))
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_calls_run_on_the_current_stream_in_order(pkg, dev, dtype):
    inp = so.make_inputs(2, 300, 130, 16, seed=71, dtype=dtype)
    base = run_gpu_fwd_bwd(pkg, inp, dev)
    side = torch.cuda.Stream(device=dev)
    work = torch.randn(1024, 1024, device=dev) * 0.03
    torch.cuda.synchronize()
    names = ("x", "delta", "A", "B", "C", "D")
    with torch.cuda.stream(side):
        # the inputs only exist once `side` has run its queue; nothing waits for it on the host
        args = [_late_copy(inp[k].to(dev), work).requires_grad_() for k in names]
        dy = _late_copy(inp["dy"].to(dev), work)
        y = pkg.selective_scan_fn(*args)
        y.backward(dy)
    side.synchronize()
    assert torch.equal(y.detach(), base["y"])
    for k, a in zip(GRAD_KEYS, args):
        assert torch.equal(a.grad, base[k]), k
    # and the result is right, not merely repeatable
    ref = so.selective_scan_grads_autograd(**inp)
    assert rel_err(y, ref["y"]) <= TOL[dtype]
    assert rel_err(args[0].grad, ref["dx"]) <= TOL[dtype]


def test_generic_scan_and_step_follow_the_current_stream(pkg, dev):
    g = torch.Generator().manual_seed(72)
    A = (torch.rand(2, 77, 12, 16, generator=g) * 0.9 + 0.05).to(dev)
    X = torch.randn(2, 77, 12, 16, generator=g).to(dev)
    H0 = pkg.pscan(A, X)
    x, dl = torch.randn(3, 40, generator=g).to(dev), torch.rand(3, 40, generator=g).to(dev) * 0.1
    Am = -torch.arange(1, 17, dtype=torch.float32).repeat(40, 1).to(dev)
    Bm, C = torch.randn(3, 16, generator=g).to(dev), torch.randn(3, 16, generator=g).to(dev)
    D, h = torch.ones(40, device=dev), torch.randn(3, 40, 16, generator=g).to(dev)
    y0, h0 = pkg.ssm_step(x, dl, Am, Bm, C, D, h)
    side = torch.cuda.Stream(device=dev)
    work = torch.randn(1024, 1024, device=dev) * 0.03
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        H1 = pkg.pscan(_late_copy(A, work), _late_copy(X, work))
        y1, h1 = pkg.ssm_step(_late_copy(x, work), dl, Am, Bm, C, D, _late_copy(h, work))
    side.synchronize()
    assert torch.equal(H1, H0) and torch.equal(y1, y0) and torch.equal(h1, h0)


def test_host_threads_on_their_own_streams_get_the_serial_bits(pkg, dev):
    """Four host threads, each with a stream and a shape of its own (plain, gated bf16, wide state
    in passes, batch 1 cut into segments), ten forward + backward calls each, all at once."""
    cases = [
        dict(shape=(2, 200, 130, 16), dtype=torch.float32, gated=False),
        dict(shape=(3, 129, 96, 16), dtype=torch.bfloat16, gated=True),
        dict(shape=(1, 100, 64, 96), dtype=torch.float32, gated=False),
        dict(shape=(1, 2048, 128, 16), dtype=torch.float32, gated=True),
    ]

    def tensors(i, c):
        Bs, L, ED, N = c["shape"]
        inp = so.make_inputs(Bs, L, ED, N, seed=80 + i, dtype=c["dtype"])
        g = torch.Generator().manual_seed(90 + i)
        z = torch.randn(Bs, L, ED, generator=g).to(c["dtype"]).to(dev) if c["gated"] else None
        return [inp[k].to(dev) for k in ("x", "delta", "A", "B", "C", "D")], z, inp["dy"].to(dev)

    def run(args, z, dy):
        leaves = [a.clone().requires_grad_() for a in args]
        zl = z.clone().requires_grad_() if z is not None else None
        y = pkg.selective_scan_fn(*leaves, z=zl)
        y.backward(dy)
        return [y.detach()] + [a.grad for a in leaves] + ([zl.grad] if zl is not None else [])

    data = [tensors(i, c) for i, c in enumerate(cases)]
    serial = [run(*d) for d in data]
    torch.cuda.synchronize()

    errors, barrier = [], threading.Barrier(len(cases))

    def worker(i):
        try:
            stream = torch.cuda.Stream(device=dev)
            barrier.wait(timeout=60)
            with torch.cuda.stream(stream):
                for _ in range(10):
                    got = run(*data[i])
                    stream.synchronize()
                    for j, (a, b) in enumerate(zip(got, serial[i])):
                        if not torch.equal(a, b):
                            errors.append((i, j))
        except Exception as exc:  # a failure inside a thread must fail the test, not vanish
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert errors == []


@pytest.mark.parametrize("gated", [False, True])
def test_forward_backward_captured_in_a_hip_graph(pkg, dev, gated):
    """The entry points allocate nothing, clear nothing with memset nodes and wait for nothing, so a
    training step of the scan can be recorded once and replayed: three replays on new input values,
    with eager calls and synchronisations in between, each equal to the eager result bit for bit."""
    shape, dtype = (2, 300, 130, 16), torch.bfloat16 if gated else torch.float32
    names = ("x", "delta", "A", "B", "C", "D")

    def values(seed):
        inp = so.make_inputs(*shape, seed=seed, dtype=dtype)
        g = torch.Generator().manual_seed(seed + 1)
        z = torch.randn(shape[0], shape[1], shape[2], generator=g).to(dtype)
        bias = torch.randn(shape[2], generator=g) * 0.3
        return [inp[k] for k in names] + [z, bias, inp["dy"]]

    def call(t):
        kw = dict(z=t[6], delta_bias=t[7], delta_softplus=True) if gated else {}
        y = pkg.selective_scan_fn(*t[:6], **kw)
        leaves = t[:8] if gated else t[:6]
        return (y,) + torch.autograd.grad(y, leaves, t[8])

    static = [v.to(dev) for v in values(100)]
    for t in static[:8]:
        t.requires_grad_()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        for _ in range(3):
            call(static)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = call(static)
    for rep in range(3):
        new = [v.to(dev) for v in values(200 + rep)]
        with torch.no_grad():
            for s_, n_ in zip(static, new):
                s_.copy_(n_)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        for t in new[:8]:
            t.requires_grad_()
        want = call(new)                      # eager, between the replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (rep, i)
