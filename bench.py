#!/usr/bin/env python3
"""Benchmark of the selective-scan hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c1|c0|c3|c4|c4-3000|pscan|thin|block|gated|layer|generate]

One step = one forward + one backward of the fused selective scan over one batch of
seeded synthetic input that is already resident in HBM.  Prints ONE JSON line.
  value      algorithmic GB/s of forward+backward (bytes formula below / time per step)
  roofline   the backward entry point (its two kernels), HIP-event time on the launch stream
  cpu_baseline  the CPU restatement of the reference's Blelloch-scan path (oracle "port"),
             timed on this host on a bounded sample of the same workload
  other      (default workload only) one timed record for each of the other benchmark
             configurations: c1, c3 (decode step), c4 / c4-3000 (LM forward), the generic pscan
             and the batch-1 launches
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOADS = {
    # name: (B, L, ED, N, dtype, seed, description)
    "c0": (2, 64, 32, 16, "float32", 1000, "configs[0]: B=2 L=64 ED=32 N=16 fp32"),
    "c1": (8, 2048, 1536, 16, "float32", 1001, "configs[1]: mamba-130m layer B=8 L=2048 ED=1536 N=16 fp32"),
    "c2": (4, 4096, 4096, 16, "bfloat16", 1002,
           "configs[2]: mamba-1.4b layer B=4 L=4096 ED=4096 N=16, bf16 I/O, fp32 state"),
}

LIBRARY_SHA = None  # mpa_source_hash() of the library that is timed, set in main()


def profile_state(workload):
    """The hardware-counter summary of a workload under profiles/ and whether it describes the
    kernels that run: the summary carries a line `source_sha = <hash of the kernel sources it was
    measured on>`, the loaded library reports the hash of the sources it was built from."""
    import re
    path = os.path.join(ROOT, "profiles", f"sscan_fwd_bwd_{workload}_pmc.md")
    try:
        text = open(path).read()
    except OSError:
        return None, {"file": None, "stale": None}
    m = re.search(r"^\s*source_sha\s*=\s*([0-9a-f]+)", text, flags=re.M)
    sha = m.group(1) if m else None
    stale = sha is None or LIBRARY_SHA is None or sha != LIBRARY_SHA
    return text, {"file": os.path.relpath(path, ROOT), "source_sha": sha, "library_sha": LIBRARY_SHA,
                  "stale": stale}


def _profile_number(workload, pattern):
    import re
    text, st = profile_state(workload)
    if text is None or st["stale"]:
        return None
    m = re.search(pattern, text)
    return float(m.group(1)) if m else None


def measured_traffic_bytes(workload):
    """HBM bytes per launch of the backward entry point, measured with rocprofv3 --pmc (FETCH_SIZE
    + WRITE_SIZE, scaled by a copy kernel of known size).  Read from the summary under profiles/
    (a line `traffic_bytes_per_launch <workload> mpa_sscan_bwd = <number>`); None when that
    workload has no summary or the summary was measured on other kernel sources than the library
    that is being timed (see profile_state)."""
    return _profile_number(workload, rf"traffic_bytes_per_launch\s+{workload}\s+mpa_sscan_bwd\s*=\s*([0-9.eE+-]+)")


def measured_valu_insts(workload, entry):
    """Wave-level VALU instructions per launch of an entry point's scan kernel (rocprofv3 --pmc
    SQ_INSTS_VALU), read from the same summary (a line `valu_insts_per_launch <workload> <entry>
    = <number>`); None when there is none or it is stale."""
    return _profile_number(workload, rf"valu_insts_per_launch\s+{workload}\s+{entry}\s*=\s*([0-9.eE+-]+)")


# Plain fp32 wave64 instructions per second the chip can issue: 1024 SIMDs x 2.4 GHz / 2 clocks
# (the published 157.3 TFLOP/s divided by the 128 flops of one wave-wide FMA).
VALU_PEAK_GINST = 1024 * 2.4 / 2.0


def valu_issue(workload, entry, ms):
    """What actually bounds the scan kernels: the rate of VALU instructions, against the rate of
    plain fp32 instructions (a DPP operand costs about twice, exp2 and lane swaps four times a plain
    instruction, so the attainable fraction of this peak is well below one)."""
    n = measured_valu_insts(workload, entry)
    if n is None:
        return None
    ach = n / (ms * 1e-3) / 1e9
    return {"wave_insts_per_launch": n, "achieved": ach, "peak": VALU_PEAK_GINST,
            "unit": "G wave64 instructions/s", "frac": ach / VALU_PEAK_GINST}


def algorithmic_bytes(B, L, ED, N, s):
    """Bytes that must cross HBM: fwd reads x, delta, B, C, A, D and writes y; bwd reads
    x, delta, dy, B, C, A, D and writes dx, ddelta, dB, dC, dA, dD (s = I/O element size;
    A, D, dA, dD float32).  Checkpoints, partial buffers and recomputation are not counted."""
    fwd = s * (3 * B * L * ED + 2 * B * L * N) + 4 * (ED * N + ED)
    bwd = s * (5 * B * L * ED + 4 * B * L * N) + 4 * (2 * ED * N + 2 * ED)
    return fwd, bwd


def cpu_baseline(workload, torch):
    """Time the reference's pure-PyTorch path (materialised (B,L,ED,N) tensors + Blelloch scan,
    forward + backward, float32, all host threads: the oracle's restatement, kind "port") on
    this host.  configs[0] and [1] run in full; configs[2] runs ONE of its four batch rows at
    full width (batch rows are independent; ten live 1.07 GB tensors instead of 4.3 GB ones) and
    the figures are per row: GB/s and tokens/s do not depend on the number of rows.  One warm-up,
    then the median of three repetitions."""
    # the checker is imported here only: this leg times it, nothing else in the benchmark uses it
    from oracle import scan_oracle as so
    import synthetic_inputs
    B, L, ED, N, _, seed, _ = WORKLOADS[workload]
    bs = 1 if workload == "c2" else B
    threads = int(os.environ.get("OMP_NUM_THREADS") or os.cpu_count() or 1)
    torch.set_num_threads(threads)
    inp = synthetic_inputs.make_inputs(bs, L, ED, N, seed=seed)
    names = ("x", "delta", "A", "B", "C", "D")

    def once(fn):
        args = [inp[k].clone().requires_grad_() for k in names]
        t0 = time.perf_counter()
        y = fn(*args)
        y.backward(inp["dy"])
        return time.perf_counter() - t0

    once(so.selective_scan_blelloch)
    ts = sorted(once(so.selective_scan_blelloch) for _ in range(3))
    dt = ts[1]
    fwd, bwd = algorithmic_bytes(bs, L, ED, N, 4)
    out = {
        "value": (fwd + bwd) / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"B={bs}" + (f" of {B} batch rows" if bs != B else "") +
                  f" L={L} ED={ED} N={N} fp32, fwd+bwd, 1 warm-up + median of 3, {dt * 1e3:.1f} ms each; "
                  "GB/s on the same algorithmic-bytes formula",
        "ms": dt * 1e3, "tokens_per_s": bs * L / dt,
    }
    if workload == "c0":
        # the reference's sequential twin (mambapy/mamba.py:297-327), timed at configs[0] only
        once(so.selective_scan_ref)
        out["sequential_loop_ms"] = sorted(once(so.selective_scan_ref) for _ in range(3))[1] * 1e3
    return out


def _timed(torch, fn, steps, warmup, settle_s=0.05):
    """Wall time per call of fn over `steps` calls, after `warmup` calls and at least `settle_s`
    seconds of the same work (device clocks and the allocator settle within tens of milliseconds;
    a timed window that starts earlier reads 5-20 % slow)."""
    t_start = time.perf_counter()
    n = 0
    while n < warmup or time.perf_counter() - t_start < settle_s:
        fn()
        n += 1
        if n >= warmup:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_decode(args, torch, pkg, dev):
    """configs[3]: decode with cached state at the mamba-2.8b layer shape, batch 64; one bench
    step = 256 tokens through (a) the state-update kernel alone (mpa_ssm_step, in place; the 256
    launches replayed as one HIP graph, and called one by one from Python) and (b) one whole
    MambaBlock.step with its projections, eager and as a HIP graph."""
    Bsz, d_model, ED, N, tokens = 64, 2560, 5120, 16, 256
    g = torch.Generator().manual_seed(1003)
    r = lambda *sh: torch.randn(*sh, generator=g).to(dev)
    # 16 state tensors (336 MB) taken in turn, as the layers of a model would be: one 21 MB state
    # updated in place over and over would stay in the 256 MB last-level cache
    hs = [r(Bsz, ED, N) for _ in range(16)]
    x, dl, z, Bm, C = r(Bsz, ED), r(Bsz, ED), r(Bsz, ED), r(Bsz, N), r(Bsz, N)
    A = -torch.arange(1, N + 1, dtype=torch.float32).repeat(ED, 1).to(dev)
    D, bias = torch.ones(ED, device=dev), r(ED) * 0.1

    def kernel_tokens():
        for i in range(tokens):
            pkg.ssm_step(x, dl, A, Bm, C, D, hs[i % 16], z=z, delta_bias=bias, delta_softplus=True, inplace=True)

    cfg = pkg.MambaConfig(d_model=d_model, n_layers=1, d_state=N)
    block = pkg.MambaBlock(cfg).to(dev)
    cache = (r(Bsz, ED, N), r(Bsz, ED, cfg.d_conv - 1))
    xin = r(Bsz, d_model)

    def block_tokens():
        c = cache
        with torch.no_grad():
            for _ in range(tokens):
                _, c = block.step(xin, c)

    # the same block step recorded once in a HIP graph and replayed per token
    stack = pkg.Mamba(cfg).to(dev)
    stack.layers[0].mixer.load_state_dict(block.state_dict())
    decoder = pkg.GraphedDecoder(stack, [cache])

    def graph_tokens():
        for _ in range(tokens):
            decoder(xin)

    # the kernel-only loop as one HIP graph: per-launch time without the Python call in between
    kernel_tokens()
    torch.cuda.synchronize()
    kgraph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(kgraph):
        kernel_tokens()

    steps, warmup = max(1, args.steps // 10), 1
    t_kernel = _timed(torch, kernel_tokens, steps, warmup) / tokens
    t_kgraph = _timed(torch, kgraph.replay, max(3, steps), warmup) / tokens
    t_block = _timed(torch, block_tokens, steps, warmup) / tokens
    t_graph = _timed(torch, graph_tokens, steps, warmup) / tokens
    bytes_step = 2 * 4 * Bsz * ED * N + 4 * 4 * Bsz * ED + 4 * (ED * N + 2 * ED) + 2 * 4 * Bsz * N
    out = {
        "metric": "decode step latency per token (state-update kernel), mamba-2.8b layer, batch 64",
        "value": t_kgraph * 1e6, "unit": "us/token-step", "higher_is_better": False,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": t_kgraph * tokens * 1e3,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic (seeded)",
        "tokens_per_s_layer_kernel": Bsz / t_kgraph,
        "kernel_step_us_called_from_python": t_kernel * 1e6,
        "block_step_us": t_block * 1e6, "tokens_per_s_layer_block": Bsz / t_block,
        "graphed_layer_step_us": t_graph * 1e6, "tokens_per_s_layer_graphed": Bsz / t_graph,
        "config": {"workload": "configs[3]: decode step, ED=5120 N=16 batch 64, 256 tokens per bench step",
                   "algorithmic_bytes_per_token_step": bytes_step},
        "roofline": {"bound": "hbm", "kernel": "ssm_step_quad_kernel", "achieved": bytes_step / t_kgraph / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bytes_step / t_kgraph / 1e9 / HBM_PEAK_GBS,
                     "traffic": None},
    }
    return out


def bench_pscan(args, torch, pkg, dev):
    """Generic PScan.apply(A, X) on materialised (B, L, ED, N) operands at the configs[1]
    shape, fp32: forward moves 3 tensors, backward 5."""
    B, L, ED, N = 8, 2048, 1536, 16
    g = torch.Generator(device=dev).manual_seed(1005)    # 1.6 GB per tensor: drawn on the GPU
    A = (torch.rand(B, L, ED, N, generator=g, device=dev) * 0.5 + 0.5).requires_grad_()
    X = torch.randn(B, L, ED, N, generator=g, device=dev).requires_grad_()
    gH = torch.randn(B, L, ED, N, generator=g, device=dev)
    steps, warmup = max(3, args.steps // 5), 2

    def step(ev=None):
        A.grad = None
        X.grad = None
        if ev:
            ev[0].record()
        H = pkg.pscan(A, X)
        if ev:
            ev[1].record()
        H.backward(gH)
        if ev:
            ev[2].record()

    t = _timed(torch, step, steps, warmup)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for ev in evs:
        step(ev)
    torch.cuda.synchronize()
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / steps
    S = B * L * ED * N * 4
    out = {
        "metric": "generic pscan(A, X) fwd+bwd GB/s, (8, 2048, 1536, 16) fp32",
        "value": 8 * S / t / 1e9, "unit": "GB/s", "higher_is_better": True,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": t * 1e3,
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic (seeded)",
        "config": {"workload": "PScan.apply on materialised operands, configs[1] shape",
                   "algorithmic_bytes_fwd": 3 * S, "algorithmic_bytes_bwd": 5 * S},
        "roofline": {"bound": "hbm", "kernel": "pscan_bwd_kernel", "achieved": 5 * S / (bwd_ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": 5 * S / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None},
        "forward": {"kernel": "pscan_fwd_kernel", "achieved": 3 * S / (fwd_ms * 1e-3) / 1e9, "unit": "GB/s",
                    "frac": 3 * S / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
    }
    return out


def bench_layer_kernels(args, torch, pkg, dev):
    """The kernels either side of the scan in one layer, at the configs[4] layer shape (B=8,
    L=4096, d_model=768, ED=1536, bf16): causal conv1d + bias + silu reading the x half of the
    in_proj output in place, and RMSNorm with the residual add folded in; forward and backward
    each, timed with HIP events on the launch stream, against the HBM roofline."""
    Bsz, L, D, ED, K = 8, 4096, 768, 1536, 4
    g = torch.Generator().manual_seed(1006)
    bf = torch.bfloat16
    # the x half of an in_proj output, as a leaf: a strided view, no slice node in the timed graph
    xh = torch.randn(Bsz, L, 2 * ED, generator=g).to(bf).to(dev)[..., :ED].requires_grad_()
    w = (torch.randn(ED, 1, K, generator=g) * 0.3).to(dev).requires_grad_()
    b = torch.randn(ED, generator=g).to(dev).requires_grad_()
    gy = torch.randn(Bsz, L, ED, generator=g).to(bf).to(dev)
    h = torch.randn(Bsz, L, D, generator=g).to(bf).to(dev).requires_grad_()
    r = torch.randn(Bsz, L, D, generator=g).to(bf).to(dev).requires_grad_()
    nw = torch.ones(D, device=dev, requires_grad=True)
    gn = torch.randn(Bsz, L, D, generator=g).to(bf).to(dev)
    gt = torch.randn(Bsz, L, D, generator=g).to(bf).to(dev)
    steps, warmup = max(5, args.steps // 2), 3

    def step():
        for t in (xh, w, b, h, r, nw):
            t.grad = None
        pkg.causal_conv1d_fn(xh, w, b).backward(gy)
        n, total = pkg.add_rmsnorm_fn(h, r, nw, 1e-5)
        torch.autograd.backward([n, total], [gn, gt])

    t = _timed(torch, step, steps, warmup)

    # The kernels run 40-80 us each, less than the Python and autograd work around one call, so
    # their durations are taken from the C entry points called back to back on preallocated
    # buffers (HIP events around `reps` launches on the launch stream).
    import ctypes
    lib, ptr, stream = pkg._lib.load(), pkg.scan._ptr, pkg.scan._stream(dev)
    io = pkg.scan._io_dtype(h)
    x_ = xh.detach()
    w2, b1 = w.detach().view(ED, K).contiguous(), b.detach()
    y, dxc = torch.empty(Bsz, L, ED, dtype=bf, device=dev), torch.empty(Bsz, L, ED, dtype=bf, device=dev)
    dwc, dbc = torch.empty(ED, K, device=dev), torch.empty(ED, device=dev)
    sh_f = pkg.conv._conv_shape(x_, y, y, K, True)
    sh_b = pkg.conv._conv_shape(x_, gy, dxc, K, True)
    nb_c = lib.mpa_conv1d_bwd_workspace_bytes(ctypes.byref(sh_b))
    ws_c = torch.empty(nb_c, dtype=torch.uint8, device=dev)
    rows = Bsz * L
    hn, rn, nwd = h.detach(), r.detach(), nw.detach()
    yn, tot, dxn = torch.empty_like(hn), torch.empty_like(hn), torch.empty_like(hn)
    dwn = torch.empty(D, device=dev)
    nb_n = lib.mpa_rmsnorm_bwd_workspace_bytes(rows, D)
    ws_n = torch.empty(nb_n, dtype=torch.uint8, device=dev)
    calls = [
        lambda: lib.mpa_conv1d_fwd(ctypes.byref(sh_f), ptr(x_), ptr(w2), ptr(b1), None, ptr(y), None, stream),
        lambda: lib.mpa_conv1d_bwd(ctypes.byref(sh_b), ptr(x_), ptr(w2), ptr(b1), None, ptr(gy), ptr(dxc), ptr(dwc),
                                   ptr(dbc), ptr(ws_c), nb_c, stream),
        lambda: lib.mpa_rmsnorm_fwd(ptr(hn), ptr(rn), ptr(nwd), ptr(yn), ptr(tot), None, rows, D, 1e-5, io, stream),
        lambda: lib.mpa_rmsnorm_bwd(ptr(tot), ptr(nwd), ptr(gn), ptr(gt), ptr(dxn), ptr(dwn), rows, D, 1e-5, io,
                                    ptr(ws_n), nb_n, stream),
    ]
    reps, ms = 20, []
    for call in calls:
        for _ in range(3):
            pkg._lib.check(call(), "layer kernel")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms.append(e0.elapsed_time(e1) / reps)
    ce, ne = Bsz * L * ED * 2, Bsz * L * D * 2          # bytes of one conv / norm activation tensor
    # conv: fwd x in, y out; bwd x, dy in, dx out.  norm+add: fwd x, residual in, y, sum out;
    # bwd sum, dy, dsum in, dx out.
    alg = [2 * ce, 3 * ce, 4 * ne, 4 * ne]
    names = ["conv1d_fwd_kernel", "conv1d_bwd_kernel (+ finish)", "rmsnorm_fwd_kernel (+ residual add)",
             "rmsnorm_bwd_kernel (+ finish)"]
    per = [{"kernel": k, "ms": m, "algorithmic_bytes": a, "achieved": a / (m * 1e-3) / 1e9, "unit": "GB/s",
            "frac": a / (m * 1e-3) / 1e9 / HBM_PEAK_GBS} for k, m, a in zip(names, ms, alg)]
    slow = max(per, key=lambda e: e["ms"])
    out = {
        "metric": "conv1d + add-RMSNorm kernels fwd+bwd GB/s, mamba-130m layer shape B=8 L=4096 bf16",
        "value": sum(alg) / t / 1e9, "unit": "GB/s", "higher_is_better": True,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": t * 1e3,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 arithmetic, bf16 I/O", "data": "synthetic (seeded)",
        "config": {"workload": "configs[4] layer shape: conv over the x half of (8,4096,3072), norm of (8,4096,768)"},
        "roofline": {"bound": "hbm", "kernel": slow["kernel"], "achieved": slow["achieved"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": slow["frac"], "traffic": None},
        "kernels": per,
    }
    return out


def bench_gated(args, torch, pkg, dev):
    """The fused form of the scan as a layer calls it (mambapy/mamba.py:252-261 reaches it through
    `use_cuda`): softplus(delta + bias) and the gate y * silu(z) inside the kernels, forward +
    backward, at the configs[2] shape and at the configs[4] layer shape, bf16 I/O.  Beside it the
    same computation with the two element-wise steps left to PyTorch around the plain scan (what the
    reference's pscan path does, mamba.py:264-270 and :229-231): four more passes over (B, L, ED)
    tensors per direction."""
    import torch.nn.functional as F
    import synthetic_inputs
    rows = {}
    steps = max(5, args.steps // 2)
    for name, (B, L, ED, N) in (("B4_L4096_ED4096", (4, 4096, 4096, 16)), ("B8_L4096_ED1536", (8, 4096, 1536, 16))):
        inp = synthetic_inputs.make_inputs(B, L, ED, N, seed=1007, dtype=torch.bfloat16)
        g = torch.Generator().manual_seed(1008)
        leaf = lambda t: t.to(dev).requires_grad_()
        x, A, Bm, C, D = (leaf(inp[k]) for k in ("x", "A", "B", "C", "D"))
        raw = leaf((torch.randn(B, L, ED, generator=g) * 0.5 - 4.0).to(torch.bfloat16))
        z = leaf(torch.randn(B, L, ED, generator=g).to(torch.bfloat16))
        bias = leaf(torch.randn(ED, generator=g) * 0.3)
        dy = inp["dy"].to(dev)
        leaves = (x, raw, A, Bm, C, D, z, bias)

        def fused(ev=None):
            for t in leaves:
                t.grad = None
            if ev:
                ev[0].record()
            y = pkg.selective_scan_fn(x, raw, A, Bm, C, D, z=z, delta_bias=bias, delta_softplus=True)
            if ev:
                ev[1].record()
            y.backward(dy)
            if ev:
                ev[2].record()

        def unfused():
            for t in leaves:
                t.grad = None
            delta = F.softplus(raw + bias.to(raw.dtype))
            y = pkg.selective_scan_fn(x, delta, A, Bm, C, D) * F.silu(z)
            y.backward(dy)

        t_f = _timed(torch, fused, steps, 3, settle_s=0.3)
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
        for e in evs:
            fused(e)
        torch.cuda.synchronize()
        fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / len(evs)
        bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / len(evs)
        t_u = _timed(torch, unfused, steps, 3, settle_s=0.3)
        # fused: fwd reads x, delta, z, B, C and writes y; bwd reads x, delta, z, dy, B, C and
        # writes dx, ddelta, dz, dB, dC (the saved pre-gate output is not counted)
        s_ = 2
        alg = s_ * (4 * B * L * ED + 2 * B * L * N) + s_ * (7 * B * L * ED + 4 * B * L * N) + 4 * (3 * ED * N + 5 * ED)
        rows[name] = {"ms_fused": t_f * 1e3, "fwd_ms": fwd_ms, "bwd_ms": bwd_ms, "ms_elementwise_outside": t_u * 1e3,
                      "speedup": t_u / t_f, "GBps_fused": alg / t_f / 1e9, "tokens_per_s_fused": B * L / t_f}
        del x, raw, z, dy, leaves, inp
        torch.cuda.empty_cache()
    first = rows["B4_L4096_ED4096"]
    return {
        "metric": "fused softplus(delta+bias) + scan + gate fwd+bwd GB/s, B=4 L=4096 ED=4096 N=16 bf16",
        "value": first["GBps_fused"], "unit": "GB/s", "higher_is_better": True, "n_gpus": 1, "steps": steps, "warmup": 3,
        "ms_per_step": first["ms_fused"], "fwd_ms": first["fwd_ms"], "bwd_ms": first["bwd_ms"],
        "pct_hbm_peak": 100.0 * first["GBps_fused"] / HBM_PEAK_GBS, "tokens_per_s": first["tokens_per_s_fused"],
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 state/accumulation, bf16 I/O", "data": "synthetic (seeded)",
        "rows": rows,
        "config": {"workload": "scan with softplus, bias and gate inside the kernels: configs[2] shape and configs[4] layer shape"},
    }


def bench_generate(args, torch, pkg, dev):
    """Generation with the mamba-130m architecture (random-init, bf16): one prefill of a 512-token
    prompt, then 128 greedy tokens, (a) with LM.step per token, (b) with the step replayed as a
    HIP graph, and, for scale, (c) the reference's way of generating (mambapy/lm.py:119-155: the
    whole sequence goes through forward again for every new token), timed on 8 tokens."""
    vocab, Lp, new = 50280, 512, 128
    cfg = pkg.MambaConfig(d_model=768, n_layers=24, d_state=16)
    torch.manual_seed(1007)
    model = pkg.LM(cfg, vocab, pad_vocab_size_multiple=8).to(dev).to(torch.bfloat16).eval()
    rows = {}
    for Bsz in (1, 64):
        prompt = torch.randint(0, vocab, (Bsz, Lp), generator=torch.Generator().manual_seed(1007)).to(dev)

        def eager():
            return model.generate(prompt, new)

        def graphed():
            logits, caches = model.prefill(prompt)
            dec = graphed.dec
            for (h, w), (h0, w0) in zip(dec.caches, caches):
                h.copy_(h0)
                w.copy_(w0)
            out = []
            for _ in range(new):
                nxt = logits.argmax(-1)
                out.append(nxt)
                logits = dec(nxt)
            return out

        def rerun():
            seq = prompt
            for _ in range(8):
                logits = model(seq)[:, -1]
                seq = torch.cat([seq, logits.argmax(-1, keepdim=True)], 1)
            return seq

        with torch.no_grad():
            _, caches = model.prefill(prompt)
            graphed.dec = pkg.GraphedDecoder(model, caches)
            t_pre = _timed(torch, lambda: model.prefill(prompt), 5, 2)
            t_eager = _timed(torch, eager, 2, 1)
            t_graph = _timed(torch, graphed, 3, 1)
            t_rerun = _timed(torch, rerun, 2, 1) / 8
        rows[Bsz] = {"prefill_ms": t_pre * 1e3,
                     "eager_step_tokens_per_s": Bsz * new / (t_eager - t_pre),
                     "graphed_step_tokens_per_s": Bsz * new / (t_graph - t_pre),
                     "ms_per_token_step_graphed": (t_graph - t_pre) / new * 1e3,
                     "rerun_forward_tokens_per_s": Bsz / t_rerun}
    out = {
        "metric": "generated tokens/s, mamba-130m architecture, 512-token prompt + 128 new tokens, batch 64",
        "value": rows[64]["graphed_step_tokens_per_s"], "unit": "tokens/s", "higher_is_better": True,
        "n_gpus": 1, "steps": 3, "warmup": 1, "ms_per_step": rows[64]["ms_per_token_step_graphed"],
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16 weights/activations, f32 scan state",
        "data": "synthetic (random-init weights, uniform-random prompt)",
        "config": {"workload": "prefill once + one state-update step per token (HIP graph); batch 1 and 64"},
        "batch_1": rows[1], "batch_64": rows[64],
    }
    return out


def bench_thin(args, torch, pkg, dev):
    """Launches that offer few workgroups: the reference's published regime is batch 1
    (README.md:203-204).  (a) fused scan forward + backward at B=1, L=4096, d_model 1024
    (ED 2048), N=16, bf16: 32 workgroups of 64 channels on 256 CUs unless the sequence is cut;
    (b) generic pscan forward + backward at B=1, L=65536, d_model 16 (ED 32), N=16, fp32: 512
    lanes.  Each is timed as the library runs it (cut into segments) and with the cut switched
    off through the launch plan."""
    import synthetic_inputs
    steps, warmup = max(3, args.steps // 5), 2
    rows = {}

    B, L, ED, N = 1, 4096, 2048, 16
    inp = synthetic_inputs.make_inputs(B, L, ED, N, seed=1010, dtype=torch.bfloat16)
    gpu = [inp[k].to(dev).requires_grad_() for k in ("x", "delta", "A", "B", "C", "D")]
    dy = inp["dy"].to(dev)

    def sscan_step():
        for a in gpu:
            a.grad = None
        pkg.selective_scan_fn(*gpu).backward(dy)

    fwd_b, bwd_b = algorithmic_bytes(B, L, ED, N, 2)
    t_cut = _timed(torch, sscan_step, steps, warmup)
    with pkg.plan_override(fwd_segments=1, bwd_segments=1):
        t_one = _timed(torch, sscan_step, steps, warmup)
    rows["sscan_B1_L4096_ED2048_bf16"] = {
        "ms_cut": t_cut * 1e3, "ms_not_cut": t_one * 1e3, "speedup": t_one / t_cut,
        "GBps_cut": (fwd_b + bwd_b) / t_cut / 1e9, "tokens_per_s_cut": B * L / t_cut}

    B, L, ED, N = 1, 65536, 32, 16
    g = torch.Generator().manual_seed(1011)
    A = (1.0 - torch.rand(B, L, ED, N, generator=g) * 0.05).to(dev).requires_grad_()
    X = torch.randn(B, L, ED, N, generator=g).to(dev).requires_grad_()
    gH = torch.randn(B, L, ED, N, generator=g).to(dev)

    def pscan_step():
        A.grad = None
        X.grad = None
        pkg.pscan(A, X).backward(gH)

    S = B * L * ED * N * 4
    t_cut = _timed(torch, pscan_step, steps, warmup)
    with pkg.plan_override(pscan_chunks=1):
        t_one = _timed(torch, pscan_step, max(2, steps // 2), 1)
    rows["pscan_B1_L65536_ED32_f32"] = {
        "ms_cut": t_cut * 1e3, "ms_not_cut": t_one * 1e3, "speedup": t_one / t_cut,
        "GBps_cut": 8 * S / t_cut / 1e9}

    head = rows["sscan_B1_L4096_ED2048_bf16"]
    out = {
        "metric": "selective-scan fwd+bwd GB/s at batch 1 (B=1 L=4096 ED=2048 N=16 bf16), sequence cut into segments",
        "value": head["GBps_cut"], "unit": "GB/s", "higher_is_better": True,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": head["ms_cut"],
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 state/accumulation, bf16 I/O",
        "data": "synthetic (seeded)",
        "config": {"workload": "batch-1 launches: fused scan B=1 L=4096 ED=2048; generic pscan B=1 L=65536 ED=32"},
        "rows": rows,
    }
    return out


def bench_block(args, torch, pkg, dev):
    """The regime of the reference's own plots (README.md:169-204: one whole MambaBlock, forward +
    backward, batch 1, fp32, timed on an A100 80GB): d_model 1024 and 2048 at N=16, and d_model 1024
    at N = 64, 128, 256, all at L=4096, and d_model 1024, N=16 at L=65536.  `published_ms_*` are the
    reference's figures read off its PNG plots by eye (+-10-15 %, other hardware): context, not a
    like-for-like baseline."""
    steps, warmup = max(3, args.steps // 5), 2
    published = {  # (d_model, N, L): (mamba.py pscan, official CUDA kernel), milliseconds on A100
        (1024, 16, 4096): (49, 26), (2048, 16, 4096): (110, 55), (1024, 64, 4096): (140, 28),
        (1024, 128, 4096): (260, 29), (1024, 256, 4096): (500, 38), (1024, 16, 65536): (760, 410)}
    rows = {}
    B = 1
    for (d_model, N, L), (ref_ms, cuda_ms) in published.items():
        torch.manual_seed(1020 + N)
        blk = pkg.MambaBlock(pkg.MambaConfig(d_model=d_model, n_layers=1, d_state=N)).to(dev)
        x = torch.randn(B, L, d_model, device=dev, requires_grad=True)

        def step():
            x.grad = None
            for prm in blk.parameters():
                prm.grad = None
            blk(x).sum().backward()

        t = _timed(torch, step, steps, warmup)
        rows[f"d_model{d_model}_N{N}" + ("" if L == 4096 else f"_L{L}")] = {
            "ms": t * 1e3, "tokens_per_s": B * L / t,
            "published_ms_mambapy_pscan_A100": ref_ms, "published_ms_official_cuda_A100": cuda_ms}
        del blk, x
        torch.cuda.empty_cache()
    head = rows["d_model1024_N16"]
    return {
        "metric": "MambaBlock forward+backward ms, batch 1, fp32, L=4096 (the regime of the reference's README plots)",
        "value": head["ms"], "unit": "ms", "higher_is_better": False,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": head["ms"],
        "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (random-init weights, N(0,1) input)",
        "config": {"workload": "one MambaBlock fwd+bwd, B=1 fp32: L=4096 with d_model 1024 / 2048 at N=16 and d_model 1024 at N=64 / 128 / 256; L=65536 with d_model 1024, N=16"},
        "rows": rows,
    }


_CACHE = {}


def bench_lm_forward(args, torch, pkg, dev, L):
    """configs[4]: random-init LM forward at the mamba-130m architecture, bf16 weights and
    activations, fp32 scan state, B=8, uniform-random token ids."""
    Bsz, vocab = 8, 50280
    cfg = pkg.MambaConfig(d_model=768, n_layers=24, d_state=16)
    if "lm" not in _CACHE:           # the same random-init model serves L=4096 and L=3000
        torch.manual_seed(1004)
        _CACHE["lm"] = pkg.LM(cfg, vocab, pad_vocab_size_multiple=8).to(dev).to(torch.bfloat16)
    model = _CACHE["lm"]
    ids = torch.randint(0, vocab, (Bsz, L), generator=torch.Generator().manual_seed(1004)).to(dev)

    def fwd():
        with torch.no_grad():
            model(ids)

    steps, warmup = max(2, args.steps // 5), 2
    t = _timed(torch, fwd, steps, warmup)
    ED, N = cfg.d_inner, cfg.d_state
    scan_bytes = cfg.n_layers * (2 * (3 * Bsz * L * ED + 2 * Bsz * L * N) + 4 * (ED * N + ED))
    out = {
        "metric": f"LM forward tokens/s, mamba-130m architecture, B=8 L={L}",
        "value": Bsz * L / t, "unit": "tokens/s", "higher_is_better": True,
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": t * 1e3,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16 weights/activations, f32 scan state",
        "data": "synthetic (random-init weights, uniform-random token ids)",
        "config": {"workload": f"configs[4]: LM forward 24 layers d_model=768 vocab 50280, B=8 L={L}",
                   "scan_algorithmic_bytes_all_layers": scan_bytes},
    }
    return out


def bench_sscan(args, torch, pkg, dev, workload, steps, warmup, prewarm, cpu=True):
    """configs[0..2]: forward + backward of the fused scan through the public selective_scan_fn."""
    import synthetic_inputs
    B, L, ED, N, dtname, seed, desc = WORKLOADS[workload]
    dtype = getattr(torch, dtname)
    inp = synthetic_inputs.make_inputs(B, L, ED, N, seed=seed, dtype=dtype)
    names = ("x", "delta", "A", "B", "C", "D")
    gpu = [inp[k].to(dev).requires_grad_() for k in names]
    dy = inp["dy"].to(dev)
    torch.cuda.synchronize()

    def step(events=None):
        for a in gpu:
            a.grad = None
        if events:
            events[0].record()
        y = pkg.selective_scan_fn(*gpu)
        if events:
            events[1].record()
        y.backward(dy)
        if events:
            events[2].record()

    if args.copy_probe:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).zero_()
        for _ in range(3):
            dst = src.clone()
        torch.cuda.synchronize()
        del src, dst

    # Untimed start-up: the first tens of milliseconds of GPU work after an idle period run at
    # ramping clocks and through a cold allocator (measured: 1.02 ms per step over the first 20
    # steps, 0.96 ms from then on); `prewarm` steps bring the device to its steady state before
    # the W warm-up and K timed steps of the contract.
    for _ in range(prewarm + warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / steps * 1e3

    # per-entry-point GPU time from HIP events recorded on the launch stream
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for e in evs:
        step(e)
    torch.cuda.synchronize()
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / len(evs)
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / len(evs)

    s = 2 if dtype == torch.bfloat16 else 4
    fwd_b, bwd_b = algorithmic_bytes(B, L, ED, N, s)
    gbs = (fwd_b + bwd_b) / (ms_per_step * 1e-3) / 1e9
    bwd_gbs = bwd_b / (bwd_ms * 1e-3) / 1e9
    out = {
        "metric": "selective-scan fwd+bwd GB/s (% HBM peak) + tokens/s, "
                  + ("1.4b layer L=4096" if workload == "c2" else desc),
        "value": gbs, "unit": "GB/s",
        "pct_hbm_peak": 100.0 * gbs / HBM_PEAK_GBS,
        "tokens_per_s": B * L / (ms_per_step * 1e-3),
        "n_gpus": 1, "steps": steps, "warmup": warmup, "prewarm_steps": prewarm, "ms_per_step": ms_per_step,
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 state/accumulation, " + ("bf16" if s == 2 else "f32") + " I/O",
        "data": "synthetic (seeded, S4D-real A, softplus delta; values resident in HBM)",
        "config": {"workload": desc, "B": B, "L": L, "ED": ED, "N": N,
                   "algorithmic_bytes_fwd": fwd_b, "algorithmic_bytes_bwd": bwd_b},
        "roofline": {"bound": "hbm", "kernel": "mpa_sscan_bwd (sscan_bwd_fast_kernel + sscan_bwd_finish_kernel)",
                     "achieved": bwd_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bwd_gbs / HBM_PEAK_GBS,
                     "traffic": measured_traffic_bytes(workload),
                     "traffic_source": profile_state(workload)[1],
                     "valu_issue": valu_issue(workload, "mpa_sscan_bwd", bwd_ms)},
        "forward": {"kernel": "mpa_sscan_fwd (sscan_fwd_kernel)",
                    "achieved": fwd_b / (fwd_ms * 1e-3) / 1e9, "unit": "GB/s",
                    "frac": fwd_b / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                    "valu_issue": valu_issue(workload, "mpa_sscan_fwd", fwd_ms)},
    }
    del gpu, dy, inp
    torch.cuda.empty_cache()
    if cpu:
        out["cpu_baseline"] = cpu_baseline(workload, torch)
    return out


def _brief(rec, extra=()):
    """The figures of a sub-record that belong into the headline line's `other` object."""
    keep = ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype", "tokens_per_s", "pct_hbm_peak",
            "fwd_ms", "bwd_ms", "cpu_baseline", "rows") + tuple(extra)
    out = {k: rec[k] for k in keep if k in rec}
    out["workload"] = rec["config"]["workload"]
    if "roofline" in rec:
        out["roofline"] = {k: rec["roofline"][k] for k in ("kernel", "achieved", "unit", "frac")}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--prewarm", type=int, default=40,
                    help="untimed start-up steps before the W warm-up steps (device clocks, allocator)")
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS) + ["c3", "c4", "c4-3000", "pscan", "layer", "generate", "thin", "block", "gated"],
                    help="c2 (default) is the headline workload; c3 = decode step, c4 = LM forward "
                         "(reported with their own metric, same one-line schema)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other", action="store_true",
                    help="default workload only: leave out the `other` records (c1, c3, c4, pscan, thin)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB device copy (reference point that scales the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (one process, one MI355X); "
                 "--gpus N with N > 1 is not supported.")

    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    global LIBRARY_SHA
    LIBRARY_SHA = pkg._lib.load().mpa_source_hash().decode()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")

    single = {"c3": bench_decode, "pscan": bench_pscan, "layer": bench_layer_kernels,
              "generate": bench_generate, "thin": bench_thin, "block": bench_block, "gated": bench_gated}
    if args.workload in single:
        out = single[args.workload](args, torch, pkg, dev)
    elif args.workload.startswith("c4"):
        out = bench_lm_forward(args, torch, pkg, dev, 3000 if args.workload == "c4-3000" else 4096)
    else:
        out = bench_sscan(args, torch, pkg, dev, args.workload, args.steps, args.warmup, args.prewarm,
                          cpu=not args.no_cpu_baseline)
        if args.workload == "c2" and not args.no_other:
            # one timed record per remaining benchmark configuration, inside the same JSON line
            other = {}
            cpu = not args.no_cpu_baseline
            other["c0"] = _brief(bench_sscan(args, torch, pkg, dev, "c0", max(10, args.steps), 3, 0, cpu=cpu))
            # (the CPU baseline of the headline record has just left the GPU idle for seconds: as many
            # untimed start-up steps as make about 40 ms of GPU work, like the headline's own 40)
            other["c1"] = _brief(bench_sscan(args, torch, pkg, dev, "c1", max(10, args.steps // 2), 3, 100, cpu=cpu))
            other["c3"] = _brief(bench_decode(args, torch, pkg, dev),
                                 ("kernel_step_us_called_from_python", "block_step_us", "graphed_layer_step_us"))
            torch.cuda.empty_cache()
            other["c4"] = _brief(bench_lm_forward(args, torch, pkg, dev, 4096))
            other["c4-3000"] = _brief(bench_lm_forward(args, torch, pkg, dev, 3000))
            torch.cuda.empty_cache()
            other["pscan"] = _brief(bench_pscan(args, torch, pkg, dev))
            torch.cuda.empty_cache()
            other["thin"] = _brief(bench_thin(args, torch, pkg, dev))
            torch.cuda.empty_cache()
            other["block"] = _brief(bench_block(args, torch, pkg, dev))
            torch.cuda.empty_cache()
            other["gated"] = _brief(bench_gated(args, torch, pkg, dev))
            out["other"] = other
    print(json.dumps(out))


if __name__ == "__main__":
    main()
