"""mpa_sscan_fwd_noalloc: the forward entry point that allocates nothing (its scratch is a static
device array of the library).  Called through the C ABI and compared, bit for bit, with
mpa_sscan_fwd on the same inputs, on two calls in a row, the second with a smaller input; both
shapes are ones the library cuts into segments, so the scratch is really used."""
import ctypes

import pytest
import torch

from oracle import c_oracle, scan_oracle as so
from util import TOL, rel_err

pytestmark = pytest.mark.gpu

NAMES = ("x", "delta", "A", "B", "C", "D")


def _call_both(pkg, dev, Bs, L, ED, N, seed, with_ckpt, dtype=torch.float32):
    L_ = pkg._lib
    lib = L_.load()
    scan = pkg.scan
    inp = so.make_inputs(Bs, L, ED, N, seed=seed, dtype=dtype)
    t = {k: inp[k].to(dev) for k in NAMES}
    outs = []
    for noalloc in (False, True):
        y = torch.full((Bs, L, ED), float("nan"), dtype=dtype, device=dev)
        hl = torch.full((Bs, ED, N), float("nan"), device=dev)
        shape = scan._sscan_shape(t["x"], t["delta"], t["B"], y, y, t["B"], N, 0)
        ck = None
        if with_ckpt:
            ck = torch.full((lib.mpa_sscan_ckpt_elems(ctypes.byref(shape)),), float("nan"), device=dev)
        need = lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(shape), 1 if with_ckpt else 0)
        assert 256 < need <= L_.MPA_NOALLOC_SCRATCH_BYTES, "the case must use the scratch and fit in it"
        p = scan._ptr
        args = [ctypes.byref(shape)] + [p(t[k]) for k in NAMES] + [None, None, None, p(y), None, p(ck), p(hl)]
        stream = scan._stream(dev)
        if noalloc:
            # one call first (the very first one on a device resolves the array's address and may make
            # the runtime materialise the array); after that a call must leave the DRIVER's count of
            # free device memory alone: torch's own counters would not see a hipMalloc inside the library
            assert lib.mpa_sscan_fwd_noalloc(*args, stream) == 0
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info(dev)[0]
            rc = lib.mpa_sscan_fwd_noalloc(*args, stream)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info(dev)[0] == free_before
        else:
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
            rc = lib.mpa_sscan_fwd(*args, p(ws), need, stream)
        assert rc == 0, lib.mpa_status_string(rc)
        torch.cuda.synchronize()
        outs.append((y, hl, ck))
    (y0, h0, c0), (y1, h1, c1) = outs
    assert torch.isfinite(y1.float()).all() and torch.isfinite(h1).all()
    assert torch.equal(y0, y1) and torch.equal(h0, h1)
    if with_ckpt:
        # the slot after the last tile of every batch row is never written by either call
        nch = (L + 15) // 16
        v0, v1 = c0.view(Bs, nch, N, ED)[:, :-1], c1.view(Bs, nch, N, ED)[:, :-1]
        assert torch.isfinite(v1).all() and torch.equal(v0, v1)
    ref = c_oracle.sscan_fwd(*[inp[k] for k in NAMES])
    assert rel_err(y1, ref) <= TOL[dtype]


def test_noalloc_forward_twice_second_call_smaller(pkg, dev):
    # first call: 1 x 4096 x 256, cut into 32 segments; second: a smaller, ragged one (the scratch
    # still holds the first call's states)
    _call_both(pkg, dev, 1, 4096, 256, 16, seed=8101, with_ckpt=False)
    _call_both(pkg, dev, 1, 1000, 100, 16, seed=8102, with_ckpt=False)
    # the training form (checkpoints) and bf16, again larger then smaller
    _call_both(pkg, dev, 2, 2048, 128, 16, seed=8103, with_ckpt=True, dtype=torch.bfloat16)
    _call_both(pkg, dev, 1, 600, 64, 8, seed=8104, with_ckpt=True)


def test_noalloc_inside_a_hip_graph(pkg, dev):
    # The callers the entry point is for include code under HIP graph capture.  Its first call on a
    # device (address look-up, LDS limit of the kernels) happens outside the capture; the capture then
    # records kernels only, and every replay, on new input values and with eager work in between, equals
    # the eager mpa_sscan_fwd bit for bit.
    L_ = pkg._lib
    lib = L_.load()
    scan = pkg.scan
    Bs, L, ED, N = 1, 2048, 256, 16
    inp = so.make_inputs(Bs, L, ED, N, seed=8110)
    t = {k: inp[k].to(dev) for k in NAMES}
    y = torch.zeros(Bs, L, ED, device=dev)
    hl = torch.zeros(Bs, ED, N, device=dev)
    shape = scan._sscan_shape(t["x"], t["delta"], t["B"], y, y, t["B"], N, 0)
    need = lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(shape), 0)
    assert 256 < need <= L_.MPA_NOALLOC_SCRATCH_BYTES
    p = scan._ptr
    args = [ctypes.byref(shape)] + [p(t[k]) for k in NAMES] + [None, None, None, p(y), None, None, p(hl)]
    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        assert lib.mpa_sscan_fwd_noalloc(*args, scan._stream(dev)) == 0   # outside the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert lib.mpa_sscan_fwd_noalloc(*args, scan._stream(dev)) == 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    for rep in range(3):
        new = so.make_inputs(Bs, L, ED, N, seed=8111 + rep)
        for k in ("x", "delta", "B", "C"):
            t[k].copy_(new[k].to(dev))
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        y_graph, h_graph = y.clone(), hl.clone()
        y.fill_(float("nan"))
        assert lib.mpa_sscan_fwd(*args, p(ws), need, scan._stream(dev)) == 0   # eager, between the replays
        torch.cuda.synchronize()
        assert torch.isfinite(y_graph).all()
        assert torch.equal(y_graph, y) and torch.equal(h_graph, hl)
        ref = c_oracle.sscan_fwd(*[new[k] if k in ("x", "delta", "B", "C") else inp[k] for k in NAMES])
        assert rel_err(y_graph, ref) <= TOL[torch.float32]


def test_noalloc_refuses_what_does_not_fit(pkg, dev):
    L_ = pkg._lib
    lib = L_.load()
    # d_state 256 over a long sequence as one launch (32 states per lane pinned): the packed B/C
    # alone are 8 * 512 * 2 * 16 * 256 floats
    s = L_.SscanShape()
    s.batch, s.seqlen, s.dim, s.dstate = 8, 8192, 64, 256
    s.plan_states_per_lane = 32
    assert lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(s), 0) > L_.MPA_NOALLOC_SCRATCH_BYTES
    assert lib.mpa_sscan_fwd_noalloc(ctypes.byref(s), *([None] * 13), None) == 6   # MPA_ERR_WORKSPACE
    assert lib.mpa_status_string(6) == b"workspace too small"
