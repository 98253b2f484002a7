"""Pins the CPU oracle (oracle/) against the reference's own known-answer vectors and
against what the mathematics fixes, so that a plausible mistake in the oracle (a dropped
term, a wrong sign or index, a transposed operand) fails here.  Runs without a GPU."""
import json
import math
import os

import pytest
import torch

from oracle import c_oracle, scan_oracle as so

torch.set_default_dtype(torch.float32)


with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.json")) as _f:
    GOLDEN = json.load(_f)


def _as4d(v):
    return torch.tensor(v, dtype=torch.float64).reshape(1, -1, 1, 1)


# ---- golden vectors held by the reference ---------------------------------------------

def test_reference_cumsum_vector_1234():
    # docs/pscan.ipynb cells 5, 8, 11: cumsum([1,2,3,4]) = [1,3,6,10]  (A == 1)
    X = _as4d(GOLDEN["cumsum_1234"]["X"])
    A = torch.ones_like(X)
    want = GOLDEN["cumsum_1234"]["H"]
    assert want == [1, 3, 6, 10]
    assert so.linear_recurrence(A, X).flatten().tolist() == want
    assert so.pscan_blelloch(A, X).flatten().tolist() == want


def test_reference_upsweep_vector():
    # docs/pscan.ipynb cell 43: up-sweep only of [1..8] leaves [1,3,3,10,5,11,7,36]
    X = _as4d(GOLDEN["upsweep_1_to_8"]["X"])
    A = torch.ones_like(X)
    so.blelloch_upsweep_(A, X)
    assert X.flatten().tolist() == GOLDEN["upsweep_1_to_8"]["X_after_upsweep"]


def test_reference_padded_scan_vector():
    # docs/tests.ipynb cell 1: inclusive scan with a zero-padded tail
    X = _as4d(GOLDEN["padded_scan"]["X"])
    A = torch.ones_like(X)
    want = GOLDEN["padded_scan"]["H"]
    H = X.clone()
    so.blelloch_scan_(A.clone(), H)
    assert H.flatten().tolist() == want
    assert so.linear_recurrence(A, X).flatten().tolist() == want


def test_next_pow2_matches_reference_table():
    # mambapy/pscan.py:13-18 : 64->64, 3000->4096, 4097->8192, 1->1
    assert [so.next_pow2(v) for v in GOLDEN["next_pow2"]["in"]] == GOLDEN["next_pow2"]["out"]


# ---- closed forms and brute force -----------------------------------------------------

def test_geometric_closed_form():
    # A == a, X == 1  =>  H[t] = (1 - a^(t+1)) / (1 - a)
    a, L = 0.9, 37
    A = torch.full((1, L, 1, 1), a, dtype=torch.float64)
    X = torch.ones_like(A)
    want = torch.tensor([(1 - a ** (t + 1)) / (1 - a) for t in range(L)], dtype=torch.float64)
    assert torch.allclose(so.linear_recurrence(A, X).flatten(), want, rtol=1e-13)
    assert torch.allclose(so.pscan_blelloch(A, X).flatten(), want, rtol=1e-13)


def test_zero_decay_is_identity():
    X = torch.randn(2, 9, 3, 4, dtype=torch.float64)
    assert torch.equal(so.linear_recurrence(torch.zeros_like(X), X), X)


@pytest.mark.parametrize("L", [1, 2, 3, 5, 8, 13])
def test_recurrence_vs_bruteforce_and_blelloch(L):
    g = torch.Generator().manual_seed(L)
    A = torch.rand(2, L, 3, 2, generator=g, dtype=torch.float64) * 1.5 - 0.5
    X = torch.randn(2, L, 3, 2, generator=g, dtype=torch.float64)
    H = so.linear_recurrence(A, X)
    assert torch.allclose(H, so.linear_recurrence_bruteforce(A, X), rtol=1e-12, atol=1e-12)
    assert torch.allclose(H, so.pscan_blelloch(A, X), rtol=1e-12, atol=1e-12)


def test_reverse_scan_is_flip_scan_flip():
    # mambapy/pscan.py:99-101
    g = torch.Generator().manual_seed(0)
    A = torch.rand(2, 16, 3, 2, generator=g, dtype=torch.float64)
    X = torch.randn(2, 16, 3, 2, generator=g, dtype=torch.float64)
    R = X.clone()
    so.blelloch_scan_(A.clone(), R, reverse=True)
    F = so.linear_recurrence(A.flip(1), X.flip(1)).flip(1)
    assert torch.allclose(R, F, rtol=1e-12, atol=1e-12)


def test_chunk_split_and_linearity():
    g = torch.Generator().manual_seed(1)
    A = torch.rand(1, 20, 2, 3, generator=g, dtype=torch.float64)
    X = torch.randn(1, 20, 2, 3, generator=g, dtype=torch.float64)
    Y = torch.randn(1, 20, 2, 3, generator=g, dtype=torch.float64)
    H = so.linear_recurrence(A, X)
    H1 = so.linear_recurrence(A[:, :7], X[:, :7])
    H2 = so.linear_recurrence(A[:, 7:], X[:, 7:], h0=H1[:, -1])
    assert torch.allclose(torch.cat([H1, H2], 1), H, rtol=1e-13)
    assert torch.allclose(so.linear_recurrence(A, 2 * X + Y), 2 * H + so.linear_recurrence(A, Y), rtol=1e-12)


def test_blelloch_backward_matches_autograd_of_the_definition():
    # pins pscan.py:188-224 as restated: shifted-A reverse scan and gradA[t] = H[t-1] gradX[t]
    for L in (1, 6, 8, 13):
        g = torch.Generator().manual_seed(10 + L)
        A = torch.rand(2, L, 3, 2, generator=g, dtype=torch.float64, requires_grad=True)
        X = torch.randn(2, L, 3, 2, generator=g, dtype=torch.float64, requires_grad=True)
        G = torch.randn(2, L, 3, 2, generator=g, dtype=torch.float64)
        ga1, gx1 = torch.autograd.grad(so.linear_recurrence(A, X), (A, X), G)
        ga2, gx2 = torch.autograd.grad(so.pscan_blelloch(A, X), (A, X), G)
        assert torch.allclose(ga1, ga2, rtol=1e-12, atol=1e-12)
        assert torch.allclose(gx1, gx2, rtol=1e-12, atol=1e-12)
        assert torch.all(ga2[:, 0] == 0)


# ---- selective scan -------------------------------------------------------------------

def _small(seed=0, Bs=2, L=6, ED=3, N=4):
    d = so.make_inputs(Bs, L, ED, N, seed=seed)
    return {k: v.double() for k, v in d.items()}


def test_selective_scan_special_cases():
    d = _small()
    x, dl, A, Bm, C, D = (d[k] for k in ("x", "delta", "A", "B", "C", "D"))
    assert torch.allclose(so.selective_scan_ref(x, torch.zeros_like(dl), A, Bm, C, D), D * x)
    assert torch.allclose(so.selective_scan_ref(x, dl, A, Bm, torch.zeros_like(C), D), D * x)
    # A = 0: y_t = sum_{s<=t} delta_s x_s (B_s . C_t) + D x_t
    G = torch.einsum("btn,bsn->bts", C, Bm).tril()
    want = torch.einsum("bts,bsd->btd", G, dl * x) + D * x
    assert torch.allclose(so.selective_scan_ref(x, dl, torch.zeros_like(A), Bm, C, D), want, rtol=1e-12)


def test_selective_scan_vs_bruteforce_and_blelloch_path():
    d = _small(seed=3)
    args = [d[k] for k in ("x", "delta", "A", "B", "C", "D")]
    y = so.selective_scan_ref(*args)
    assert torch.allclose(y, so.selective_scan_bruteforce(*args), rtol=1e-11, atol=1e-12)
    assert torch.allclose(y, so.selective_scan_blelloch(*args), rtol=1e-11, atol=1e-12)


def test_selective_scan_gradcheck():
    d = _small(seed=4, Bs=1, L=5, ED=2, N=3)
    args = [d[k].clone().requires_grad_() for k in ("x", "delta", "A", "B", "C", "D")]
    assert torch.autograd.gradcheck(so.selective_scan_ref, args, eps=1e-6, atol=1e-7, rtol=1e-5)
    assert torch.autograd.gradcheck(so.selective_scan_blelloch, args, eps=1e-6, atol=1e-7, rtol=1e-5)


def test_c_oracle_matches_autograd_oracle():
    # the C file derives the gradients by hand; autograd through the Python loop is the
    # independent derivation that pins them (configs[0] shape and a ragged one)
    for shape, seed in (((2, 64, 32, 16), 1000), ((3, 37, 5, 7), 5)):
        inp = so.make_inputs(*shape, seed=seed)
        ref = so.selective_scan_grads_autograd(**inp)
        got = c_oracle.sscan_fwd_bwd(**inp)
        for k in ref:
            assert torch.allclose(got[k], ref[k], rtol=1e-10, atol=1e-12), k


def test_c_oracle_initial_and_last_state():
    inp = so.make_inputs(2, 9, 4, 3, seed=9)
    h0 = torch.randn(2, 4, 3, dtype=torch.float64)
    args = [inp[k] for k in ("x", "delta", "A", "B", "C", "D")]
    y, hl = c_oracle.sscan_fwd(*args, h0=h0, return_last_state=True)
    yr, hr = so.selective_scan_ref(*[a.double() for a in args], h0=h0, return_last_state=True)
    assert torch.allclose(y, yr, rtol=1e-12) and torch.allclose(hl, hr, rtol=1e-12)


# ---- decode step ----------------------------------------------------------------------

def test_steps_equal_scan():
    # mambapy/mamba.py:344-346: h = None is h = 0, and L steps reproduce one scan over L
    d = _small(seed=6, L=9)
    x, dl, A, Bm, C, D = (d[k] for k in ("x", "delta", "A", "B", "C", "D"))
    y_scan, h_scan = so.selective_scan_ref(x, dl, A, Bm, C, D, return_last_state=True)
    h, ys = None, []
    for t in range(x.shape[1]):
        y, h = so.ssm_step_ref(x[:, t], dl[:, t], A, Bm[:, t], C[:, t], D, h)
        ys.append(y)
    assert torch.allclose(torch.stack(ys, 1), y_scan, rtol=1e-12)
    assert torch.allclose(h, h_scan, rtol=1e-12)


def test_conv_window_step_matches_padded_conv1d():
    # mambapy/mamba.py:217-219 vs :366-367, 379: zero window == left zero padding
    g = torch.Generator().manual_seed(2)
    Bs, ED, L, K = 2, 5, 7, 4
    x = torch.randn(Bs, L, ED, generator=g, dtype=torch.float64)
    w = torch.randn(ED, 1, K, generator=g, dtype=torch.float64)
    b = torch.randn(ED, generator=g, dtype=torch.float64)
    full = torch.nn.functional.conv1d(x.transpose(1, 2), w, b, padding=K - 1, groups=ED)[:, :, :L]
    win = torch.zeros(Bs, ED, K - 1, dtype=torch.float64)
    for t in range(L):
        out, win = so.conv_window_step_ref(win, x[:, t], w, b)
        assert torch.allclose(out, full[:, :, t], rtol=1e-12, atol=1e-12)


def test_softplus_ref_and_input_recipe():
    v = torch.linspace(-30, 30, 61, dtype=torch.float64)
    assert torch.allclose(so.softplus_ref(v), torch.nn.functional.softplus(v), rtol=1e-12)
    inp = so.make_inputs(2, 50, 64, 16, seed=0)
    # delta = softplus(w + inv_softplus(dt)), dt in [1e-3, 0.1], |w| small
    assert 5e-4 < inp["delta"].min().item() and inp["delta"].max().item() < 0.2
    assert torch.equal(inp["A"][0], -torch.arange(1, 17, dtype=torch.float32))
    assert torch.equal(inp["D"], torch.ones(64))


def test_causal_conv1d_ref_against_explicit_loops_and_nn_conv1d():
    # definition: y[b,t,d] = bias[d] + sum_k w[d,k] * x[b, t-(K-1)+k, d], inputs before step 0
    # taken from `window` (zeros without one)  (mambapy/mamba.py:217-221, 344-346)
    g = torch.Generator().manual_seed(5)
    Bsz, L, ED, K = 2, 7, 3, 4
    x = torch.randn(Bsz, L, ED, generator=g, dtype=torch.float64)
    w = torch.randn(ED, 1, K, generator=g, dtype=torch.float64)
    b = torch.randn(ED, generator=g, dtype=torch.float64)
    win = torch.randn(Bsz, ED, K - 1, generator=g, dtype=torch.float64)
    for window in (None, win):
        want = torch.zeros(Bsz, L, ED, dtype=torch.float64)
        for bb in range(Bsz):
            for t in range(L):
                for d in range(ED):
                    acc = b[d].item()
                    for k in range(K):
                        src = t - (K - 1) + k
                        if src >= 0:
                            acc += w[d, 0, k].item() * x[bb, src, d].item()
                        elif window is not None:
                            acc += w[d, 0, k].item() * window[bb, d, src + K - 1].item()
                    want[bb, t, d] = acc
        got = so.causal_conv1d_ref(x, w, b, window, silu=False)
        assert (got - want).abs().max().item() < 1e-12
    conv = torch.nn.Conv1d(ED, ED, K, groups=ED, padding=K - 1).double()
    ref = torch.nn.functional.silu(conv(x.transpose(1, 2))[:, :, :L].transpose(1, 2))
    assert (so.causal_conv1d_ref(x, conv.weight, conv.bias) - ref).abs().max().item() < 1e-12


def test_rmsnorm_ref_known_answer_loops_and_invariants():
    # mambapy/mamba.py:427-433
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    want = torch.tensor([[3.0, 4.0]], dtype=torch.float64) / math.sqrt(12.5)
    assert (so.rmsnorm_ref(x, None, 0.0) - want).abs().max().item() < 1e-15
    g = torch.Generator().manual_seed(9)
    x = torch.randn(3, 5, 6, generator=g, dtype=torch.float64) * 2 + 0.5
    w = torch.randn(6, generator=g, dtype=torch.float64)
    eps = 1e-3
    got = so.rmsnorm_ref(x, w, eps)
    for i in range(3):
        for j in range(5):
            ms = sum(x[i, j, k].item() ** 2 for k in range(6)) / 6
            for k in range(6):
                assert abs(got[i, j, k].item() - x[i, j, k].item() / math.sqrt(ms + eps) * w[k].item()) < 1e-12
    y0 = so.rmsnorm_ref(x, None, 0.0)
    assert (y0.pow(2).mean(-1) - 1.0).abs().max().item() < 1e-12
    assert (so.rmsnorm_ref(x * 7.5, None, 0.0) - y0).abs().max().item() < 1e-12
