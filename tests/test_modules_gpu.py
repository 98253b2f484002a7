"""GPU tests of the callers around the scan (MambaBlock / Mamba / LM) against a float64
restatement of the same layer built from the oracle's sequential scan."""
import pytest
import torch
import torch.nn.functional as F

from oracle import scan_oracle as so
from util import rel_err

pytestmark = pytest.mark.gpu


def block_forward_ref(blk, x):
    """float64 MambaBlock.forward (mambapy/mamba.py:205-295) on CPU copies of the weights."""
    p = {k: v.detach().double().cpu().requires_grad_() for k, v in blk.named_parameters()}
    cfg = blk.config
    L = x.shape[1]
    xz = F.linear(x, p["in_proj.weight"])
    xin, z = xz.chunk(2, dim=-1)
    xc = F.conv1d(xin.transpose(1, 2), p["conv1d.weight"], p["conv1d.bias"], padding=cfg.d_conv - 1,
                  groups=cfg.d_inner)[:, :, :L].transpose(1, 2)
    xs = F.silu(xc)
    dbc = F.linear(xs, p["x_proj.weight"])
    dlow, Bm, C = torch.split(dbc, [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
    delta = so.softplus_ref(F.linear(dlow, p["dt_proj.weight"], p["dt_proj.bias"]))
    y = so.selective_scan_ref(xs, delta, -torch.exp(p["A_log"]), Bm, C, p["D"])
    return F.linear(y * F.silu(z), p["out_proj.weight"]), p


@pytest.mark.parametrize("fused", [True, False])
def test_block_forward_backward_matches_float64_layer(pkg, dev, fused):
    torch.manual_seed(1)
    cfg = pkg.MambaConfig(d_model=48, n_layers=1, fused_softplus=fused)
    blk = pkg.MambaBlock(cfg).to(dev)
    x = torch.randn(2, 75, 48)                      # L = 75: not a power of two, ragged tile
    g = torch.randn(2, 75, 48)
    xr = x.double().requires_grad_()
    yr, pr = block_forward_ref(blk, xr)
    yr.backward(g.double())
    xg = x.to(dev).requires_grad_()
    y = blk(xg)
    y.backward(g.to(dev))
    assert rel_err(y, yr) <= 1e-4
    assert rel_err(xg.grad, xr.grad) <= 2e-4
    for k, v in blk.named_parameters():
        assert rel_err(v.grad, pr[k].grad) <= 5e-4, k


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_stack_with_folded_residual_adds_equals_layer_by_layer(pkg, dev, dtype, tol):
    # Mamba.forward folds every residual add into the next layer's norm kernel; the reference's
    # order is x = layer(x) for each layer (mambapy/mamba.py:87-95, 106-112)
    torch.manual_seed(5)
    cfg = pkg.MambaConfig(d_model=64, n_layers=4)
    model = pkg.Mamba(cfg).to(dev).to(dtype)
    x = torch.randn(2, 40, 64, device=dev, dtype=dtype)
    g = torch.randn(2, 40, 64, device=dev, dtype=dtype)
    xa = x.clone().requires_grad_()
    ya = model(xa)
    ya.backward(g)
    grads_a = {k: v.grad.clone() for k, v in model.named_parameters()}
    model.zero_grad()
    xb = x.clone().requires_grad_()
    yb = xb
    for layer in model.layers:
        yb = layer(yb)
    yb.backward(g)
    assert rel_err(ya, yb.double()) <= tol
    assert rel_err(xa.grad, xb.grad.double()) <= tol
    for k, v in model.named_parameters():
        assert rel_err(grads_a[k], v.grad.double()) <= 5 * tol, k


def test_steps_equal_forward_and_prefill_handoff(pkg, dev):
    # mambapy/mamba.py:330-349: zero conv window + h=None reproduce the parallel forward
    torch.manual_seed(2)
    cfg = pkg.MambaConfig(d_model=32, n_layers=3)
    model = pkg.Mamba(cfg).to(dev)
    x = torch.randn(2, 21, 32, device=dev)
    with torch.no_grad():
        y_par = model(x)
        caches = model.empty_caches(2)
        ys = []
        for t in range(21):
            y, caches = model.step(x[:, t], caches)
            ys.append(y)
        y_seq = torch.stack(ys, 1)
        assert rel_err(y_seq, y_par) <= 1e-4
        # prefill 13 positions, then continue step by step from the returned caches
        y_pre, caches2 = model(x[:, :13], return_caches=True)
        rest = []
        for t in range(13, 21):
            y, caches2 = model.step(x[:, t], caches2)
            rest.append(y)
        assert rel_err(torch.cat([y_pre, torch.stack(rest, 1)], 1), y_par) <= 1e-4


def test_lm_forward_generate_and_bf16(pkg, dev):
    torch.manual_seed(3)
    cfg = pkg.MambaConfig(d_model=64, n_layers=2)
    lm = pkg.LM(cfg, 101).to(dev)
    tok = torch.randint(0, 101, (2, 37), device=dev)
    with torch.no_grad():
        logits = lm(tok)
        assert logits.shape == (2, 37, 101) and torch.isfinite(logits).all()
        last, caches = lm.prefill(tok)
        assert rel_err(last, logits[:, -1]) <= 1e-4
        # the reference's contract (lm.py:119-155): only the new tokens come back, on the prompt's
        # device, and the module is left in train mode
        new = lm.generate(tok[:, :5], 6, sample=False)
        assert new.shape == (2, 6) and lm.training
        # greedy continuation must agree with re-running the full forward (the reference's
        # O(L^2) generate)
        out = torch.cat([tok[:, :5], new], 1)
        again = lm(out[:, :-1]).argmax(-1)
        assert torch.equal(again[:, 4:], out[:, 5:])
        torch.manual_seed(11)
        sampled = lm.generate(tok[:, :5].cpu(), 4, top_k=3)   # default: sampling; prompt on the CPU
        assert sampled.shape == (2, 4) and sampled.device.type == "cpu"
        top3 = lm(tok[:, :5])[:, -1].topk(3).indices.cpu()
        assert all(sampled[b, 0] in top3[b] for b in range(2))
        lm16 = lm.to(torch.bfloat16)
        l16 = lm16(tok)
        assert l16.dtype == torch.bfloat16 and rel_err(l16, logits) <= 5e-2


def test_lm_full_size_causality_and_prefill_handoff_bf16(pkg, dev):
    # configs[4] at full size (24 layers, d_model 768, vocab 50280, B=8, bf16): properties that
    # do not need an oracle of that size.  (1) Causality: the logits of the first 3000 positions
    # do not depend on what follows, and L=3000 (ragged tiles, no power-of-two padding) must
    # give what the first 3000 positions of L=4096 give.  (2) Prefill of 4095 tokens + one
    # decode step reproduces position 4095 of the parallel forward.
    torch.manual_seed(1004)
    cfg = pkg.MambaConfig(d_model=768, n_layers=24, d_state=16)
    model = pkg.LM(cfg, 50280, pad_vocab_size_multiple=8).to(dev).to(torch.bfloat16).eval()
    ids = torch.randint(0, 50280, (8, 4096), generator=torch.Generator().manual_seed(1004)).to(dev)
    with torch.no_grad():
        full = model(ids)
        part = model(ids[:, :3000])
        assert rel_err(part, full[:, :3000].double()) <= 2e-2
        del part
        last, caches = model.prefill(ids[:, :4095])
        assert rel_err(last, full[:, 4094].double()) <= 2e-2
        nxt, _ = model.step(ids[:, 4095], caches)
        assert rel_err(nxt, full[:, 4095].double()) <= 2e-2


def test_softplus_path_without_gate_full_gradients(pkg, dev):
    # delta = softplus(raw + bias) inside the kernel, no gate: the fast backward path
    Bs, L, ED, N = 2, 150, 128, 16
    inp = so.make_inputs(Bs, L, ED, N, seed=91)
    g = torch.Generator().manual_seed(92)
    raw = torch.randn(Bs, L, ED, generator=g) * 0.5 - 4.0
    bias = torch.randn(ED, generator=g) * 0.3
    f64 = lambda t: t.double().requires_grad_()
    x, r, A, Bm, C, D, bb = map(f64, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], bias))
    yr = so.selective_scan_ref(x, so.softplus_ref(r + bb), A, Bm, C, D)
    yr.backward(inp["dy"].double())
    t = lambda v: v.to(dev).requires_grad_()
    gx, gr, gA, gB, gC, gD, gb = map(t, (inp["x"], raw, inp["A"], inp["B"], inp["C"], inp["D"], bias))
    y = pkg.selective_scan_fn(gx, gr, gA, gB, gC, gD, delta_bias=gb, delta_softplus=True)
    y.backward(inp["dy"].to(dev))
    for got, ref, name in ((y, yr, "y"), (gx.grad, x.grad, "dx"), (gr.grad, r.grad, "ddelta"),
                           (gA.grad, A.grad, "dA"), (gB.grad, Bm.grad, "dB"), (gC.grad, C.grad, "dC"),
                           (gD.grad, D.grad, "dD"), (gb.grad, bb.grad, "dbias")):
        assert rel_err(got, ref) <= 1e-4, name


def test_graphed_decoder_replays_match_eager_steps(pkg, dev):
    # one decode step recorded in a HIP graph: every replay must equal the eager step, with
    # eager work and synchronisations between the replays
    torch.manual_seed(7)
    cfg = pkg.MambaConfig(d_model=64, n_layers=3)
    lm = pkg.LM(cfg, 100).to(dev)
    prompt = torch.randint(0, 100, (4, 9), device=dev)
    with torch.no_grad():
        logits, caches = lm.prefill(prompt)
        decoder = pkg.GraphedDecoder(lm, caches)
        tok = logits.argmax(-1)
        for i in range(6):
            want, caches = lm.step(tok, caches)          # eager
            got = decoder(tok).clone()                   # graph replay
            torch.cuda.synchronize()
            _ = (want.float() @ want.float().T).sum().item()   # unrelated eager work + sync
            assert rel_err(got, want) <= 1e-5, i
            for (h, w), (hg, wg) in zip(caches, decoder.caches):
                assert rel_err(hg, h) <= 1e-5 and torch.equal(wg, w), i
            tok = want.argmax(-1)
    # a bare stack, starting from empty caches (h = None)
    model = pkg.Mamba(cfg).to(dev)
    x = torch.randn(5, 2, 64, device=dev)
    with torch.no_grad():
        caches = model.empty_caches(2)
        decoder = pkg.GraphedDecoder(model, caches)
        for t in range(5):
            want, caches = model.step(x[t], caches)
            assert rel_err(decoder(x[t]), want) <= 1e-5, t


def test_forward_continues_from_a_cache(pkg, dev):
    # a sequence fed in pieces (each piece started from the cache the piece before returned)
    # gives what one pass gives, at block, stack and LM level; a cache must never be ignored
    torch.manual_seed(21)
    cfg = pkg.MambaConfig(d_model=32, n_layers=3)
    model = pkg.Mamba(cfg).to(dev)
    x = torch.randn(2, 50, 32, device=dev)
    with torch.no_grad():
        y_full, c_full = model(x, return_caches=True)
        y1, c1 = model(x[:, :17], return_caches=True)
        y2, c2 = model(x[:, 17:18], caches=c1, return_caches=True)      # a piece shorter than the window
        y3, c3 = model(x[:, 18:], caches=c2, return_caches=True)
        assert rel_err(torch.cat([y1, y2, y3], 1), y_full) <= 1e-5
        for (h, w), (hf, wf) in zip(c3, c_full):
            assert rel_err(h, hf) <= 1e-5 and torch.equal(w, wf)
        # from the caches of step(): empty caches, two steps, then the rest in one call
        caches = model.empty_caches(2)
        ys = []
        for t in range(2):
            y, caches = model.step(x[:, t], caches)
            ys.append(y)
        rest = model(x[:, 2:], caches=caches)
        assert rel_err(torch.cat([torch.stack(ys, 1), rest], 1), y_full) <= 1e-5
        blk = model.layers[0].mixer
        a = blk(x)
        b1, c = blk(x[:, :30], return_cache=True)
        b2 = blk(x[:, 30:], cache=c)
        assert rel_err(torch.cat([b1, b2], 1), a) <= 1e-5
        assert rel_err(blk(x[:, 30:]), a[:, 30:]) > 1e-3     # the cache matters
    lm = pkg.LM(cfg, 77).to(dev)
    tok = torch.randint(0, 77, (2, 40), device=dev)
    l_all, _ = lm.prefill(tok)
    _, c = lm.prefill(tok[:, :25])
    l_cont, _ = lm.prefill(tok[:, 25:], caches=c)
    assert rel_err(l_cont, l_all) <= 1e-5


def test_training_through_a_continued_forward(pkg, dev):
    # truncated backpropagation: the second piece is trained from the detached state of the first
    torch.manual_seed(23)
    cfg = pkg.MambaConfig(d_model=32, n_layers=1)
    blk = pkg.MambaBlock(cfg).to(dev)
    x = torch.randn(2, 40, 32, device=dev)
    with torch.no_grad():
        _, cache = blk(x[:, :20], return_cache=True)
    xr = x[:, 20:].clone().requires_grad_()
    y = blk(xr, cache=cache)
    y.square().mean().backward()
    assert torch.isfinite(xr.grad).all() and xr.grad.abs().max() > 0


def test_block_with_inner_layernorms_matches_float64_layer(pkg, dev):
    # inner_layernorms=True (mambapy/mamba.py:196-203, 246): RMSNorm over the dt_rank, d_state and
    # d_state slices of the x_proj output, i.e. rows that are strided slices of one projection
    torch.manual_seed(31)
    cfg = pkg.MambaConfig(d_model=64, n_layers=1, inner_layernorms=True)
    blk = pkg.MambaBlock(cfg).to(dev)
    with torch.no_grad():
        for n in (blk.dt_layernorm, blk.B_layernorm, blk.C_layernorm):
            n.weight.uniform_(0.5, 1.5)
    x = torch.randn(2, 45, 64)
    g = torch.randn(2, 45, 64)

    p = {k: v.detach().double().cpu().requires_grad_() for k, v in blk.named_parameters()}

    def ref_forward(xx):
        L = xx.shape[1]
        xz = F.linear(xx, p["in_proj.weight"])
        xin, z = xz.chunk(2, dim=-1)
        xc = F.conv1d(xin.transpose(1, 2), p["conv1d.weight"], p["conv1d.bias"], padding=cfg.d_conv - 1,
                      groups=cfg.d_inner)[:, :, :L].transpose(1, 2)
        xs = F.silu(xc)
        dlow, Bm, C = torch.split(F.linear(xs, p["x_proj.weight"]), [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
        dlow = so.rmsnorm_ref(dlow, p["dt_layernorm.weight"], cfg.rms_norm_eps)
        Bm = so.rmsnorm_ref(Bm, p["B_layernorm.weight"], cfg.rms_norm_eps)
        C = so.rmsnorm_ref(C, p["C_layernorm.weight"], cfg.rms_norm_eps)
        delta = so.softplus_ref(F.linear(dlow, p["dt_proj.weight"], p["dt_proj.bias"]))
        y = so.selective_scan_ref(xs, delta, -torch.exp(p["A_log"]), Bm, C, p["D"])
        return F.linear(y * F.silu(z), p["out_proj.weight"])

    xr = x.double().requires_grad_()
    yr = ref_forward(xr)
    yr.backward(g.double())
    xg = x.to(dev).requires_grad_()
    y = blk(xg)
    y.backward(g.to(dev))
    assert rel_err(y, yr) <= 1e-4
    assert rel_err(xg.grad, xr.grad) <= 2e-4
    for k, v in blk.named_parameters():
        assert rel_err(v.grad, p[k].grad) <= 5e-4, k
    # decode: steps from empty caches reproduce the parallel forward with the norms in place
    with torch.no_grad():
        cache = (None, torch.zeros(2, cfg.d_inner, cfg.d_conv - 1, device=dev))
        ys = []
        for t in range(12):
            yt, cache = blk.step(x[:, t].to(dev), cache)
            ys.append(yt)
        assert rel_err(torch.stack(ys, 1), yr[:, :12]) <= 1e-4


def test_lm_training_step_matches_float64_model_and_learns(pkg, dev):
    """The whole training path the reference's examples drive (mambapy/lm.py:97-117 forward,
    cross-entropy on the logits, backward through every layer): loss and the gradient of every
    parameter against a float64 restatement of the model built from the oracle's scan, then a few
    AdamW steps on a repeating sequence, which must bring the loss down."""
    torch.manual_seed(21)
    cfg = pkg.MambaConfig(d_model=32, n_layers=2, d_state=16)
    V, Bs, L = 53, 3, 45
    lm = pkg.LM(cfg, V).to(dev)
    tok = torch.randint(1, V, (Bs, L + 1))
    inp, tgt = tok[:, :-1], tok[:, 1:]

    # float64 restatement on CPU copies of the weights
    p = {k: v.detach().double().cpu().requires_grad_() for k, v in lm.named_parameters()}

    def rms(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps) * w

    x = F.embedding(inp, p["embedding.weight"])
    for i in range(cfg.n_layers):
        pre = "mamba.layers.%d." % i
        h = rms(x, p[pre + "norm.weight"])
        q = {k[len(pre) + 6:]: v for k, v in p.items() if k.startswith(pre + "mixer.")}
        xz = F.linear(h, q["in_proj.weight"])
        xin, z = xz.chunk(2, dim=-1)
        xc = F.conv1d(xin.transpose(1, 2), q["conv1d.weight"], q["conv1d.bias"], padding=cfg.d_conv - 1,
                      groups=cfg.d_inner)[:, :, :L].transpose(1, 2)
        xs = F.silu(xc)
        dlow, Bm, C = torch.split(F.linear(xs, q["x_proj.weight"]), [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
        delta = so.softplus_ref(F.linear(dlow, q["dt_proj.weight"], q["dt_proj.bias"]))
        y = so.selective_scan_ref(xs, delta, -torch.exp(q["A_log"]), Bm, C, q["D"])
        x = x + F.linear(y * F.silu(z), q["out_proj.weight"])
    logits_ref = F.linear(rms(x, p["norm_f.weight"]), p["lm_head.weight"])
    loss_ref = F.cross_entropy(logits_ref.reshape(-1, V), tgt.reshape(-1))
    loss_ref.backward()

    logits = lm(inp.to(dev))
    loss = F.cross_entropy(logits.reshape(-1, V), tgt.to(dev).reshape(-1))
    loss.backward()
    assert rel_err(logits, logits_ref) <= 1e-4
    assert abs(loss.item() - loss_ref.item()) <= 1e-5 * abs(loss_ref.item())
    for k, v in lm.named_parameters():
        assert v.grad is not None, k
        assert rel_err(v.grad, p[k].grad) <= 1e-3, k

    opt = torch.optim.AdamW(lm.parameters(), lr=3e-3)
    first = loss.item()
    for _ in range(30):
        opt.zero_grad()
        out = lm(inp.to(dev))
        cur = F.cross_entropy(out.reshape(-1, V), tgt.to(dev).reshape(-1))
        cur.backward()
        opt.step()
    assert torch.isfinite(cur) and cur.item() < 0.8 * first
