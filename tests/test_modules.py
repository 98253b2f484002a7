"""Host-side mirror of the reference's callers: names, shapes, state_dict keys, parameter
count (no GPU needed: nothing is launched)."""
import math

import torch


def test_config_derived_values(pkg):
    cfg = pkg.MambaConfig(d_model=768, n_layers=24)       # mamba-130m
    assert cfg.d_inner == 1536 and cfg.dt_rank == 48 and cfg.d_state == 16 and cfg.d_conv == 4
    assert pkg.MambaConfig(d_model=2560, n_layers=1).dt_rank == math.ceil(2560 / 16)


def test_parameter_count_known_answer(pkg):
    # examples/example_e2e_training.ipynb cell 5 of the reference: d_model=16, n_layers=4,
    # vocab 9 with a TIED head has 13 664 parameters; this LM keeps the head untied (lm.py:41)
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.json")) as f:
        g = json.load(f)["param_count"]
    m = pkg.LM(pkg.MambaConfig(d_model=g["d_model"], n_layers=g["n_layers"]), g["vocab_size"])
    n = sum(p.numel() for p in m.parameters())
    assert g["parameters"] == 13664 and n - m.lm_head.weight.numel() == g["parameters"]


def test_state_dict_keys_match_reference_layout(pkg):
    m = pkg.LM(pkg.MambaConfig(d_model=32, n_layers=2), 50)
    keys = set(m.state_dict().keys())
    want = {"embedding.weight", "norm_f.weight", "lm_head.weight"}
    for i in range(2):
        want |= {f"mamba.layers.{i}.norm.weight"} | {
            f"mamba.layers.{i}.mixer.{k}" for k in (
                "in_proj.weight", "conv1d.weight", "conv1d.bias", "x_proj.weight",
                "dt_proj.weight", "dt_proj.bias", "A_log", "D", "out_proj.weight")}
    assert keys == want
    sd = m.state_dict()
    assert sd["mamba.layers.0.mixer.conv1d.weight"].shape == (64, 1, 4)
    assert sd["mamba.layers.0.mixer.A_log"].shape == (64, 16)
    assert sd["mamba.layers.0.mixer.x_proj.weight"].shape == (2 + 32, 64)


def test_block_initial_values(pkg):
    torch.manual_seed(0)
    blk = pkg.MambaBlock(pkg.MambaConfig(d_model=64, n_layers=1))
    A = -torch.exp(blk.A_log)
    assert torch.allclose(A[3], -torch.arange(1, 17, dtype=torch.float32), rtol=1e-6)
    assert torch.equal(blk.D, torch.ones(128))
    dt = torch.nn.functional.softplus(blk.dt_proj.bias)
    assert dt.min() >= 1e-4 - 1e-9 and dt.max() <= 0.1 + 1e-6   # mamba.py:158-163


def test_vocab_padding(pkg):
    m = pkg.LM(pkg.MambaConfig(d_model=16, n_layers=1), 50277, pad_vocab_size_multiple=8)
    assert m.lm_head.weight.shape[0] == 50280


def test_generate_without_new_tokens_returns_the_prompt(pkg):
    # mambapy/lm.py:119-155 with num_tokens = 0: the loop does not run and `generated[:, -0:]` is the
    # whole prompt; a negative count slices the prompt from that position on; the module ends in train mode
    m = pkg.LM(pkg.MambaConfig(d_model=16, n_layers=1), 11)
    prompt = torch.tensor([[1, 2, 3, 4, 5]])
    m.eval()
    out = m.generate(prompt, 0)
    assert torch.equal(out, prompt) and out.data_ptr() != prompt.data_ptr() and m.training
    assert torch.equal(m.generate(prompt, -2), prompt[:, 2:])
