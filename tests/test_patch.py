"""patch_mambapy(): the drop-in binding a maintainer of the reference calls.

The reference binds its scan by name (`from mambapy.pscan import pscan`, mambapy/mamba.py:9) and
picks the scan as a bound method (`self.selective_scan(x, delta, A, B, C, D)` /
`self.selective_scan_seq(...)`, mamba.py:267-270; `self.ssm_step(x, h)`, mamba.py:371).  The tests
run against a stand-in package named `mambapy` that this file writes itself, with the reference's
module layout, attribute names and call signatures (the reference's own code is neither imported
nor present on the GPU box): a CPU test of what gets rebound, and GPU tests that drive the
patched methods the way the reference's `ssm()` and `step()` drive them."""
import inspect
import sys
import types

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import scan_oracle as so
from util import rel_err


class _Cfg:
    def __init__(self, d_model=32, d_state=16, expand=2, inner_layernorms=False):
        self.d_model, self.d_state, self.d_inner = d_model, d_state, expand * d_model
        self.dt_rank = -(-d_model // 16)
        self.pscan = True
        self.inner_layernorms = inner_layernorms


def _make_stub(with_vim=False):
    """Modules `mambapy`, `mambapy.pscan`, `mambapy.mamba` (and `mambapy.vim`) with the names the
    binding touches."""
    root = types.ModuleType("mambapy")
    root.__path__ = []
    m_pscan = types.ModuleType("mambapy.pscan")
    m_mamba = types.ModuleType("mambapy.mamba")

    def pscan(A, X):  # stand-in for PScan.apply
        return so.linear_recurrence(A, X)

    m_pscan.pscan = pscan
    m_mamba.pscan = pscan          # `from mambapy.pscan import pscan` binds the name here too

    class MambaBlock(nn.Module):
        """Carries the attributes the patched methods read: config, x_proj, dt_proj, A_log, D,
        _apply_layernorms; ssm() and step-level calls go through the three patched methods."""

        def __init__(self, config):
            super().__init__()
            self.config = config
            ED, N, R = config.d_inner, config.d_state, config.dt_rank
            self.x_proj = nn.Linear(ED, R + 2 * N, bias=False)
            self.dt_proj = nn.Linear(R, ED, bias=True)
            self.A_log = nn.Parameter(torch.log(torch.arange(1, N + 1, dtype=torch.float32)).repeat(ED, 1))
            self.D = nn.Parameter(torch.ones(ED))
            with torch.no_grad():
                self.dt_proj.bias.uniform_(-5.0, -2.0)

        def _apply_layernorms(self, dt, B, C):
            return dt, B, C

        def ssm(self, x, z=None):
            cfg = self.config
            A, D = -torch.exp(self.A_log.float()), self.D.float()
            dlow, B, C = torch.split(self.x_proj(x), [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
            dlow, B, C = self._apply_layernorms(dlow, B, C)
            # the reference forms the transposed product: delta is a (B, ED, L)-memory view
            delta = (self.dt_proj.weight @ dlow.transpose(1, 2)).transpose(1, 2)
            delta = F.softplus(delta + self.dt_proj.bias)
            if cfg.pscan:
                return self.selective_scan(x, delta, A, B, C, D)
            return self.selective_scan_seq(x, delta, A, B, C, D)

        def selective_scan(self, x, delta, A, B, C, D):
            raise AssertionError("unpatched selective_scan was called")

        def selective_scan_seq(self, x, delta, A, B, C, D):
            raise AssertionError("unpatched selective_scan_seq was called")

        def ssm_step(self, x, h):
            raise AssertionError("unpatched ssm_step was called")

    m_mamba.MambaBlock = MambaBlock
    root.pscan, root.mamba = m_pscan, m_mamba
    mods = {"mambapy": root, "mambapy.pscan": m_pscan, "mambapy.mamba": m_mamba}
    if not with_vim:
        return mods

    m_vim = types.ModuleType("mambapy.vim")
    m_vim.pscan = pscan            # mambapy/vim.py:9 binds the name as mamba.py does

    class VMambaBlock(nn.Module):
        """The scan side of the bidirectional block (mambapy/vim.py:113-441): two sets of scan
        weights, ssm() takes the set to use, and the second direction is the same call on the
        flipped sequence whose output is flipped back (vim.py:222-261)."""

        def __init__(self, config):
            super().__init__()
            self.config = config
            ED, N, R = config.d_inner, config.d_state, config.dt_rank
            for sfx in ("", "_b"):
                setattr(self, "x_proj" + sfx, nn.Linear(ED, R + 2 * N, bias=False))
                dt = nn.Linear(R, ED, bias=True)
                with torch.no_grad():
                    dt.bias.uniform_(-5.0, -2.0)
                setattr(self, "dt_proj" + sfx, dt)
                setattr(self, "A_log" + sfx, nn.Parameter(
                    torch.log(torch.arange(1, N + 1, dtype=torch.float32)).repeat(ED, 1)))
                setattr(self, "D" + sfx, nn.Parameter(torch.ones(ED)))

        def _apply_layernorms(self, dt, B, C):
            return dt, B, C

        def ssm(self, x, z, A_log, D, x_proj, dt_proj):
            cfg = self.config
            A, D = -torch.exp(A_log.float()), D.float()
            dlow, B, C = torch.split(x_proj(x), [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
            dlow, B, C = self._apply_layernorms(dlow, B, C)
            delta = (dt_proj.weight @ dlow.transpose(1, 2)).transpose(1, 2)
            delta = F.softplus(delta + dt_proj.bias)
            if cfg.pscan:
                return self.selective_scan(x, delta, A, B, C, D)
            return self.selective_scan_seq(x, delta, A, B, C, D)

        def both_directions(self, x):
            """y + flip(y_b) of vim.py:222-261 without the convolutions and the gate."""
            y = self.ssm(x, None, self.A_log, self.D, self.x_proj, self.dt_proj)
            y_b = self.ssm(x.flip([1]), None, self.A_log_b, self.D_b, self.x_proj_b, self.dt_proj_b)
            return y + y_b.flip([1])

        def selective_scan(self, x, delta, A, B, C, D):
            raise AssertionError("unpatched selective_scan was called")

        def selective_scan_seq(self, x, delta, A, B, C, D):
            raise AssertionError("unpatched selective_scan_seq was called")

        def ssm_step(self, x, h):
            raise AssertionError("unpatched ssm_step was called")

    m_vim.VMambaBlock = VMambaBlock
    root.vim = m_vim
    mods["mambapy.vim"] = m_vim
    return mods


@pytest.fixture
def stub(monkeypatch):
    mods = _make_stub()
    for k, v in mods.items():
        monkeypatch.setitem(sys.modules, k, v)
    return mods


@pytest.fixture
def stub_vim(monkeypatch):
    mods = _make_stub(with_vim=True)
    for k, v in mods.items():
        monkeypatch.setitem(sys.modules, k, v)
    return mods


def test_patch_rebinds_the_three_symbols_and_keeps_their_signatures(pkg, stub):
    ref_mamba = pkg.patch_mambapy()
    assert ref_mamba is stub["mambapy.mamba"]
    assert stub["mambapy.pscan"].pscan is pkg.pscan and ref_mamba.pscan is pkg.pscan
    Blk = ref_mamba.MambaBlock
    sig = lambda f: list(inspect.signature(f).parameters)
    assert sig(Blk.selective_scan) == ["self", "x", "delta", "A", "B", "C", "D"]
    assert sig(Blk.selective_scan_seq) == ["self", "x", "delta", "A", "B", "C", "D"]
    assert sig(Blk.ssm_step) == ["self", "x", "h"]
    # the replacements have no CPU path: they refuse CPU tensors instead of computing on the host
    blk = Blk(_Cfg())
    with pytest.raises(RuntimeError, match="ROCm device"):
        blk.ssm(torch.zeros(1, 4, blk.config.d_inner))


def test_patch_covers_the_bidirectional_copy_of_the_block(pkg, stub_vim):
    """mambapy/vim.py binds `pscan` by name and carries its own copy of the three methods."""
    pkg.patch_mambapy()
    vim = stub_vim["mambapy.vim"]
    assert vim.pscan is pkg.pscan
    assert stub_vim["mambapy"].pscan is stub_vim["mambapy.pscan"]   # the submodule, left alone
    sig = lambda f: list(inspect.signature(f).parameters)
    assert sig(vim.VMambaBlock.selective_scan) == ["self", "x", "delta", "A", "B", "C", "D"]
    assert sig(vim.VMambaBlock.selective_scan_seq) == ["self", "x", "delta", "A", "B", "C", "D"]
    assert sig(vim.VMambaBlock.ssm_step) == ["self", "x", "h"]
    blk = vim.VMambaBlock(_Cfg())
    with pytest.raises(RuntimeError, match="ROCm device"):
        blk.both_directions(torch.zeros(1, 4, blk.config.d_inner))


def test_patch_needs_an_importable_mambapy(pkg, monkeypatch):
    for k in [k for k in sys.modules if k == "mambapy" or k.startswith("mambapy.")]:
        monkeypatch.delitem(sys.modules, k)
    monkeypatch.setattr(sys, "path", [p for p in sys.path if "reference" not in p])
    monkeypatch.setattr(sys, "meta_path", [_Blocker()] + list(sys.meta_path))
    with pytest.raises(ImportError):
        pkg.patch_mambapy()


class _Blocker:
    @staticmethod
    def find_spec(name, path=None, target=None):
        if name == "mambapy" or name.startswith("mambapy."):
            raise ImportError("mambapy is not installed (test)")
        return None


@pytest.mark.gpu
@pytest.mark.parametrize("use_pscan", [True, False])
def test_patched_block_ssm_matches_float64_oracle(pkg, dev, stub, use_pscan):
    ref_mamba = pkg.patch_mambapy()
    torch.manual_seed(41)
    cfg = _Cfg()
    cfg.pscan = use_pscan
    blk = ref_mamba.MambaBlock(cfg).to(dev)
    x = torch.randn(2, 53, cfg.d_inner)
    g = torch.randn(2, 53, cfg.d_inner)
    # float64 restatement of ssm() (mambapy/mamba.py:236-272) on copies of the weights
    p = {k: v.detach().double().cpu().requires_grad_() for k, v in blk.named_parameters()}
    xr = x.double().requires_grad_()
    dlow, B, C = torch.split(F.linear(xr, p["x_proj.weight"]), [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
    delta = so.softplus_ref(F.linear(dlow, p["dt_proj.weight"], p["dt_proj.bias"]))
    yr = so.selective_scan_ref(xr, delta, -torch.exp(p["A_log"]), B, C, p["D"])
    yr.backward(g.double())
    xg = x.to(dev).requires_grad_()
    y = blk.ssm(xg)
    y.backward(g.to(dev))
    assert rel_err(y, yr) <= 1e-4
    assert rel_err(xg.grad, xr.grad) <= 2e-4
    for k, v in blk.named_parameters():
        assert rel_err(v.grad, p[k].grad) <= 5e-4, k


@pytest.mark.gpu
def test_patched_pscan_and_ssm_step(pkg, dev, stub):
    ref_mamba = pkg.patch_mambapy()
    # pscan(A, X) as mambapy/mamba.py:289 calls it, on materialised (B, L, ED, N) tensors
    g = torch.Generator().manual_seed(43)
    A = torch.rand(2, 19, 8, 16, generator=g) * 0.9 + 0.05
    X = torch.randn(2, 19, 8, 16, generator=g)
    H = ref_mamba.pscan(A.to(dev), X.to(dev))
    assert rel_err(H, so.linear_recurrence(A.double(), X.double())) <= 1e-5
    # ssm_step(x, h) (mambapy/mamba.py:384-414): L steps from h = None equal one scan
    torch.manual_seed(44)
    cfg = _Cfg()
    blk = ref_mamba.MambaBlock(cfg).to(dev)
    x = torch.randn(2, 11, cfg.d_inner, device=dev)
    with torch.no_grad():
        y_par = blk.ssm(x)
        h, ys = None, []
        for t in range(11):
            y, h_new = blk.ssm_step(x[:, t], h)
            assert h is None or h_new.data_ptr() != h.data_ptr()   # a new tensor, as in the reference
            h = h_new
            ys.append(y)
    assert rel_err(torch.stack(ys, 1), y_par) <= 1e-5


@pytest.mark.gpu
def test_patched_bidirectional_block_matches_oracle_and_the_reverse_entry(pkg, dev, stub_vim):
    """The second direction as the reference runs it (flip, scan, flip back; mambapy/vim.py:222-261)
    through the patched methods, against the float64 oracle and against this library's
    reverse-direction entry on the sequence as it lies in memory."""
    pkg.patch_mambapy()
    torch.manual_seed(47)
    cfg = _Cfg()
    blk = stub_vim["mambapy.vim"].VMambaBlock(cfg).to(dev)
    x = torch.randn(2, 37, cfg.d_inner)
    g = torch.randn(2, 37, cfg.d_inner)
    p = {k: v.detach().double().cpu().requires_grad_() for k, v in blk.named_parameters()}
    xr = x.double().requires_grad_()

    def direction(xin, sfx):
        dlow, B, C = torch.split(F.linear(xin, p["x_proj%s.weight" % sfx]),
                                 [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
        delta = so.softplus_ref(F.linear(dlow, p["dt_proj%s.weight" % sfx], p["dt_proj%s.bias" % sfx]))
        return so.selective_scan_ref(xin, delta, -torch.exp(p["A_log" + sfx]), B, C, p["D" + sfx])

    yr = direction(xr, "") + direction(xr.flip([1]), "_b").flip([1])
    yr.backward(g.double())
    xg = x.to(dev).requires_grad_()
    y = blk.both_directions(xg)
    y.backward(g.to(dev))
    assert rel_err(y, yr) <= 1e-4
    assert rel_err(xg.grad, xr.grad) <= 2e-4
    for k, v in blk.named_parameters():
        assert rel_err(v.grad, p[k].grad) <= 5e-4, k
    # the same second direction without the two flipped copies
    with torch.no_grad():
        xd = x.to(dev)
        dlow, B, C = torch.split(blk.x_proj_b(xd), [cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
        raw = F.linear(dlow, blk.dt_proj_b.weight)
        y_rev = pkg.selective_scan_fn(xd, raw, -torch.exp(blk.A_log_b), B, C, blk.D_b,
                                      delta_bias=blk.dt_proj_b.bias, delta_softplus=True, reverse=True)
        y_flip = blk.ssm(xd.flip([1]), None, blk.A_log_b, blk.D_b, blk.x_proj_b, blk.dt_proj_b).flip([1])
    assert rel_err(y_rev, y_flip) <= 1e-5
