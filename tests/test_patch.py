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


def _make_stub():
    """Modules `mambapy`, `mambapy.pscan`, `mambapy.mamba` with the names the binding touches."""
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
    return {"mambapy": root, "mambapy.pscan": m_pscan, "mambapy.mamba": m_mamba}


@pytest.fixture
def stub(monkeypatch):
    mods = _make_stub()
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
