"""The C-ABI library loads and exports every symbol include/mambapy_amd.h declares, and
rejects malformed calls with status codes (no GPU needed: nothing is launched)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mambapy_amd.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mpa_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for n in ("mpa_sscan_fwd", "mpa_sscan_bwd", "mpa_pscan_fwd", "mpa_pscan_bwd", "mpa_ssm_step",
              "mpa_sscan_ckpt_elems", "mpa_sscan_bwd_workspace_bytes", "mpa_version", "mpa_arch"):
        assert n in names


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg._lib.load()
    for n in _declared_functions():
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert set(pkg._lib.EXPORTS) == set(_declared_functions())
    assert lib.mpa_arch() == b"gfx950"
    assert lib.mpa_version() == 20100   # major*10000 + minor*100 + patch
    # the library names the sources it was built from; after a build in this tree that is the tree's hash
    import importlib.util
    spec = importlib.util.spec_from_file_location("_mpa_build", os.path.join(ROOT, "mamba.py_amd", "build.py"))
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    assert re.fullmatch(r"[0-9a-f]{16}", lib.mpa_source_hash().decode())
    assert lib.mpa_source_hash().decode() == b.source_hash(), "csrc/ changed since the library was built"


def test_status_codes_without_launch(pkg):
    L = pkg._lib
    lib = L.load()
    s = L.SscanShape()
    assert lib.mpa_sscan_fwd(None, *([None] * 14), 0, None) == 1          # MPA_ERR_NULL_POINTER
    s.batch, s.seqlen, s.dim, s.dstate = 1, 0, 8, 16
    assert lib.mpa_sscan_fwd(ctypes.byref(s), *([None] * 14), 0, None) == 2  # bad shape
    s.seqlen, s.dstate = 8, 1000
    assert lib.mpa_sscan_fwd(ctypes.byref(s), *([None] * 14), 0, None) == 2  # d_state too large
    s.dstate, s.io_dtype = 16, 7
    assert lib.mpa_sscan_fwd(ctypes.byref(s), *([None] * 14), 0, None) == 3  # bad dtype
    s.io_dtype = 0
    assert lib.mpa_sscan_fwd(ctypes.byref(s), *([None] * 14), 0, None) == 1  # null data pointers
    assert lib.mpa_sscan_ckpt_elems(ctypes.byref(s)) == 1 * 1 * 16 * 8
    assert lib.mpa_sscan_bwd_workspace_bytes(ctypes.byref(s)) > 0
    assert lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(s), 0) > 0
    s.delta_dtype = 7
    assert lib.mpa_sscan_fwd(ctypes.byref(s), *([None] * 14), 0, None) == 3  # delta_dtype: 0 or MPA_DELTA_F32
    s.delta_dtype = L.MPA_DELTA_F32
    assert lib.mpa_sscan_fwd(ctypes.byref(s), *([None] * 14), 0, None) == 1  # accepted: next complaint is the pointers
    s.delta_dtype = 0
    assert lib.mpa_status_string(6) == b"workspace too small"
    p = L.PscanShape()
    assert lib.mpa_pscan_fwd(ctypes.byref(p), None, None, None, None, 0, None) == 2
    p.batch, p.seqlen, p.dim, p.dstate = 1, 65536, 32, 16
    cut = lib.mpa_pscan_workspace_bytes(ctypes.byref(p))
    p.plan_chunks = 1
    assert 0 < lib.mpa_pscan_workspace_bytes(ctypes.byref(p)) < cut   # a thin, long scan is cut by default


def test_missing_library_is_a_loud_import_error(pkg, monkeypatch):
    L = pkg._lib
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", os.path.join(ROOT, "does", "not", "exist.so"))
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        L.load()


def test_cpu_tensors_are_rejected(pkg):
    import torch
    x = torch.zeros(1, 4, 8)
    with pytest.raises(RuntimeError, match="ROCm device"):
        pkg.selective_scan(x, x, torch.zeros(8, 16), torch.zeros(1, 4, 16), torch.zeros(1, 4, 16),
                           torch.zeros(8))
    with pytest.raises(RuntimeError, match="ROCm device"):
        pkg.pscan(torch.zeros(1, 4, 8, 16), torch.zeros(1, 4, 8, 16))


def test_workspace_queries_follow_the_plan_fields_not_the_environment(pkg, monkeypatch):
    # the library keeps no global state and reads no environment: the segment count a caller
    # pins in the shape struct decides the workspace, a variable of the same name does not
    L = pkg._lib
    lib = L.load()
    s = L.SscanShape()
    s.batch, s.seqlen, s.dim, s.dstate = 1, 4096, 64, 16
    base = lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(s), 1)
    monkeypatch.setenv("MPA_FWD_NSEG", "1")
    monkeypatch.setenv("MPA_FWD_NS", "16")
    assert lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(s), 1) == base
    s.plan_segments = 1
    never_cut = lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(s), 1)
    s.plan_segments = 8
    cut8 = lib.mpa_sscan_fwd_workspace_bytes(ctypes.byref(s), 1)
    assert never_cut < cut8
    assert cut8 >= 2 * 8 * 64 * 16 * 4          # start and end states of 8 segments
    b0 = lib.mpa_sscan_bwd_workspace_bytes(ctypes.byref(s))
    s.plan_segments = 1
    assert lib.mpa_sscan_bwd_workspace_bytes(ctypes.byref(s)) < b0


def test_launch_plan_reads_the_environment_once_in_python(pkg, monkeypatch):
    scan = pkg.scan
    monkeypatch.setenv("MPA_BWD_NSEG", "5")
    monkeypatch.setenv("MPA_BWD_GENERAL", "1")
    p = scan.LaunchPlan()
    s = pkg._lib.SscanShape()
    p.fill(s, backward=True)
    assert s.plan_segments == 5 and s.plan_flags == pkg._lib.MPA_PLAN_BWD_GENERAL
    p.fill(s, backward=False)
    assert s.plan_segments == 0
    with pkg.plan_override(fwd_segments=3):
        assert pkg.plan.fwd_segments == 3
    assert pkg.plan.fwd_segments is None
    with pytest.raises(TypeError):
        with pkg.plan_override(nonsense=1):
            pass
