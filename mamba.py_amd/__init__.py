"""mambapy_amd: MI355X (gfx950) kernels for the selective-scan hot path of alxndrTL/mamba.py.

The directory is named `mamba.py_amd`; import it under the name `mambapy_amd` with
importlib.util.spec_from_file_location("mambapy_amd", ".../mamba.py_amd/__init__.py",
submodule_search_locations=[".../mamba.py_amd"]), as `__graft_entry__.load_package()` does.
"""
from . import _lib
from .scan import (PScan, pscan, pscan_rev, selective_scan, selective_scan_fn, ssm_step, SelectiveScanFn,
                   plan, plan_override)
from .conv import CausalConv1dFn, causal_conv1d_fn, causal_conv1d_update
from .norm import AddRMSNormFn, RMSNormFn, add_rmsnorm_fn, rmsnorm_fn
from .modules import Mamba, MambaBlock, MambaConfig, ResidualBlock, RMSNorm
from .language_model import LM
from .decode import GraphedDecoder
from .patch import patch_mambapy

__all__ = ["PScan", "pscan", "pscan_rev", "plan", "plan_override", "selective_scan", "selective_scan_fn", "ssm_step",
           "SelectiveScanFn", "CausalConv1dFn", "causal_conv1d_fn", "causal_conv1d_update", "RMSNormFn", "rmsnorm_fn",
           "AddRMSNormFn", "add_rmsnorm_fn", "Mamba", "MambaBlock", "MambaConfig", "ResidualBlock", "RMSNorm",
           "LM", "GraphedDecoder", "patch_mambapy", "library_path", "library_version"]


def library_path() -> str:
    return _lib.LIB_PATH


def library_version() -> int:
    return _lib.load().mpa_version()
