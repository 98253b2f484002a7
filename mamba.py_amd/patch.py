"""Reference-side binding: route an installed `mambapy` through the gfx950 kernels.

The reference binds its scan by name at import time (`from mambapy.pscan import pscan`,
mambapy/mamba.py:9) and picks the scan method in `MambaBlock.ssm` (mamba.py:267-270), so a
drop-in replaces three symbols:
    mambapy.pscan.pscan / mambapy.mamba.pscan        -> mambapy_amd.pscan
    mambapy.mamba.MambaBlock.selective_scan[_seq]    -> fused HIP scan
    mambapy.mamba.MambaBlock.ssm_step                -> fused HIP decode step
and the same three on the bidirectional copy of the block, `mambapy.vim.VMambaBlock`
(vim.py:9, 301-354, 411-441), when that module is there.  The ONNX copy
(`mambapy/onnx/mamba_onnx.py`) exists to be traced into an exportable graph and is left alone.
`mambapy` itself is not a dependency of this package: patch_mambapy() imports it only when
called.
"""
import importlib
import sys

import torch.nn.functional as F

from .scan import pscan, selective_scan, ssm_step


def patch_mambapy():
    """Monkey-patch an importable `mambapy`; returns the patched mambapy.mamba module."""
    import mambapy.mamba as ref_mamba
    import mambapy.pscan as ref_pscan

    try:
        ref_vim = importlib.import_module("mambapy.vim")
    except ImportError:  # a mambapy without the vision model
        ref_vim = None

    # `from mambapy.pscan import pscan` copies the function into the importing module, so the
    # name is rebound in the defining module and in every loaded module of the package that
    # copied it (mamba.py:9, vim.py:9)
    original = ref_pscan.pscan
    ref_pscan.pscan = pscan
    for name, mod in list(sys.modules.items()):
        if mod is None or not name.startswith("mambapy.") or name.startswith("mambapy.onnx"):
            continue
        if vars(mod).get("pscan") is original:
            mod.pscan = pscan

    def _selective_scan(self, x, delta, A, B, C, D):
        return selective_scan(x, delta, A, B, C, D)

    def _ssm_step(self, x, h):
        cfg = self.config
        A = -self.A_log.float().exp()
        dbc = self.x_proj(x)
        dlow, Bm, C = dbc.split([cfg.dt_rank, cfg.d_state, cfg.d_state], dim=-1)
        dlow, Bm, C = self._apply_layernorms(dlow, Bm, C)
        raw = F.linear(dlow, self.dt_proj.weight)
        return ssm_step(x, raw, A, Bm, C, self.D.float(), h, delta_bias=self.dt_proj.bias,
                        delta_softplus=True)

    blocks = [ref_mamba.MambaBlock]
    if ref_vim is not None and hasattr(ref_vim, "VMambaBlock"):
        # both directions of a bidirectional block go through selective_scan (vim.py:222-241 hands
        # ssm() the flipped sequence and the second set of weights); ssm_step is the forward one
        blocks.append(ref_vim.VMambaBlock)
    for blk in blocks:
        blk.selective_scan = _selective_scan
        blk.selective_scan_seq = _selective_scan
        blk.ssm_step = _ssm_step
    return ref_mamba
