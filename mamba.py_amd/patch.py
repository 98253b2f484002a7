"""Reference-side binding: route an installed `mambapy` through the gfx950 kernels.

The reference binds its scan by name at import time (`from mambapy.pscan import pscan`,
mambapy/mamba.py:9) and picks the scan method in `MambaBlock.ssm` (mamba.py:267-270), so a
drop-in replaces three symbols:
    mambapy.pscan.pscan / mambapy.mamba.pscan        -> mambapy_amd.pscan
    mambapy.mamba.MambaBlock.selective_scan[_seq]    -> fused HIP scan
    mambapy.mamba.MambaBlock.ssm_step                -> fused HIP decode step
`mambapy` itself is not a dependency of this package: patch_mambapy() imports it only when
called.
"""
import torch.nn.functional as F

from .scan import pscan, selective_scan, ssm_step


def patch_mambapy():
    """Monkey-patch an importable `mambapy`; returns the patched mambapy.mamba module."""
    import mambapy.mamba as ref_mamba
    import mambapy.pscan as ref_pscan

    ref_pscan.pscan = pscan
    ref_mamba.pscan = pscan

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

    ref_mamba.MambaBlock.selective_scan = _selective_scan
    ref_mamba.MambaBlock.selective_scan_seq = _selective_scan
    ref_mamba.MambaBlock.ssm_step = _ssm_step
    return ref_mamba
