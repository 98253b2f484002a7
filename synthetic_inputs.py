"""Seeded synthetic inputs of the selective scan, shared by bench.py, __graft_entry__.smoke()
and the parity tests.  This is the workload recipe, not checker code: it imports nothing from
oracle/ and nothing from the package."""
import math

import torch
import torch.nn.functional as F


def make_inputs(Bs, L, ED, N, seed, dtype=torch.float32, dt_min=1e-3, dt_max=0.1,
                dt_floor=1e-4):
    """Seeded inputs with the value distributions of the reference's layer initialisation
    (mambapy/mamba.py:158-172): A = -(1..N) per channel (S4D-real), delta =
    softplus(w + inv_softplus(dt)), dt log-uniform in [dt_min, dt_max], w ~ N(0, 0.02),
    D = 1; x, B, C, dy ~ N(0, 1).  Generated in float32 on the CPU, then rounded to
    `dtype` (A and D stay float32)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(Bs, L, ED, generator=g)
    Bm = torch.randn(Bs, L, N, generator=g)
    C = torch.randn(Bs, L, N, generator=g)
    dt = torch.exp(torch.rand(ED, generator=g) * (math.log(dt_max) - math.log(dt_min))
                   + math.log(dt_min)).clamp(min=dt_floor)
    bias = dt + torch.log(-torch.expm1(-dt))
    w = 0.02 * torch.randn(Bs, L, ED, generator=g)
    delta = F.softplus(w + bias)
    A = -torch.arange(1, N + 1, dtype=torch.float32).repeat(ED, 1)
    D = torch.ones(ED)
    dy = torch.randn(Bs, L, ED, generator=g)
    cast = lambda t: t.to(dtype)
    return dict(x=cast(x), delta=cast(delta), A=A, B=cast(Bm), C=cast(C), D=D, dy=cast(dy))
