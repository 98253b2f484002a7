"""Build recipe and ctypes binding for oracle/sscan_oracle.c (float64 CPU oracle).

TEST INFRASTRUCTURE ONLY.  `build()` compiles the C file with gcc into
oracle/_build/libsscan_oracle.so; `load()` opens what is built (building it if it is
missing and gcc is present).
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "sscan_oracle.c")
_OUT = os.path.join(_HERE, "_build", "libsscan_oracle.so")
_lib = None


def build(force: bool = True) -> str:
    if not force and os.path.exists(_OUT) and os.path.getmtime(_OUT) >= os.path.getmtime(_SRC):
        return _OUT
    os.makedirs(os.path.dirname(_OUT), exist_ok=True)
    cmd = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", _OUT, _SRC, "-lm"]
    subprocess.run(cmd, check=True)
    return _OUT


def load():
    global _lib
    if _lib is None:
        path = build(force=False)
        _lib = ctypes.CDLL(path)
        dp, fp, lg = ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long
        _lib.oracle_sscan_fwd.argtypes = [fp] * 6 + [dp, dp, dp] + [lg] * 4
        _lib.oracle_sscan_bwd.argtypes = [fp] * 7 + [dp] * 6 + [lg] * 4
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return load().oracle_num_threads()


def _f32(t):
    return np.ascontiguousarray(t.detach().to(torch.float32).cpu().numpy())


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def sscan_fwd(x, delta, A, B, C, D, h0=None, return_last_state=False):
    """float64 y (and final state) of the selective scan for float-valued torch inputs."""
    lib = load()
    Bs, L, ED = x.shape
    N = A.shape[1]
    xs, ds, As, Bs_, Cs, Ds = map(_f32, (x, delta, A, B, C, D))
    h0a = None if h0 is None else np.ascontiguousarray(h0.detach().cpu().numpy(), dtype=np.float64)
    y = np.empty((Bs, L, ED), np.float64)
    hl = np.empty((Bs, ED, N), np.float64)
    rc = lib.oracle_sscan_fwd(_ptr(xs), _ptr(ds), _ptr(As), _ptr(Bs_), _ptr(Cs), _ptr(Ds),
                              _ptr(h0a), _ptr(y), _ptr(hl), Bs, L, ED, N)
    if rc != 0:
        raise RuntimeError(f"oracle_sscan_fwd failed: {rc}")
    if return_last_state:
        return torch.from_numpy(y), torch.from_numpy(hl)
    return torch.from_numpy(y)


def sscan_fwd_bwd(x, delta, A, B, C, D, dy):
    """dict(y, dx, ddelta, dA, dB, dC, dD) in float64."""
    lib = load()
    Bs, L, ED = x.shape
    N = A.shape[1]
    xs, ds, As, Bs_, Cs, Ds, dys = map(_f32, (x, delta, A, B, C, D, dy))
    y = np.empty((Bs, L, ED), np.float64)
    rc = lib.oracle_sscan_fwd(_ptr(xs), _ptr(ds), _ptr(As), _ptr(Bs_), _ptr(Cs), _ptr(Ds),
                              None, _ptr(y), None, Bs, L, ED, N)
    if rc != 0:
        raise RuntimeError(f"oracle_sscan_fwd failed: {rc}")
    dx = np.empty((Bs, L, ED), np.float64)
    dd = np.empty((Bs, L, ED), np.float64)
    dA = np.empty((ED, N), np.float64)
    dB = np.empty((Bs, L, N), np.float64)
    dC = np.empty((Bs, L, N), np.float64)
    dD = np.empty((ED,), np.float64)
    rc = lib.oracle_sscan_bwd(_ptr(xs), _ptr(ds), _ptr(As), _ptr(Bs_), _ptr(Cs), _ptr(Ds),
                              _ptr(dys), _ptr(dx), _ptr(dd), _ptr(dA), _ptr(dB), _ptr(dC),
                              _ptr(dD), Bs, L, ED, N)
    if rc != 0:
        raise RuntimeError(f"oracle_sscan_bwd failed: {rc}")
    t = torch.from_numpy
    return dict(y=t(y), dx=t(dx), ddelta=t(dd), dA=t(dA), dB=t(dB), dC=t(dC), dD=t(dD))


if __name__ == "__main__":
    print(build())
