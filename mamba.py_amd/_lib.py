"""ctypes binding of libmambapy_amd.so (declarations: include/mambapy_amd.h).

There is no fallback: if the library is missing or cannot be loaded, importing the ops
raises ImportError with the build command; nothing here computes on the CPU.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmambapy_amd.so")

MPA_F32, MPA_BF16 = 0, 1
MPA_SSCAN_DELTA_SOFTPLUS = 1
MPA_SSCAN_REVERSE = 2
MPA_PLAN_BWD_GENERAL = 1
MPA_PLAN_EXPIRE_WAITS = 2
MPA_PLAN_GROUP_64 = 4
MPA_PLAN_GROUP_48 = 8
MPA_DELTA_F32 = 1
MPA_CONV_SILU = 1
MPA_CKPT_STEPS = 16
MPA_MAX_DSTATE = 256

MPA_NOALLOC_SCRATCH_BYTES = 16 << 20

EXPORTS = ("mpa_version", "mpa_arch", "mpa_source_hash", "mpa_status_string", "mpa_sscan_fwd", "mpa_sscan_fwd_noalloc",
           "mpa_sscan_ckpt_elems", "mpa_sscan_fwd_workspace_bytes", "mpa_sscan_bwd", "mpa_sscan_bwd_workspace_bytes",
           "mpa_pscan_fwd", "mpa_pscan_bwd", "mpa_pscan_workspace_bytes", "mpa_ssm_step",
           "mpa_conv1d_fwd", "mpa_conv1d_bwd", "mpa_conv1d_bwd_workspace_bytes",
           "mpa_rmsnorm_fwd", "mpa_rmsnorm_bwd", "mpa_rmsnorm_bwd_workspace_bytes")


class SscanShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("batch", "seqlen", "dim", "dstate")] + \
               [("io_dtype", ctypes.c_int32), ("flags", ctypes.c_int32)] + \
               [(n, ctypes.c_int64) for n in (
                   "u_sb", "u_sl", "u_sd", "z_sb", "z_sl", "z_sd", "d_sb", "d_sl", "d_sd", "y_sb", "y_sl", "y_sd",
                   "g_sb", "g_sl", "g_sd", "bc_sb", "bc_sl", "dbc_sb", "dbc_sl")] + \
               [(n, ctypes.c_int32) for n in ("plan_states_per_lane", "plan_segments", "plan_flags", "delta_dtype")]


class ConvShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("batch", "seqlen", "dim")] + \
               [(n, ctypes.c_int32) for n in ("kernel", "io_dtype", "flags", "reserved")] + \
               [(n, ctypes.c_int64) for n in (
                   "x_sb", "x_sl", "x_sd", "y_sb", "y_sl", "y_sd", "g_sb", "g_sl", "g_sd")]


class PscanShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("batch", "seqlen", "dim", "dstate")] + \
               [("io_dtype", ctypes.c_int32), ("reverse", ctypes.c_int32)] + \
               [(n, ctypes.c_int64 * 4) for n in ("a_st", "x_st", "h_st", "ga_st", "gx_st")] + \
               [("plan_chunks", ctypes.c_int32), ("reserved", ctypes.c_int32)]


_lib = None


def load():
    """Open the library once; raise ImportError (never fall back) when it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python mamba.py_amd/build.py` "
            "(needs hipcc; targets gfx950).  There is no CPU or PyTorch fallback.")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise ImportError(f"cannot load {LIB_PATH}: {e}") from e
    vp, i64, i32, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_size_t
    lib.mpa_version.restype = ctypes.c_int
    lib.mpa_arch.restype = ctypes.c_char_p
    lib.mpa_source_hash.restype = ctypes.c_char_p
    lib.mpa_status_string.restype = ctypes.c_char_p
    lib.mpa_status_string.argtypes = [ctypes.c_int]
    sp = ctypes.POINTER(SscanShape)
    lib.mpa_sscan_fwd.argtypes = [sp] + [vp] * 14 + [sz, vp]
    lib.mpa_sscan_fwd_noalloc.argtypes = [sp] + [vp] * 13 + [vp]
    lib.mpa_sscan_fwd_workspace_bytes.argtypes = [sp, ctypes.c_int]
    lib.mpa_sscan_fwd_workspace_bytes.restype = sz
    lib.mpa_sscan_ckpt_elems.argtypes = [sp]
    lib.mpa_sscan_ckpt_elems.restype = i64
    lib.mpa_sscan_bwd.argtypes = [sp] + [vp] * 21 + [sz, vp]
    lib.mpa_sscan_bwd_workspace_bytes.argtypes = [sp]
    lib.mpa_sscan_bwd_workspace_bytes.restype = sz
    pp = ctypes.POINTER(PscanShape)
    lib.mpa_pscan_workspace_bytes.argtypes = [pp]
    lib.mpa_pscan_workspace_bytes.restype = sz
    lib.mpa_pscan_fwd.argtypes = [pp] + [vp] * 4 + [sz, vp]
    lib.mpa_pscan_bwd.argtypes = [pp] + [vp] * 6 + [sz, vp]
    lib.mpa_ssm_step.argtypes = [vp] * 11 + [i64] * 5 + [i32, i32, vp]
    cp = ctypes.POINTER(ConvShape)
    lib.mpa_conv1d_fwd.argtypes = [cp] + [vp] * 7
    lib.mpa_conv1d_bwd.argtypes = [cp] + [vp] * 9 + [sz, vp]
    lib.mpa_conv1d_bwd_workspace_bytes.argtypes = [cp]
    lib.mpa_conv1d_bwd_workspace_bytes.restype = sz
    f32 = ctypes.c_float
    lib.mpa_rmsnorm_fwd.argtypes = [vp] * 6 + [i64, i64, f32, i32, vp]
    lib.mpa_rmsnorm_bwd.argtypes = [vp] * 6 + [i64, i64, f32, i32, vp, sz, vp]
    lib.mpa_rmsnorm_bwd_workspace_bytes.argtypes = [i64, i64]
    lib.mpa_rmsnorm_bwd_workspace_bytes.restype = sz
    for name in EXPORTS:
        getattr(lib, name)
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().mpa_status_string(status).decode()
        raise RuntimeError(f"{what} failed with status {status}: {msg}")
