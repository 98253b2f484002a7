"""Build recipe for libmambapy_amd.so (hand-written HIP kernels, gfx950 only).

    python mamba.py_amd/build.py          # compile every csrc/*.hip and link the library

The library is built in-tree (csrc/libmambapy_amd.so) with hipcc; packed-FP32 code
generation is switched off for the device pass.
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(CSRC, "libmambapy_amd.so")
SOURCES = ["sscan_fwd.hip", "sscan_bwd.hip", "sscan_bwd_fast.hip", "pscan.hip", "step.hip", "conv1d.hip", "rmsnorm.hip"]
ARCH = "gfx950"
HIPCC_FLAGS = [f"--offload-arch={ARCH}", "-fPIC", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]
# Optimisation level per source.  The fast backward kernel is built at -O2: at -O3 the compiler
# hoists more address arithmetic out of the service waves' tile loop than the scalar register
# file holds, parks it in lanes of a vector register and reads it back with vector instructions
# (gated backward at (4, 4096, 4096): 0.721 ms at -O3, 0.702 ms at -O2; the ungated kernels and
# every other source measure the same either way).
OPT_LEVEL = {"sscan_bwd_fast.hip": "-O2"}
DEFAULT_OPT_LEVEL = "-O3"


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def source_hash() -> str:
    """sha256 over the kernel sources (csrc/*.hip, csrc/*.h and the public header, by name) and the
    compiler flags.  The
    library is built with this string inside (mpa_source_hash()); a profile summary that quotes
    counters of a kernel names the hash of the sources it was measured on."""
    h = hashlib.sha256()
    files = sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".h")))
    for path in [os.path.join(CSRC, f) for f in files] + [os.path.join(_HERE, "..", "include", "mambapy_amd.h")]:
        h.update(os.path.basename(path).encode() + b"\0")
        h.update(open(path, "rb").read())
    # (the compiler flags decide the generated code as much as the sources do)
    h.update(repr((HIPCC_FLAGS, DEFAULT_OPT_LEVEL, sorted(OPT_LEVEL.items()))).encode())
    return h.hexdigest()[:16]


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), OPT_LEVEL.get(src, DEFAULT_OPT_LEVEL), *HIPCC_FLAGS, f'-DMPA_SOURCE_SHA="{source_hash()}"',
           "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False) -> str:
    """Compile all sources for gfx950 and link csrc/libmambapy_amd.so.  Always recompiles."""
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
