"""Achieved parity errors of the fused scan at the benchmark configurations.

    python tests/parity_report.py            (needs the GPU; prints a Markdown table)

For configs[0], [1] and [2] at full size: max|out - ref| / max|ref| per tensor (the error measure of
every parity test, see util.rel_err) of the HIP path against the float64 C oracle, next to the
tolerance the tests assert.  The same comparisons run, as assertions, in tests/test_sscan_gpu.py;
this script only prints the margins.
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))

import torch  # noqa: E402

import __graft_entry__ as entry  # noqa: E402
from oracle import c_oracle, scan_oracle as so  # noqa: E402
from util import GRAD_KEYS, TOL, rel_err, run_gpu_fwd_bwd  # noqa: E402

CONFIGS = [
    ("configs[0]", (2, 64, 32, 16), torch.float32, 1000),
    ("configs[1]", (8, 2048, 1536, 16), torch.float32, 1001),
    ("configs[2]", (4, 4096, 4096, 16), torch.bfloat16, 1002),
]


def main():
    pkg = entry.load_package()
    dev = torch.device("cuda:0")
    keys = ("y",) + GRAD_KEYS
    print("| configuration | I/O | tolerance | " + " | ".join(keys) + " |")
    print("|---|---|---|" + "---|" * len(keys))
    for name, shape, dtype, seed in CONFIGS:
        inp = so.make_inputs(*shape, seed=seed, dtype=dtype)
        ref = c_oracle.sscan_fwd_bwd(**inp)
        for reverse in (False, True):
            if reverse:
                fl = {k: (v.flip(1) if v.dim() == 3 else v) for k, v in inp.items()}
                ref = c_oracle.sscan_fwd_bwd(**fl)
                ref = {k: (v.flip(1) if k in ("y", "dx", "ddelta", "dB", "dC") else v) for k, v in ref.items()}
            got = run_gpu_fwd_bwd(pkg, inp, dev, reverse=reverse)
            errs = [rel_err(got[k], ref[k]) for k in keys]
            label = name + (" reverse" if reverse else "")
            print(f"| {label} B{shape[0]} L{shape[1]} ED{shape[2]} N{shape[3]} | {str(dtype).split('.')[-1]} | "
                  f"{TOL[dtype]:.0e} | " + " | ".join(f"{e:.2e}" for e in errs) + " |", flush=True)
            assert max(errs) <= TOL[dtype]
            del got


if __name__ == "__main__":
    main()
