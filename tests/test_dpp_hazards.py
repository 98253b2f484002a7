"""Static check of the generated gfx950 code of the scan kernels (CPU only; needs hipcc).

The kernels use DPP instructions written as inline assembly (common.h: fmac_bcast,
mul_bcast).  On gfx9-family hardware a DPP instruction that reads a vector register written
by a VALU instruction less than two wait states earlier reads the old value; the compiler
inserts the wait states for its own DPP instructions but cannot see into inline assembly.
This test compiles the two scan kernels to assembly and checks that no DPP instruction reads,
as its DPP operand, a register that one of the two preceding instructions wrote on the VALU.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "mamba.py_amd", "csrc")


def _build_recipe():
    """the flags libmambapy_amd.so is built with (the checked code must be the shipped code)"""
    import importlib.util
    spec = importlib.util.spec_from_file_location("mpa_build", os.path.join(ROOT, "mamba.py_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod



def _vgprs(tok):
    tok = tok.strip().rstrip(",")
    m = re.match(r"^v(\d+)$", tok)
    if m:
        return {int(m.group(1))}
    m = re.match(r"^v\[(\d+):(\d+)\]$", tok)
    return set(range(int(m.group(1)), int(m.group(2)) + 1)) if m else set()


def find_dpp_hazards(asm_text):
    ins = []
    for raw in asm_text.splitlines():
        line = raw.split(";")[0].strip()
        if line and not line.startswith(".") and not line.endswith(":"):
            ins.append(line)
    hazards, ndpp = [], 0
    for i, line in enumerate(ins):
        op = line.split()[0]
        if "_dpp" not in op:
            continue
        ndpp += 1
        operands = line.split(None, 1)[1].split(",")
        src0 = _vgprs(operands[1].split()[0]) if len(operands) > 1 else set()
        waited, j = 0, i - 1
        while j >= 0 and waited < 2:
            prev = ins[j]
            pop = prev.split()[0]
            if pop == "s_nop":
                waited += int(prev.split()[1]) + 1
            else:
                if pop.startswith("v_") and len(prev.split(None, 1)) > 1 \
                        and _vgprs(prev.split(None, 1)[1].split(",")[0]) & src0:
                    hazards.append((prev, line))
                    break
                waited += 1
            j -= 1
    return ndpp, hazards


def test_checker_sees_a_hazard_and_accepts_wait_states():
    bad = "v_add_f32_e32 v3, v1, v2\nv_add_f32_dpp v4, v3, v3 row_mirror row_mask:0xf bank_mask:0xf\n"
    ok = "v_add_f32_e32 v3, v1, v2\ns_nop 1\nv_add_f32_dpp v4, v3, v3 row_mirror row_mask:0xf bank_mask:0xf\n"
    far = "v_add_f32_e32 v3, v1, v2\nv_mov_b32_e32 v9, v8\nv_mov_b32_e32 v10, v8\nv_add_f32_dpp v4, v3, v3 row_mirror\n"
    assert find_dpp_hazards(bad)[1] and not find_dpp_hazards(ok)[1] and not find_dpp_hazards(far)[1]


@pytest.mark.parametrize("src", ["sscan_fwd.hip", "sscan_bwd_fast.hip"])
def test_no_dpp_operand_is_read_too_early(src, tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    out = tmp_path / (src + ".s")
    recipe = _build_recipe()
    flags = [recipe.OPT_LEVEL.get(src, recipe.DEFAULT_OPT_LEVEL), *[f for f in recipe.HIPCC_FLAGS if f != "-fPIC"],
             "-S", "--cuda-device-only"]
    res = subprocess.run([hipcc, *flags, os.path.join(CSRC, src), "-o", str(out)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    ndpp, hazards = find_dpp_hazards(out.read_text())
    assert ndpp > 100, "the kernels are expected to contain DPP instructions"
    assert not hazards, hazards[:5]
