"""The quantizer divides by the group scale with a three-instruction sequence instead of a general IEEE division
(kvcomp_amd/csrc/kvc_quant_math.h).  tests/division_check.c walks every (fp16 x, positive fp16 scale) pair on
the CPU, with the same IEEE fp32 operations, and compares with the true quotient."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_three_instruction_division_is_exact_for_all_fp16_pairs(tmp_path):
    exe = str(tmp_path / "division_check")
    subprocess.check_call(["gcc", "-O2", "-mfma", "-mf16c", "-fopenmp", "-ffp-contract=off", "-o", exe,
                           os.path.join(HERE, "division_check.c"), "-lm"])
    out = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=600).stdout.split()
    vals = dict(zip(out[0::2], (int(v) for v in out[1::2])))
    assert vals["pairs"] == 31743 * 63488
    assert vals["fp32_mismatches"] == 0 and vals["fp16_mismatches"] == 0
    assert vals["zero_sign_only"] == 31743          # x = -0: +0 instead of -0, one per scale
