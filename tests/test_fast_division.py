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


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_packed_fp16_quantizer_rounds_to_the_reference_integer(tmp_path):
    """The fused store quantizes two values per instruction in fp16 (kvc_quant_pair_biased): tests/division_check_f16.c
    models every fp16 operation of it exactly and compares rint(q) with rint(RN16(x / scale)) for all fp16 x and every
    mantissa of the scale at a spread of exponents (KVCOMP_FULL_CHECKS=1: every scale, 1.5e9 pairs, about a minute on
    eight cores; the default subset takes a third of that)."""
    exe = str(tmp_path / "division_check_f16")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-o", exe, os.path.join(HERE, "division_check_f16.c"), "-lm"])
    full = os.environ.get("KVCOMP_FULL_CHECKS") == "1"
    out = subprocess.run([exe] + (["all"] if full else []), check=True, capture_output=True, text=True, timeout=1800).stdout.split()
    vals = dict(zip(out[0::2], (int(v) for v in out[1::2])))
    assert vals["scales"] == (31743 if full else 12 * 1024 - 1)
    assert vals["pairs"] > 5e8 and vals["mismatches"] == 0
