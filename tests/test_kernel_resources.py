"""The code generator's account of every kernel, written by the build beside the objects: no kernel may spill vector
registers, and the kernels of the decode-attention and store paths use no scratch memory at all.  A spill in a
per-tile path shows up as HBM writes of the size of the compressed stream itself (the V kernel for head sizes that are
no multiple of 64 once wrote 37 MB per launch instead of 13 MB because one loop variant needed a single register
beyond what six waves per SIMD leave)."""
import json
import os

import pytest

from kvcomp_amd import build as B

# kernels allowed a private segment, with the bytes per lane they may use: the V expansion keeps the raw words of a
# tile in a small array that it indexes with a run-time slot (not a spill, and once per tile)
SCRATCH_ALLOWED = {"_Z17kvc_expand_kernelILi2ELb1EEv12KvcFusedArgs": 16}


@pytest.fixture(scope="module")
def resources():
    if not os.path.exists(B.RESOURCES):
        B.build(verbose=False)
    with open(B.RESOURCES) as f:
        return json.load(f)


def test_every_source_reports_its_kernels(resources):
    assert set(resources) == {os.path.basename(s) for s in B.sources()}
    names = [k for per in resources.values() for k in per]
    assert len(names) == len(set(names))
    for want in ("kvc_fused_mfma_kernel", "kvc_fused_kernel", "kvc_expand_kernel", "kvc_encode_once_kernel",
                 "kvc_store_count_kernel", "kvc_store_emit_kernel", "kvc_attention_combine_kernel", "kvc_build_lut_kernel"):
        assert any(want in n for n in names), want


def test_no_kernel_spills_vector_registers_or_uses_scratch(resources):
    for src, per in resources.items():
        for name, r in per.items():
            assert r["VGPRs Spill"] == 0, "%s: %s spills %d vector registers" % (src, name, r["VGPRs Spill"])
            assert r["Dynamic Stack"] == "False", "%s: %s has a dynamic stack" % (src, name)
            assert r["ScratchSize [bytes/lane]"] <= SCRATCH_ALLOWED.get(name, 0), \
                "%s: %s uses %d bytes of scratch per lane" % (src, name, r["ScratchSize [bytes/lane]"])


def test_matrix_core_kernels_keep_the_occupancy_they_are_launched_for(resources):
    """Launch bounds promise waves per SIMD; the register count the generator settled on must keep that promise
    (with one query head per KV head: 8 for the K kernel, 7 for the V kernels that decode attention uses -- softmax on
    the fly, kinds 3 and 4 --, at least 6 for the others)."""
    per = {}
    for src in ("kvc_fused_mfma.hip", "kvc_fused_mfma_v96.hip"):
        per.update(resources[src])
    assert any("ILi1ELi4ELb1E" in name for name in resources["kvc_fused_mfma_v96.hip"])
    for name, r in per.items():
        if "kvc_fused_mfma_kernel" not in name:
            continue
        if "ILi1ELi0E" in name:
            assert r["Occupancy [waves/SIMD]"] >= 8, (name, r)
        elif "ILi1ELi3E" in name or "ILi1ELi4E" in name:
            assert r["Occupancy [waves/SIMD]"] >= 7, (name, r)
        elif "ILi1E" in name:
            assert r["Occupancy [waves/SIMD]"] >= 6, (name, r)


def test_hot_kernels_keep_their_scalars_in_scalar_registers(resources):
    """A scalar value that does not fit the scalar register file lives in a lane of a vector register, and every access
    to it is an instruction on the vector ALU that these kernels are bound by (the one-pass encoder once kept 32 loop-
    invariant lane masks that way: 87 to 265 spilled scalars, 12 % of its vector instructions)."""
    ceilings = {"kvc_encode_once_kernel": 16, "kvc_fused_mfma_kernelILi1ELi0E": 24, "kvc_fused_mfma_kernelILi1ELi4E": 8,
                "kvc_fused_mfma_kernelILi4ELi0E": 8, "kvc_fused_mfma_kernelILi4ELi3E": 8}
    seen = set()
    for per in resources.values():
        for name, r in per.items():
            for key, most in ceilings.items():
                if key in name:
                    seen.add(key)
                    assert r["SGPRs Spill"] <= most, "%s spills %d scalar registers" % (name, r["SGPRs Spill"])
    assert seen == set(ceilings)
