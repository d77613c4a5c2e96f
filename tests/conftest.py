import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before any GPU work starts, so a fault can be attributed
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield


class FusedMode:
    """One arithmetic / kernel variant of the fused decode + matvec kernels."""
    def __init__(self, name, rounded, mfma):
        self.name, self.rounded, self.mfma = name, rounded, mfma
        # against fp32 attention over the fp16 cache that get() returns: the rounded kernels reproduce that cache's
        # values exactly (1e-3); the unrounded ones differ from it by the cache's own rounding noise, which the
        # softmax amplifies to a few 1e-3 at these sizes
        self.tol_vs_fp16_cache = 1e-3 if rounded else 3e-3

    def __repr__(self):
        return self.name


FUSED_MODES = [FusedMode("rounded", 1, -1),            # the default: fp16-rounded dequantization, matrix-core kernels
               FusedMode("rounded_fma", 1, 0),         # the same arithmetic on the fp32-FMA kernels
               FusedMode("unrounded", 0, 0),           # dequantized values left in fp32, fp32-FMA kernels
               FusedMode("unrounded_mfma", 0, -1)]     # the same on the matrix-core kernels


@pytest.fixture(params=FUSED_MODES, ids=[m.name for m in FUSED_MODES])
def fused_mode(request):
    """Runs the test once per variant of the fused kernels (options restored afterwards)."""
    from kvcomp_amd import _lib
    m = request.param
    was_r, was_m = _lib.set_option("fused_rounded", m.rounded), _lib.set_option("fused_mfma", m.mfma)
    try:
        yield m
    finally:
        _lib.set_option("fused_rounded", was_r)
        _lib.set_option("fused_mfma", was_m)
