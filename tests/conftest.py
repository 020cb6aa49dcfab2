import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # The small layers of this suite (8 .. 32 experts) stand in for the DeepSeek-V3 shape's paths:
    # they keep the V3 token thresholds, so that "T = 16" is the one-launch decode path and
    # "T = 130" the grouped GEMM on them as on the real shape.  (The library's own defaults follow
    # the picks per expert and would send 16 tokens on 16 experts to the GEMMs; those defaults are
    # checked in tests/test_capi.py, and layers of 64 experts and more run on them.)
    try:
        from deepstrix_amd.executor import MoeLayer
        MoeLayer.v3_thresholds_below_experts = 64
    except ImportError:      # no torch in this interpreter: the CPU-only tests do not need it
        pass


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
