"""Shared test plumbing: import paths, the `gpu` marker, small helpers."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "ladder-residual-inference_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def bf16_round_np(x):
    """Round float64/float32 values to the nearest bfloat16 (ties to even) with integer
    arithmetic only -- independent of torch's cast.  Returns float32."""
    a = np.asarray(x, dtype=np.float32).copy()
    u = a.view(np.uint32)
    lsb = (u >> 16) & 1
    r = (u + np.uint32(0x7FFF) + lsb) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


@pytest.fixture
def bf16_round():
    return bf16_round_np
