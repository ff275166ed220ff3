"""pytest configuration: import paths, the ``gpu`` marker and shared fixtures."""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "dartmoq-qwen3.5_amd")
for p in (ROOT, PKG_DIR):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def small_layer():
    """16 experts, H=256, I=256, top-4, mixed 2/1/4-bit pools (CPU oracle object)."""
    from oracle import moe
    bits = moe.assign_bits(16, {2: 0.75, 1: 0.125, 4: 0.125}, seed=1)
    return moe.build_layer(256, 256, 16, 4, bits, seed=3)


@pytest.fixture(scope="session")
def small_layer_bit4():
    from oracle import moe
    return moe.build_layer(256, 256, 8, 2, [4] * 8, seed=5)
