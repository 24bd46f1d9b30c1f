import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "flash-dmattn_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


@pytest.fixture(autouse=True)
def _library_decides_compaction():
    """Tests that pin the compaction policy (tests/_util.set_compact) do not leak it into the next test."""
    yield
    mod = sys.modules.get("flash_sparse_attn._cabi")
    if mod is not None:
        mod.set_compact_mode(mod.COMPACT_AUTO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) when no device is visible, so `-m "not gpu"` and a plain
    run both stay green on a CPU-only machine."""
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
