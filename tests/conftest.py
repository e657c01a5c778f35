import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _sort_parameters_at_their_defaults():
    """The sort's test hooks are process-wide: whatever a test sets (or leaves
    set when it fails half way) is put back before the next test runs."""
    yield
    try:
        from ilgpu_amd import capi
    except Exception:
        return
    for parameter in (capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT,
                      capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU,
                      capi.SORT_PARAM_ONE_TILE_KERNEL,
                      capi.SORT_PARAM_SHORT_TILE_MAX_TILES):
        capi.lib().ilgpu_hip_sort_set_parameter(parameter, -1)
