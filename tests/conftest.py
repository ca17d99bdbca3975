import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run with -m gpu on the GPU box)")


def _gpu_present() -> bool:
    try:
        from aster_amd.execution import system_has_gpu

        return system_has_gpu("gfx950")
    except Exception:
        return False


@pytest.fixture(scope="session")
def gpu():
    """Skips when no gfx950 device is visible; the HIP library itself must load."""
    from aster_amd import _capi

    _capi.load()  # a missing library is an error, never a skip
    if not _gpu_present():
        pytest.skip("no gfx950 GPU visible")
    return True


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN
