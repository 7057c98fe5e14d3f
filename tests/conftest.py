import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _have_gpu() -> bool:
    try:
        from mononn_amd import binding
        return binding.device_count() > 0
    except Exception:
        return False


@pytest.fixture(scope="session")
def gpu_device():
    if not _have_gpu():
        pytest.fail("no GPU visible: -m gpu tests must run on the MI355X box")
    return 0
