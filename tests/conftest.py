import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu():
    try:
        import morok_amd

        return morok_amd.device_count() > 0
    except Exception:
        return False


@pytest.fixture(scope="session")
def oracle():
    from tests.oracle_lib import Oracle

    return Oracle()


@pytest.fixture(scope="session")
def dev():
    import morok_amd

    return morok_amd.Device("HIP")


def pytest_collection_modifyitems(config, items):
    # GPU tests must never silently pass on a box without a GPU: they fail in the
    # library (no device) rather than being skipped, except when explicitly deselected.
    pass
