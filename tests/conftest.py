import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) GPU")
    config.addinivalue_line("markers", "slow: long-running test")


def _has_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:  # noqa: BLE001
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)


@pytest.fixture(autouse=True)
def _stop_leftover_watchdogs():
    """Engines that tests drop without ``shutdown`` leave their watchdog threads polling the
    process-wide communicator registry; a later test that records a collective error there on
    purpose would be ended by one of them (exit 75).  Stop them when the test that made them ends."""
    yield
    from ome_amd.runtime import watchdog

    watchdog.stop_all()
