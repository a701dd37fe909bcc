import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def worker():
    """One ChipWorker for the whole GPU session (the library binds one device per process)."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pypto_amd.runtime import ChipWorker, RunConfig

    w = ChipWorker(RunConfig(platform="mi355x", device_id=0))
    yield w
    w.close()
