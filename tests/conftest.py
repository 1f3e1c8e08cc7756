import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 (MI355X) GPU; runs through the HIP library")


@pytest.fixture(autouse=True)
def _seed():
    # the reference suite seeds every test with 1235 (tests/conftest.py:43-47)
    torch.manual_seed(1235)
    yield


@pytest.fixture()
def clean_registry():
    """Run a test against an empty backend registry and put the real one back afterwards."""
    from tileops_amd import backend

    backend.ensure_loaded()
    saved = backend.snapshot()
    backend.restore(backend._State({}, {}, [], None))
    yield backend
    backend.restore(saved)


def require_gfx950():
    from tileops_amd import native

    if not torch.cuda.is_available():
        pytest.fail("GPU test collected on a machine without a GPU (run with -m 'not gpu')")
    native.require_gfx950(torch.device("cuda", 0))
    native.load()
