import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_lib():
    import oracle
    return oracle.load()


@pytest.fixture(scope="session")
def gpu():
    """The C-ABI library plus torch as device-memory plumbing."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from juzhen_amd import capi
    capi.load()  # raises if libjzhip.so is missing: no fallback
    return capi.jz


@pytest.fixture(autouse=True)
def _release_kept_buffers():
    yield
    import util
    util._KEEP.clear()
