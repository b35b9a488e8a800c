import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for q in (str(ROOT), str(ROOT / "tests")):
    if q not in sys.path:
        sys.path.insert(0, q)


# The tests that compare kernel forms steer the library's measurement switches: opt in before the library loads.
os.environ.setdefault("DGPP_AMD_BENCH", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """torch device for the GPU tests; the HIP library must be built (no fallback)."""
    import torch
    from dgpp_amd import _lib

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    _lib.load()
    return torch.device("cuda:0")
