import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle binding (built on demand)."""
    from oracle import binding
    binding.lib()
    return binding


@pytest.fixture(scope="session")
def hip():
    """The C-ABI HIP library; fails loudly when it is missing or no GPU is present."""
    from cera_amd import hip_api
    ctx = hip_api.Context(0)
    yield ctx
    ctx.close()
