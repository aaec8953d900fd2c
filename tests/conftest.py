import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def cx8():
    """The 8-core machine description the reference was probed with."""
    import oracle
    return oracle.make_cntx(mr=6, nr=16, L1=48 << 10, L2=2 << 20, L3=105 << 20, ncores=8)
