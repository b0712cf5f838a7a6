import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__
    return __graft_entry__.load_package()


@pytest.fixture(scope="session")
def golden_tables():
    return np.load(GOLDEN / "dequant_tables.npz")


@pytest.fixture(scope="session")
def golden_linear():
    return np.load(GOLDEN / "linear_cases.npz")


@pytest.fixture(scope="session")
def gpu(pkg):
    """(torch, device, library) on the GPU box; the library synchronises after every call."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    lib = pkg.library()
    lib.set_sync(True)
    return torch, torch.device("cuda:0"), lib
