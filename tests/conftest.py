import os
import random
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _reseed():
    # the reference reseeds every test to 0xC001A1 (tests/pytest_working/conftest.py:34-44)
    torch.manual_seed(0xC001A1)
    np.random.seed(0xC001A1 & 0xFFFFFFFF)
    random.seed(0xC001A1)
    yield


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__ as ge
    return ge.load_package()


@pytest.fixture(scope="session")
def dev(pkg):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
