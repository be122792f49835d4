import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for p in (HERE, ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    """tests/golden/record_fixtures.npz: inputs/expected records dumped from the
    compiled reference by tests/golden/make_fixtures.py."""
    return np.load(os.path.join(HERE, "golden", "record_fixtures.npz"))


@pytest.fixture(scope="session")
def pkg():
    """The product package (loads libcfpolicy.so; no fallback)."""
    import __graft_entry__ as ge
    return ge.load_package()


@pytest.fixture(scope="session")
def cuda(pkg):
    import torch
    if not torch.cuda.is_available():
        pytest.fail("gpu-marked test selected but no GPU is visible")
    torch.cuda.set_device(0)
    return torch.device("cuda:0")
