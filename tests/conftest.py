import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import __graft_entry__ as ge
    return ge.import_oracle()


@pytest.fixture(scope="session")
def pkg():
    """The GPU package; importing it loads libmoe_gfx950.so (and fails if it has not been built)."""
    import __graft_entry__ as ge
    return ge.import_package()


@pytest.fixture(scope="session")
def wl(pkg):
    import importlib
    return importlib.import_module("gpt_oss_amd_amd.workloads")


@pytest.fixture(scope="session")
def dev(pkg):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
