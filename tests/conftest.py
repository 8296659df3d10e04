import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def pkg():
    """The product package, with its HIP library built if it is not there yet."""
    entry.ensure_built()
    return entry.load_package()


@pytest.fixture(scope="session")
def orc():
    from oracle import moe_oracle

    return moe_oracle


@pytest.fixture(scope="session")
def dev():
    import torch

    return torch.device("cuda:0")
