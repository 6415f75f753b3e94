import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import checkers
    return checkers.Oracle()


@pytest.fixture(scope="session")
def reflib():
    import checkers
    if not checkers.have_ref():
        pytest.skip("oracle/_ref/libxnor_nn_ref.so not built (needs the upstream sources)")
    return checkers.RefLib()


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "golden.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def gpu():
    """torch device handle; fails (not skips) when the marker promised a GPU."""
    import torch
    assert torch.cuda.is_available(), "tests marked gpu need a GPU"
    return torch.device("cuda:0")
