import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture
def lib_option():
    """Sets process-wide diagnostic switches of the library for one test and restores them after it:
    lib_option("force_generic"), lib_option("target_items", 64), lib_option("separate_merge")."""
    from xllm_wxh_amd import ops

    active = []

    def set_option(name, value=1):
        ctx = ops.option(name, value)
        ctx.__enter__()
        active.append(ctx)

    yield set_option
    for ctx in reversed(active):
        ctx.__exit__(None, None, None)
