import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "hyper-parallel_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu")


def pytest_collection_modifyitems(config, items):
    """GPU tests fail (not skip) when selected without a GPU; they are simply deselected by -m "not gpu"."""
    return


@pytest.fixture(scope="session")
def gpu():
    import torch
    assert torch.cuda.is_available(), "this test needs a GPU"
    import hpfp8
    assert hpfp8._lib.load().hpfp8_check_device() == 0, hpfp8._lib.load().hpfp8_last_error()
    return torch.device("cuda:0")
