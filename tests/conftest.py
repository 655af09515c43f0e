import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import pccl_oracle
    pccl_oracle.lib()
    return pccl_oracle


@pytest.fixture(scope="session")
def hip():
    """The product library on a GPU box; no fallback of any kind."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pccl_amd import hip as h
    h.lib()
    torch.cuda.init()
    assert h.device_count() >= 1
    return h
