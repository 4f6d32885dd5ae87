import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc
    orc.build()
    return orc


@pytest.fixture(scope="session")
def lib():
    from mcsparse_amd import _lib
    return _lib.load()


@pytest.fixture(scope="session")
def torch_gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a -m gpu test was started without a GPU")
    torch.cuda.set_device(0)
    return torch


@pytest.fixture()
def handle(torch_gpu):
    from mcsparse_amd import api
    h = api.Handle(stream=torch_gpu.cuda.current_stream().cuda_stream)
    yield h
    torch_gpu.cuda.synchronize()
    h.destroy()
