import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def ops32(gpu):
    import torch
    from hf_cpu_amd.kernels import Ops
    return Ops(torch.float32, gpu)


@pytest.fixture(scope="session")
def ops16(gpu):
    import torch
    from hf_cpu_amd.kernels import Ops
    return Ops(torch.bfloat16, gpu)
