import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (MI355X) and the built libtrakhip.so")


@pytest.fixture(scope="session")
def c_oracle():
    from oracle import jl_oracle

    jl_oracle.build_c_oracle()
    return jl_oracle.COracle()


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("test marked gpu but no GPU is visible")
    from trak_amd import _lib

    _lib.load()  # raises ImportError when the HIP library is not built: no fallback
    return torch.device("cuda:0")
