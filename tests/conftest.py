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
    from oracle import rock_oracle
    rock_oracle.lib()  # builds on first use if the .so is absent
    return rock_oracle


@pytest.fixture(scope="session")
def rock():
    """The product library through its Python binding; fails loudly if the
    HIP library has not been built."""
    import rocmlir_amd
    rocmlir_amd.load_library()
    return rocmlir_amd


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    return torch.device("cuda:0")
