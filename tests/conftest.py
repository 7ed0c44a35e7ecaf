import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def psi():
    """The shipped package (ctypes over libpsi_hip.so)."""
    return importlib.import_module("psi-dec_amd")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle: the checker, never the thing under test."""
    from oracle import binding

    binding.load()
    return binding


@pytest.fixture(scope="session")
def host_oracle():
    from oracle import host_oracle

    return host_oracle


@pytest.fixture(scope="session")
def device(psi):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = psi.Device(0)
    yield dev
    dev.close()
