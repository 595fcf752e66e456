import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def package():
    return importlib.import_module("tokspur-public_amd")


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    return oracle.lib()


@pytest.fixture(scope="session")
def ref():
    from oracle import oracle
    r = oracle.ref()
    if r is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    return r


@pytest.fixture(scope="session", params=["oracle", "reference"])
def cpu(request):
    """The C restatement and, where oracle/_ref has been built, the reference's own CPU code."""
    from oracle import oracle
    if request.param == "oracle":
        return oracle.lib()
    r = oracle.ref()
    if r is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    return r


@pytest.fixture(scope="session")
def synth():
    return importlib.import_module("tokspur-public_amd.synth")


@pytest.fixture(scope="session")
def tsp():
    """The product's C-ABI library through ctypes."""
    return importlib.import_module("tokspur-public_amd.capi")


@pytest.fixture(scope="session")
def gpu(tsp):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    torch.cuda.set_device(0)
    return tsp.Device()
