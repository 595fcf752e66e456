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
def _device(tsp):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    torch.cuda.set_device(0)
    return tsp.Device()


@pytest.fixture
def gpu(_device):
    """The device with a clean sticky error word, so one failing test cannot poison the next."""
    _device.clear_error()
    return _device


def nmse(got, ref):
    """Normalised mean squared error, the engine's bound for MoE outputs (native/tests/test_planar_pack_v3.cpp:181-192)."""
    import numpy as np
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert np.isfinite(got).all() and np.isfinite(ref).all()
    return float(((got - ref) ** 2).sum() / max((ref ** 2).sum(), 1e-300))


def max_rel_error(got, ref):
    """max |a - e| / max(1, |e|, rms(e_row)): element-wise error in units of the row's own scale. With f32
    accumulation the absolute error grows with sum |w||x|, so an element that cancels to near zero in a row of
    large values cannot be judged against its own magnitude."""
    import numpy as np
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    ref2 = ref.reshape(-1, ref.shape[-1]) if ref.ndim > 1 else ref.reshape(1, -1)
    got2 = got.reshape(ref2.shape)
    rms = np.sqrt((ref2 ** 2).mean(axis=1, keepdims=True))
    return float(np.max(np.abs(got2 - ref2) / np.maximum(np.maximum(1.0, np.abs(ref2)), rms)))


def reference_metric(got, ref):
    """The engine's own scaled error, max |a - e| / max(1, |e|) (native/tools/ffn_check.cpp:48-56), and where it is reached:
    (value, flat index, actual, expected, rms of the expected row). With outputs of magnitude 1e3..1e8, as the synthetic
    configurations produce, an element that cancels to near zero is judged against 1 while the f32 accumulation error of
    its row scales with the row's magnitude; the number is printed and recorded for that reason, and asserted where it
    holds."""
    import numpy as np
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    ref2 = ref.reshape(-1, ref.shape[-1]) if ref.ndim > 1 else ref.reshape(1, -1)
    got2 = got.reshape(ref2.shape)
    err = np.abs(got2 - ref2) / np.maximum(1.0, np.abs(ref2))
    at = int(np.argmax(err))
    r = at // ref2.shape[1]
    return float(err.reshape(-1)[at]), at, float(got2.reshape(-1)[at]), float(ref2.reshape(-1)[at]), float(np.sqrt((ref2[r] ** 2).mean()))
