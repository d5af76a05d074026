import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def _gpu_count():
    from rwkv_lightning_cuda_amd import hip
    return hip.device_count()


@pytest.fixture(scope="session")
def gpu():
    """The loaded HIP library binding; GPU tests fail (not skip) when the library is missing."""
    from rwkv_lightning_cuda_amd import hip
    hip.load()
    if hip.device_count() < 1:
        pytest.fail("no GPU visible to librwkv_hip.so")
    return hip


@pytest.fixture(scope="session")
def orc():
    import oracle
    oracle.lib()
    return oracle


def rel_err(got, ref):
    """Normalised max error used for the floating-point bars: max|got-ref| / max(|ref|)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.max(np.abs(got - ref)) / max(float(np.max(np.abs(ref))), 1e-30))


def elem_err(got, ref):
    """Element-wise error with a floor at the tensor's rms: max_i |d_i| / (|ref_i| + rms(ref))."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) + 1e-30
    return float(np.max(np.abs(got - ref) / (np.abs(ref) + rms)))
