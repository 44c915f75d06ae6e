import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def nmse(got, want):
    """Normalised mean squared error against a float64 reference."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    den = float(np.sum(want * want))
    num = float(np.sum((got - want) ** 2))
    return num / den if den > 0 else num


def rel_l2(got, want):
    return float(np.sqrt(nmse(got, want)))


@pytest.fixture(scope="session")
def dev():
    """One device context for the whole GPU session.  No fallback: a missing
    library or GPU is an error, not a skip."""
    from jitllm_amd.device import Device
    d = Device(device=0, act_window=32)
    yield d
    d.close()


def _devbuf(arr=None, shape=None, dtype=None, fill=None):
    """A numpy array mirrored in device memory (hipMalloc through ctypes)."""
    from jitllm_amd.hipmem import DeviceArray
    return DeviceArray(arr, shape, dtype, fill)


@pytest.fixture(scope="session")
def devbuf(dev):
    return _devbuf
