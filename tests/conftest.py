import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def po():
    """The CPU oracle (test infrastructure)."""
    from oracle import pyoracle
    pyoracle.lib()
    return pyoracle


@pytest.fixture(scope="session")
def liger():
    """The shipped package (ctypes over the native libraries); import fails loudly if they are not built."""
    return importlib.import_module("24ppopp-liger_amd")


@pytest.fixture(scope="session")
def dev(liger):
    """GPU helpers: torch is used for device memory and streams only."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from tests import gpu_util
    return gpu_util.Dev(liger)


def max_rel_err(a, b):
    """max |a - b| / max |b|: the layer-level metric of the stated tolerance (<= 1e-2 for fp16)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def elementwise_err(a, b):
    """max over the elements of |a - b| / (|b| + rms(b)): a bound of 1e-2 on it says |a - b| <= 1e-2 |b| + 1e-2 rms(b) for
    every element, which (unlike max_rel_err, whose yardstick is the largest output) a wrong small output cannot hide behind."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    rms = max(float(np.sqrt(np.mean(b * b))), 1e-30)
    return float((np.abs(a - b) / (np.abs(b) + rms)).max())


def rms_rel_err(a, b):
    """rms(a - b) / rms(b): the typical error, next to the two worst-case figures."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.sqrt(np.mean((a - b) ** 2)) / max(float(np.sqrt(np.mean(b * b))), 1e-30))
