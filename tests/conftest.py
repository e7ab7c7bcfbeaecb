import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    return oracle


@pytest.fixture(scope="session")
def gpu():
    """One device context for the whole GPU session (tests marked `gpu` only)."""
    from aion_amd.backend import HipBackend
    b = HipBackend(0)
    yield b
    b.close()


def norm_err(got, ref):
    """max |err| / max(|ref|, 1e-3 * rms(ref)): elementwise relative error with a floor, since an
    output that is a sum of +- terms can sit arbitrarily close to zero."""
    import numpy as np
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt((ref ** 2).mean())) if ref.size else 0.0
    den = np.maximum(np.abs(ref), 1e-3 * rms + 1e-30)
    return float((np.abs(got - ref) / den).max()) if ref.size else 0.0


def rms_err(got, ref):
    """max |err| / rms(ref)"""
    import numpy as np
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt((ref ** 2).mean())) if ref.size else 0.0
    return float(np.abs(got - ref).max() / (rms + 1e-30)) if ref.size else 0.0
