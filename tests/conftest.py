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


def _row_err(got, ref, norm):
    import numpy as np
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if ref.size == 0:
        return 0.0
    den = norm(ref)
    err = np.abs(got - ref).max(axis=-1)
    rel = np.where(den > 0, err / np.where(den > 0, den, 1.0), np.where(err > 0, np.inf, 0.0))
    return float(rel.max())


def row_rel_err(got, ref):
    """Attention's gate: the max relative error of every output row (last axis = one head's values for one query) in
    the maximum norm, max |err| / max |ref row|, worst row. An attention output is an average of values, so its size
    shrinks with the number of visible keys; an absolute bound that fits a row seeing one key says nothing about a row
    seeing 16384. A row whose reference is all zeros (empty window) must be all zeros."""
    import numpy as np
    return _row_err(got, ref, lambda r: np.abs(r).max(axis=-1))


def row_rms_err(got, ref):
    """The same per row against the row's rms (2.5 to 3 times smaller than its largest element): max |err| / rms(ref row)"""
    import numpy as np
    return _row_err(got, ref, lambda r: np.sqrt((r ** 2).mean(axis=-1)))


def rows_kernel(q8, m, n, k):
    """The kernel 2..8 activation rows against an [n, k] weight run on (what aionhip_last_kernel reports): the matrix-pipe GEMV for
    many weight rows and a K of 2048..4096 in whole 256-code stages (q4: from 14336 rows at 5..8 activation rows, from 65536 at
    3..4; q8: from 65536 rows up to 300 M weights), the exact GEMM's 16-row tile for 5..8 rows over a K past 4096, else the
    vector-ALU rows kernel."""
    tag = "q8" if q8 else "q4"
    if 3 <= m <= 8 and 2048 <= k <= 4096 and k % 256 == 0:
        if (not q8 and n >= (14336 if m >= 5 else 65536)) or (q8 and n >= 65536 and n * k <= 300_000_000):
            return "gemv_%s_mfma" % tag
    return ("gemm_i8_" if m >= 5 and k > 4096 else "gemv_") + tag
