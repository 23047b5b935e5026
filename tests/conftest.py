import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    from oracle import orc as _orc
    _orc.lib()
    return _orc


@pytest.fixture(scope="session")
def hip():
    """The C-ABI library on a live device.  No fallback: a missing library or a
    device that does not come up fails the GPU tests."""
    from cwick_amd import hip as _hip
    _hip.lib()
    assert _hip.ready(), "libcwick_hip.so could not bring the GPU up: " + _hip.last_error()
    print("\n[device]", _hip.device_info(), flush=True)
    return _hip


# Tolerance of the attention outputs against the CPU oracle: max-abs 2e-3 and
# max-abs / max|reference| 1e-2 (the form the reference's own self-check prints,
# src/attention.c:881-891).
ATOL, RTOL = 2e-3, 1e-2


def assert_close(got, ref, what=""):
    import numpy as np
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), what + ": non-finite output"
    diff = np.abs(got - ref).max()
    refmax = np.abs(ref).max()
    rel = diff / refmax if refmax > 0 else diff
    print("[parity] %-40s maxabs %.3e  rel %.3e  refmax %.3e" % (what, diff, rel, refmax),
          flush=True)
    assert diff <= ATOL, "%s: max-abs %.3e > %.1e" % (what, diff, ATOL)
    assert rel <= RTOL, "%s: rel %.3e > %.1e" % (what, rel, RTOL)
