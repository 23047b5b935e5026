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
    # Some tests hold operands in torch tensors.  torch brings its own copy of the HIP runtime;
    # loaded after the library's it finds no GPU, loaded first the library shares it (the order
    # bench.py uses).
    import torch  # noqa: F401
    from cwick_amd import hip as _hip
    _hip.lib()
    assert _hip.ready(), "libcwick_hip.so could not bring the GPU up: " + _hip.last_error()
    print("\n[device]", _hip.device_info(), flush=True)
    return _hip


# Tolerance of the attention outputs against the CPU oracle: max-abs 2e-3 and
# max-abs / max|reference| 1e-2 (the form the reference's own self-check prints,
# src/attention.c:881-891).
#
# strict=True (the five benchmark configurations and everything shaped like them):
#     max|got-ref| <= 2e-3  AND  max|got-ref| / max|ref| <= 1e-2.
# strict=False (edge cases whose outputs are O(1), e.g. a single key, where the
# output IS a latent value and a bf16-rounded weight alone moves it by 2^-9 of
# itself): the elementwise form |got-ref| <= 2e-3 + 1e-2*|ref|.
ATOL, RTOL = 2e-3, 1e-2


def assert_close(got, ref, what="", strict=True):
    import numpy as np
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), what + ": non-finite output"
    err = np.abs(got - ref)
    diff = err.max()
    refmax = np.abs(ref).max()
    rel = diff / refmax if refmax > 0 else diff
    print("[parity] %-44s maxabs %.3e  rel %.3e  refmax %.3e%s" %
          (what, diff, rel, refmax, "" if strict else "  (elementwise)"), flush=True)
    if strict:
        assert diff <= ATOL, "%s: max-abs %.3e > %.1e" % (what, diff, ATOL)
        assert rel <= RTOL, "%s: rel %.3e > %.1e" % (what, rel, RTOL)
    else:
        bad = err > ATOL + RTOL * np.abs(ref)
        assert not bad.any(), "%s: %d elements outside 2e-3 + 1e-2*|ref| (max-abs %.3e)" % (
            what, int(bad.sum()), diff)
