"""cwick_hip_mla_decode_static_dev: the MLA decode entry point that allocates nothing (its
split-K partials live in a fixed area inside the library) against cwick_hip_mla_decode_dev on
the same operands: same kernels, same split, so the outputs must be bit-identical; both are
also checked against the oracle.  Two calls in a row, the second with a smaller input (the
area keeps the first call's partials: nothing of them may show)."""
import numpy as np
import pytest

from cwick_amd import synth
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu


def _run(hip, torch, fn, c, n_list, sel=None):
    rows = torch.from_numpy(c["rows"]).cuda()
    scales = torch.from_numpy(c["scales"]).cuda()
    q = torch.from_numpy(c["q"].view(np.int16)).cuda()
    out = torch.full((c["nh"], synth.VDIM), float("nan"), dtype=torch.float32, device="cuda")
    dsel = torch.from_numpy(sel).cuda() if sel is not None else None
    s = torch.cuda.current_stream().cuda_stream
    fn(rows, scales, 0, 0, c["n_keys"], 1, dsel, n_list, q, c["nh"], c["scale"], out, s)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_mla_decode_static_matches_the_allocating_entry_point(hip, orc):
    import torch
    print("[case] mla_decode_static_dev: 32768 keys, then 5000 keys through a list", flush=True)
    big = synth.cfg3_mla_decode(32768, 128, seed=2100)
    small = synth.cfg3_mla_decode(5000, 96, seed=2101)
    sel = np.sort(synth.rng(2102).permutation(5000)[:1500]).astype(np.int32)
    sel[::50] = -1
    for c, n_list, s in ((big, 32768, None), (small, 1500, sel)):
        got = _run(hip, torch, hip.mla_decode_static_dev, c, n_list, s)
        want = _run(hip, torch, hip.mla_decode_dev, c, n_list, s)
        assert np.isfinite(got).all()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
            "static-scratch entry point differs from cwick_hip_mla_decode_dev (max-abs %.3e)" % np.abs(got - want).max()
        ref = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=s, nlist=n_list, nthreads=0)
        assert_close(got, ref, "mla_decode_static_dev %d keys" % c["n_keys"])


_CHILD = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1])
from cwick_amd import hip, synth
assert hip.ready(), hip.last_error()
c = synth.cfg3_mla_decode(20000, 128, seed=2103)
rows = torch.from_numpy(c["rows"]).cuda(); scales = torch.from_numpy(c["scales"]).cuda()
q = torch.from_numpy(c["q"].view(np.int16)).cuda()
out = torch.full((128, synth.VDIM), 7.0, dtype=torch.float32, device="cuda")
s = torch.cuda.current_stream().cuda_stream
rc = hip.mla_decode_static_dev(rows, scales, 0, 0, 20000, 1, None, 20000, q, 128, c["scale"], out, s, raw=True)
torch.cuda.synchronize()
print("RC", rc, "UNTOUCHED", bool((out == 7.0).all()), "ERR", hip.last_error())
"""


def test_mla_decode_static_declines_what_does_not_fit(hip):
    """With four workgroups per compute unit (CWICK_HIP_MLA_WG_PER_CU=4, read once per process,
    hence the child process) the partials of a 20000-key decode take 35 MB: more than the fixed
    area.  The call is refused with a reason and the output is untouched."""
    import os
    import subprocess
    import sys
    print("[case] mla_decode_static_dev declines", flush=True)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, CWICK_HIP_MLA_WG_PER_CU="4")
    r = subprocess.run([sys.executable, "-c", _CHILD, root], env=env, capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("RC ")][0]
    assert line.startswith("RC 0 UNTOUCHED True") and "static scratch" in line, line
