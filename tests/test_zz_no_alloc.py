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


_CHILD_FIRST = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1])
from cwick_amd import hip, synth
assert hip.ready(), hip.last_error()
c = synth.cfg3_mla_decode(9000, 128, seed=2104)
rows = torch.from_numpy(c["rows"]).cuda(); scales = torch.from_numpy(c["scales"]).cuda()
q = torch.from_numpy(c["q"].view(np.int16)).cuda()
out = torch.full((128, synth.VDIM), float("nan"), dtype=torch.float32, device="cuda")
out2 = torch.full((128, synth.VDIM), float("nan"), dtype=torch.float32, device="cuda")
ref = torch.empty_like(out)
ref2 = torch.empty_like(out)
s = torch.cuda.Stream()
torch.cuda.synchronize()
free0, _ = torch.cuda.mem_get_info()
# the very first call of this process into the entry point, under capture, no warm-up of any kind
g = torch.cuda.CUDAGraph()
with torch.cuda.graph(g, stream=s):
    rc = hip.mla_decode_static_dev(rows, scales, 0, 0, 9000, 1, None, 9000, q, 128, c["scale"], out, s.cuda_stream, raw=True)
g.replay()
torch.cuda.synchronize()
free1, _ = torch.cuda.mem_get_info()
# a second capture, of a smaller shape, and an eager call: the device's free memory must not move
g2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g2, stream=s):
    rc2 = hip.mla_decode_static_dev(rows, scales, 0, 0, 9000, 1, None, 3000, q, 128, c["scale"], out2, s.cuda_stream, raw=True)
g2.replay()
torch.cuda.synchronize()
free2, _ = torch.cuda.mem_get_info()
rc3 = hip.mla_decode_static_dev(rows, scales, 0, 0, 9000, 1, None, 9000, q, 128, c["scale"], out, None, raw=True)
torch.cuda.synchronize()
free3, _ = torch.cuda.mem_get_info()
hip.mla_decode_dev(rows, scales, 0, 0, 9000, 1, None, 9000, q, 128, c["scale"], ref, None)
hip.mla_decode_dev(rows, scales, 0, 0, 9000, 1, None, 3000, q, 128, c["scale"], ref2, None)
torch.cuda.synchronize()
print("RC", rc, rc2, rc3, "SAME", bool(torch.equal(out.view(torch.int32), ref.view(torch.int32))),
      "SAME2", bool(torch.equal(out2.view(torch.int32), ref2.view(torch.int32))),
      "FREE", free0 - free1, free1 - free2, free2 - free3, "ERR", hip.last_error())
"""


def test_mla_decode_static_first_call_under_capture_allocates_nothing(hip):
    """In a fresh process the first call ever made to the entry point is captured into a graph with no
    warm-up (its one-time set-up -- the kernels' LDS attribute, the address of the scratch symbol --
    runs under the capture) and the replay equals the allocating entry point bit for bit.  The
    runtime loads the device image of the source file that holds the kernels and the 16 MiB area
    at that first launch (once per process: at most 32 MiB go from the device's free memory
    there); from then on -- a second capture of another shape, an eager call -- the free memory
    does not move."""
    import os
    import subprocess
    import sys
    print("[case] mla_decode_static_dev: first call of a process, under capture", flush=True)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", _CHILD_FIRST, root], capture_output=True, text=True, timeout=150)
    assert r.returncode == 0, r.stderr[-3000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("RC ")][0]
    f = line.split()
    assert f[1:4] == ["1", "1", "1"], line
    assert "SAME True SAME2 True" in line, line
    d = [int(x) for x in f[f.index("FREE") + 1:f.index("FREE") + 4]]
    assert 0 <= d[0] <= 32 << 20 and d[1] == 0 and d[2] == 0, line
