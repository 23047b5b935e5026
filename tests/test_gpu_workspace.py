"""The per-stream workspace of the device-pointer entry points: it grows by allocating (never by
freeing or waiting), so kernels and captured graphs that carry an older buffer's address stay
valid; a call that would have to allocate while its stream is being captured declines and leaves
the capture intact; cwick_hip_reserve_dev sizes it up front; cwick_hip_stream_release drops it."""
import numpy as np
import pytest

from cwick_amd import synth

pytestmark = pytest.mark.gpu


def _mla_operands(torch, n_rows, seed):
    c = synth.cfg3_mla_decode(n_rows, 128, seed=seed)
    return (c, torch.from_numpy(c["rows"]).cuda(), torch.from_numpy(c["scales"]).cuda(),
            torch.from_numpy(c["q"].view(np.int16)).cuda())


def test_growth_after_capture_keeps_the_graph_valid(hip):
    import torch
    print("[case] workspace: a graph captured before the workspace grows", flush=True)
    c, rows, scales, q = _mla_operands(torch, 700, 3200)
    out = torch.empty((128, synth.VDIM), dtype=torch.float32, device="cuda")
    s = torch.cuda.Stream()
    sp = s.cuda_stream

    def small(ptr):
        # batch 1, 700 keys: a few slices of partials
        hip.mla_decode_dev(rows, scales, 0, 0, 700, 1, None, 700, q, 128, c["scale"], out, ptr)
    with torch.cuda.stream(s):
        small(sp)
    s.synchronize()
    want = out.clone()
    held = hip.workspace_bytes_dev(sp)
    assert held > 0
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        small(sp)
    # a much larger shape on the same stream: the workspace has to grow
    B = 48
    c2, rows2, scales2, _ = _mla_operands(torch, 4096, 3201)
    q2 = torch.from_numpy(np.repeat(c2["q"][None], B, 0).view(np.int16)).cuda()
    out2 = torch.empty((B, 128, synth.VDIM), dtype=torch.float32, device="cuda")
    with torch.cuda.stream(s):
        hip.mla_decode_dev(rows2, scales2, 0, 0, 4096, B, None, 4096, q2, 128, c2["scale"], out2, sp)
        hip.mla_decode_dev(rows2, scales2, 0, 0, 4096, B, None, 4096, q2, 128, c2["scale"], out2, sp)
    s.synchronize()
    assert hip.workspace_bytes_dev(sp) >= held
    big = out2.clone()
    for rep in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), want.view(torch.int32)), "replay %d after the growth" % rep
        # and the large shape again between the replays (its buffer is the current one)
        with torch.cuda.stream(s):
            hip.mla_decode_dev(rows2, scales2, 0, 0, 4096, B, None, 4096, q2, 128, c2["scale"], out2, sp)
        s.synchronize()
        assert torch.equal(out2.view(torch.int32), big.view(torch.int32))
    del g
    assert hip.stream_release(sp) == 1
    assert hip.workspace_bytes_dev(sp) == 0


def test_capture_declines_instead_of_allocating_and_reserve_prevents_it(hip):
    import torch
    print("[case] workspace: first call of a stream under capture, then with a reservation", flush=True)
    c, rows, scales, q = _mla_operands(torch, 5000, 3202)
    out = torch.empty((128, synth.VDIM), dtype=torch.float32, device="cuda")
    # the kernels' one-time attributes are set by an eager call on another stream
    hip.mla_decode_dev(rows, scales, 0, 0, 5000, 1, None, 5000, q, 128, c["scale"], out, None)
    torch.cuda.synchronize()
    want = out.clone()
    s = torch.cuda.Stream()
    sp = s.cuda_stream
    assert hip.workspace_bytes_dev(sp) == 0
    marker = torch.zeros(4, device="cuda")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        marker.add_(1.0)                                  # the capture holds something of its own
        rc = hip.mla_decode_dev(rows, scales, 0, 0, 5000, 1, None, 5000, q, 128, c["scale"], out, sp, raw=True)
        why = hip.last_error()
    assert rc == 0 and "captured" in why, why
    assert hip.workspace_bytes_dev(sp) == 0
    g.replay()                                            # the capture survived the declined call
    torch.cuda.synchronize()
    assert float(marker[0]) == 1.0
    # with a reservation the same first call is captured and replays to the eager result
    assert hip.reserve_dev(sp, 32 << 20) == 1
    assert hip.workspace_bytes_dev(sp) >= 32 << 20
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=s):
        hip.mla_decode_dev(rows, scales, 0, 0, 5000, 1, None, 5000, q, 128, c["scale"], out, sp)
    for rep in range(2):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), want.view(torch.int32)), "replay %d" % rep
    del g, g2
    assert hip.stream_release(sp) == 1
