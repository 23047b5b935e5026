"""The device-pointer entry points under HIP graph capture.  They only enqueue kernels (no
memset nodes, no copies), take their scratch from a per-stream workspace that a warm-up call has
already sized, or -- cwick_hip_mla_decode_static_dev -- from a fixed area inside the library.
Each case is captured once on a side stream and replayed several times with the operands changed
in place and eager work and synchronisations between the replays; every replay must equal the
eager call on the same operands bit for bit (the same kernels run either way)."""
import numpy as np
import pytest

from cwick_amd import synth

pytestmark = pytest.mark.gpu


def _replay_equals_eager(torch, call, mutable, out, stream, what):
    """call(stream_ptr) enqueues the op; `mutable` is an operand changed between replays."""
    with torch.cuda.stream(stream):
        call(stream.cuda_stream)                       # warm-up: workspaces, attributes, counters
    stream.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        call(stream.cuda_stream)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    for rep in range(3):
        # new operand values (same bit patterns permuted: every value stays a valid bf16 / list entry)
        perm = torch.randperm(mutable.shape[0], device="cuda", generator=gen)
        mutable.copy_(mutable[perm].clone())
        torch.cuda.synchronize()
        out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        got = out.clone()
        out.fill_(float("nan"))
        with torch.cuda.stream(stream):
            call(stream.cuda_stream)
        stream.synchronize()
        assert torch.isfinite(got).all(), "%s: replay %d left the output unwritten" % (what, rep)
        assert torch.equal(got.view(torch.int32), out.view(torch.int32)), "%s: replay %d differs from the eager call" % (what, rep)


def test_mla_decode_entries_under_graph_capture(hip):
    import torch
    print("[case] graph capture: mla_decode_static_dev, mla_decode_dev", flush=True)
    c = synth.cfg3_mla_decode(6000, 128, seed=3100)
    rows = torch.from_numpy(c["rows"]).cuda()
    scales = torch.from_numpy(c["scales"]).cuda()
    q = torch.from_numpy(c["q"].view(np.int16)).cuda()               # [128][576]: heads are permuted between replays
    out = torch.empty((128, synth.VDIM), dtype=torch.float32, device="cuda")
    s = torch.cuda.Stream()
    for name, fn in (("mla_decode_static_dev", hip.mla_decode_static_dev), ("mla_decode_dev", hip.mla_decode_dev)):
        _replay_equals_eager(torch, lambda sp: fn(rows, scales, 0, 0, 6000, 1, None, 6000, q, 128, c["scale"], out, sp),
                             q, out, s, name)


def test_gqa_and_prefill_entries_under_graph_capture(hip):
    import torch
    print("[case] graph capture: gqa_prefill_dev (ticket counters), gqa_decode_dev, mla_prefill_chunk_dev", flush=True)
    c = synth.cfg2_gqa_prefill(700, 16, 4, 256, 0, seed=3101)
    d = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    k, v, q = d(c["k"]), d(c["v"]), d(c["q"])                        # q [700][16][256]: positions are permuted
    out = torch.empty((700, 16, 256), dtype=torch.float32, device="cuda")
    s = torch.cuda.Stream()
    _replay_equals_eager(torch, lambda sp: hip.gqa_prefill_dev(k, v, 0, 700, 4, 256, q, 16, c["scale"], out, sp),
                         q, out, s, "gqa_prefill_dev")
    q1 = q[699].clone()                                              # [16][256]: heads are permuted
    out1 = torch.empty((16, 256), dtype=torch.float32, device="cuda")
    _replay_equals_eager(torch, lambda sp: hip.gqa_decode_dev(k, v, 700, 4, 256, q1, 16, c["scale"], out1, sp),
                         q1, out1, s, "gqa_decode_dev")
    m = synth.cfg4_mla_prefill(9, 500, 128, seed=3102)
    rows = torch.from_numpy(m["rows"]).cuda()
    scales = torch.from_numpy(m["scales"]).cuda()
    mq = torch.from_numpy(m["q"].view(np.int16)).cuda()              # [9][128][576]: queries are permuted
    mout = torch.empty((9, 128, synth.VDIM), dtype=torch.float32, device="cuda")
    _replay_equals_eager(torch, lambda sp: hip.mla_prefill_chunk_dev(rows, scales, 500, 9, mq, 128, m["scale"], mout, sp),
                         mq, mout, s, "mla_prefill_chunk_dev")


def test_dsa_decode_under_graph_capture(hip):
    import torch
    print("[case] graph capture: dsa_decode_dev (fused select + sparse MLA)", flush=True)
    B, N, K = 2, 20000, 1024
    c = synth.cfg5_dsa(n_keys=N, batch=B, ih=64, topk=K, nh=128, shared=True, seed=3103)
    d8 = lambda a: torch.from_numpy(a).cuda()
    ik, iks = d8(c["ikeys"][0]), d8(c["ikscale"][0])
    rows, scales = d8(c["rows"][0]), d8(c["scales"][0])
    qi = torch.from_numpy(c["q_idx"].view(np.int16)).cuda()          # [B][64][128]: the two queries swap
    w = d8(c["w"])
    q = torch.from_numpy(c["q"].view(np.int16)).cuda()
    out = torch.empty((B, 128, synth.VDIM), dtype=torch.float32, device="cuda")
    sel = torch.empty((B, K), dtype=torch.int32, device="cuda")
    tmp = torch.empty((B, N), dtype=torch.float32, device="cuda")
    s = torch.cuda.Stream()

    def call(sp):
        hip.dsa_decode_dev(ik, iks, 0, 0, rows, scales, 0, 0, B, N, qi, w, 64, K, q, 128, c["scale"], tmp, sel, out, sp)
    _replay_equals_eager(torch, call, qi, out, s, "dsa_decode_dev")


def test_block_sparse_decode_under_graph_capture(hip):
    import torch
    print("[case] graph capture: mm_select_dev -> gqa_decode_sel_dev", flush=True)
    n, nh, nkv, hd, ih, idim, bs, keep = 5000, 64, 4, 128, 4, 128, 128, 16
    g = synth.rng(3104)
    c = synth.cfg1_gqa_decode(n, nh, nkv, hd, seed=3105)
    d = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    k, v, q = d(c["k"]), d(c["v"]), d(c["q"])
    keys = d(synth.normal_bf16(g, (n, idim)))
    iq = torch.from_numpy(g.standard_normal((ih * idim // 8, 8)).astype(np.float32)).cuda()   # pieces of eight dims are permuted
    max_sel = (keep + 1) * bs
    sc = torch.empty((1, n), dtype=torch.float32, device="cuda")
    sel = torch.empty((1, max_sel), dtype=torch.int32, device="cuda")
    out = torch.empty((nh, hd), dtype=torch.float32, device="cuda")
    s = torch.cuda.Stream()

    def call(sp):
        hip.mm_select_dev(keys, iq, 1, n, ih, idim, bs, keep, sc, n, None, sel, max_sel, None, sp)
        hip.gqa_decode_sel_dev(k, v, n, nkv, hd, sel, max_sel, q, nh, c["scale"], out, sp)
    _replay_equals_eager(torch, call, iq, out, s, "mm_select_dev -> gqa_decode_sel_dev")
