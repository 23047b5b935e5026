"""GPU parity on shapes drawn at random: lengths that end anywhere inside a tile, a workgroup's
share or a selection round, head counts and batch sizes in every supported combination.  The
fixed cases of test_gpu_parity.py name the borders the kernels are known to have; these draw
around them.  Each draw prints its shape before it runs, so a failure names its case."""
import numpy as np
import pytest

from cwick_amd import synth
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _seed(g):
    return int(g.integers(1, 1 << 30))


@pytest.mark.parametrize("seed", [101, 102])
def test_topk_random_rows(hip, orc, seed):
    """Row lengths across the one-workgroup, many-workgroup and long-row kernels; scores that
    are distinct, heavily tied, mostly -inf, or all in the denormal range."""
    g = np.random.default_rng(seed)
    for _ in range(20):
        n = int(g.choice([g.integers(1, 3000), g.integers(3000, 20000), g.integers(16384, 131073),
                          g.integers(131073, 400000)]))
        k = int(min(n, g.choice([1, 7, 64, 512, 2048, g.integers(1, 4097)])))
        kind = str(g.choice(["normal", "ties", "inf", "small"]))
        if kind == "normal":
            sc = g.standard_normal(n, dtype=np.float32)
        elif kind == "ties":
            sc = g.integers(-6, 6, n).astype(np.float32) * np.float32(0.5)
        elif kind == "small":
            sc = (g.standard_normal(n) * 1e-30).astype(np.float32)
        else:
            sc = g.standard_normal(n, dtype=np.float32)
            sc[g.random(n) < 0.8] = -np.inf
        say("[case] topk random", n, k, kind)
        assert np.array_equal(hip.topk(sc, k), orc.topk_contract(sc, k)), (n, k, kind)


@pytest.mark.parametrize("seed", [201, 202])
def test_dsa_decode_random_shapes(hip, orc, seed):
    """Indexer, selection and sparse attention in one call: the selected rows bit-exact, the
    output within the attention tolerance, for random key counts, k, batch and head counts."""
    g = np.random.default_rng(seed)
    for _ in range(6):
        topk = int(g.choice([64, 128, 512, 1024, 2048]))
        n_keys = int(g.integers(topk + 1, 70000))
        batch = int(g.integers(1, 9))
        ih = int(g.choice([16, 32, 64]))
        nh = int(g.choice([16, 64, 128]))
        say("[case] dsa random", n_keys, topk, batch, ih, nh)
        c = synth.cfg5_dsa(n_keys=n_keys, batch=batch, ih=ih, topk=topk, nh=nh, seed=_seed(g))
        ik = hip.IndexKeys(batch, n_keys)
        lat = hip.LatentCache(batch, n_keys)
        for b in range(batch):
            ik.write(b, 0, c["ikeys"][b], c["ikscale"][b])
            lat.write(b, 0, c["rows"][b], c["scales"][b])
        out, sel = hip.dsa_decode(ik, lat, 0, 1, n_keys, c["q_idx"], c["w"], topk, c["q"], c["scale"])
        for b in range(batch):
            sc = orc.indexer_scores(c["q_idx"][b], c["w"][b], c["ikeys"][b], c["ikscale"][b], nthreads=0)
            rsel = orc.topk_contract(sc, topk)
            assert np.array_equal(sel[b], rsel), "query %d: selected rows differ" % b
            ref = orc.mla_decode(c["q"][b], c["rows"][b], c["scales"][b], c["scale"], sel=rsel, nthreads=0)
            assert_close(out[b], ref, "dsa random query %d" % b)
        ik.free()
        lat.free()


@pytest.mark.parametrize("seed", [301])
def test_decode_random_lengths(hip, orc, seed):
    g = np.random.default_rng(seed)
    for _ in range(8):
        n_keys = int(g.choice([g.integers(256, 4000), g.integers(4000, 40000)]))
        nh = int(g.choice([16, 40, 64, 96, 128]))
        say("[case] mla decode random", n_keys, nh)
        c = synth.cfg3_mla_decode(n_keys, nh, seed=_seed(g))
        cache = hip.LatentCache(1, n_keys)
        cache.write(0, 0, c["rows"], c["scales"])
        got = hip.mla_decode(cache, 0, c["q"], c["scale"], n_list=n_keys)
        ref = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=0)
        assert_close(got, ref, "mla decode %d keys %d heads" % (n_keys, nh))
        cache.free()
    for _ in range(8):
        n_keys = int(g.integers(200, 9000))
        nh, nkv, hd = [(16, 4, 256), (8, 8, 128), (32, 4, 128), (64, 8, 128)][int(g.integers(0, 4))]
        say("[case] gqa decode random", n_keys, nh, nkv, hd)
        c = synth.cfg1_gqa_decode(n_keys, nh, nkv, hd, seed=_seed(g))
        cache = hip.KVCache(n_keys, nkv, hd)
        cache.write(0, c["k"], c["v"])
        got = hip.gqa_decode(cache, n_keys, c["q"], c["scale"])
        ref = orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"], nthreads=0)
        assert_close(got, ref, "gqa decode %d keys %d/%d x %d" % (n_keys, nh, nkv, hd))
        cache.free()


@pytest.mark.parametrize("seed", [401])
def test_prefill_random_chunks(hip, orc, seed):
    g = np.random.default_rng(seed)
    for _ in range(6):
        pos0 = int(g.choice([0, g.integers(0, 900), g.integers(900, 3000)]))
        n = int(g.integers(1, 260))
        nh, nkv = [(16, 4), (8, 8), (16, 2), (4, 2)][int(g.integers(0, 4))]
        say("[case] gqa prefill random", pos0, n, nh, nkv)
        c = synth.cfg2_gqa_prefill(n, nh, nkv, 256, pos0, seed=_seed(g))
        cache = hip.KVCache(pos0 + n, nkv, 256)
        cache.write(0, c["k"].reshape(pos0 + n, -1), c["v"].reshape(pos0 + n, -1))
        got = hip.gqa_prefill(cache, pos0, c["q"], c["scale"])
        ref = orc.gqa_prefill(c["q"], c["k"], c["v"], pos0, c["scale"], nthreads=0)
        # the first rows of a chunk at position 0 attend to a handful of keys: outputs of O(1)
        assert_close(got, ref, "gqa prefill pos0 %d n %d %d/%d" % (pos0, n, nh, nkv), strict=pos0 >= 200)
        cache.free()
    for _ in range(6):
        pos0 = int(g.choice([g.integers(200, 900), g.integers(900, 6000)]))
        n = int(g.integers(1, 200))
        nh = int(g.choice([16, 64, 96, 128]))
        say("[case] mla prefill random", pos0, n, nh)
        c = synth.cfg4_mla_prefill(n, pos0, nh, seed=_seed(g))
        cache = hip.LatentCache(1, pos0 + n)
        cache.write(0, 0, c["rows"], c["scales"])
        got = hip.mla_prefill_chunk(cache, 0, pos0, c["q"], c["scale"])
        ref = orc.mla_prefill_chunk(c["q"], c["rows"], c["scales"], pos0, c["scale"], nthreads=0)
        assert_close(got, ref, "mla prefill pos0 %d n %d heads %d" % (pos0, n, nh))
        cache.free()


@pytest.mark.parametrize("seed", [501])
def test_mm_select_random_shapes(hip, orc, seed):
    """The block selection of the block-sparse decode on random limits, chunk lengths, block
    sizes (whole scoring groups and not), head counts and list caps: scores bit for bit, blocks
    and positions equal to the oracle's."""
    import torch
    g = np.random.default_rng(seed)
    s = torch.cuda.current_stream().cuda_stream
    for _ in range(24):
        bs = int(g.choice([64, 128, 192, 256, 7, 100, 33]))
        limit0 = int(g.choice([g.integers(1, 300), g.integers(300, 9000), g.integers(9000, 80000)]))
        batch = int(g.choice([1, 1, 2, 5]))
        ih = int(g.integers(1, 9))
        idim = int(g.choice([8, 64, 128, 256]))
        keep = int(g.choice([1, 3, 16, 40]))
        max_sel = int(g.choice([4096, 500, (keep + 1) * bs]))
        say("[case] mm select random", limit0, batch, ih, idim, bs, keep, max_sel)
        n = limit0 + batch - 1
        keys = synth.normal_bf16(g, (n, idim))
        iq = g.standard_normal((batch, ih, idim)).astype(np.float32)
        d_keys = torch.from_numpy(keys.view(np.int16)).cuda()
        d_iq = torch.from_numpy(iq).cuda()
        d_sc = torch.empty((batch, n), dtype=torch.float32, device="cuda")
        d_blk = torch.empty((batch, keep + 1), dtype=torch.int32, device="cuda")
        d_sel = torch.empty((batch, max_sel), dtype=torch.int32, device="cuda")
        d_ns = torch.empty((batch,), dtype=torch.int32, device="cuda")
        hip.mm_select_dev(d_keys, d_iq, batch, limit0, ih, idim, bs, keep, d_sc, n, d_blk, d_sel, max_sel, d_ns, s)
        torch.cuda.synchronize()
        sc, blk, sel, ns = d_sc.cpu().numpy(), d_blk.cpu().numpy(), d_sel.cpu().numpy(), d_ns.cpu().numpy()
        for t in range(batch):
            limit = limit0 + t
            ref_sc = orc.mm_index_scores(iq[t], keys, limit)
            assert np.array_equal(sc[t, :limit].view(np.uint32), ref_sc.view(np.uint32)), "query %d: scores" % t
            rblk, rpos = orc.mm_select_blocks(ref_sc, limit, bs, keep, max_sel)
            assert list(blk[t, :rblk.size]) == list(rblk) and (blk[t, rblk.size:] == -1).all(), "query %d: blocks" % t
            assert ns[t] == rpos.size and list(sel[t, :rpos.size]) == list(rpos) and (sel[t, rpos.size:] == -1).all(), \
                "query %d: positions" % t

