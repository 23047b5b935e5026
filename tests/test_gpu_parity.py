"""GPU parity: libcwick_hip.so through its C ABI against the CPU oracle on the
same seeded inputs.  Bit-exact for codecs, indexer scores and top-k indices;
max-abs 2e-3 / rel 1e-2 for attention outputs (bf16/fp8 in, fp32 accumulate)."""
import numpy as np
import pytest

from cwick_amd import synth
from tests.conftest import assert_close

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ codecs
def test_lane_exchange_primitives(hip):
    """Sums, maxima and prefix sums over a wave (DPP inside a row of sixteen lanes, lane swaps
    across rows) against numpy, bit for bit: every kernel's reductions are built on them."""
    say("[case] lane exchange primitives")
    g = synth.rng(4242)
    for rep in range(8):
        w = g.integers(0, 1 << 32 if rep % 2 else 100000, size=64, dtype=np.uint64).astype(np.uint32)
        if rep == 7:
            w[:] = 0
            w[37] = 0xFFFFFFFF
        got = hip.lane_ops(w)
        f = ((w & 0x007FFFFF) | 0x3F800000).view(np.float32)
        assert np.all(got[0] == np.uint32(w.astype(np.uint64).sum() & 0xFFFFFFFF))
        assert np.all(got[1] == w.max()) and np.all(got[2] == w.min())
        assert np.array_equal(got[3], (np.cumsum(w.astype(np.uint64)) & 0xFFFFFFFF).astype(np.uint32))
        assert np.all(got[4].view(np.float32) == f.max())
        l = np.arange(64)
        assert np.array_equal(got[5].view(np.float32), np.maximum(f, f[l ^ 16]))
        assert np.array_equal(got[6].view(np.float32), np.maximum(f, f[l ^ 32]))
        # a + b in fp32 is the same whichever side a lane stands on
        assert np.array_equal(got[7].view(np.float32), f + f[l ^ 16])
        assert np.array_equal(got[8].view(np.float32), f + f[l ^ 32])
        s2 = f + f[l ^ 1]
        s4 = s2 + s2[l ^ 2]
        s8 = s4 + s4[l ^ 4]
        s16 = s8 + s8[l ^ 8]
        for row, want in ((9, s2), (10, s4), (11, s8), (12, s16)):
            assert np.array_equal(got[row].view(np.float32), want), "group sum %d" % row


def test_e4m3_hardware_decode_matches_table(hip, orc):
    say("[case] e4m3 table")
    got = hip.e4m3_table()
    ref = orc.e4m3_lut()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(got[ok].view(np.uint32), ref[ok].view(np.uint32))


def test_latent_quantise_on_append_bit_exact(hip, orc):
    say("[case] latent write_f32")
    g = synth.rng(11)
    x = g.standard_normal((300, synth.KDIM), dtype=np.float32)
    x[5] = 0.0
    x[6, :128] = 0.0
    x[7] *= 1e-6
    x[8] *= 1e4
    c = hip.LatentCache(2, 512)
    c.write_f32(1, 100, x)
    rows, scales = c.read(1, 100, 300)
    rq, rs = orc.quantize_rows_e4m3(x, 128)
    assert np.array_equal(scales.view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(rows, rq)
    nq, ns = synth.quantize_rows(x, 128)
    assert np.array_equal(nq, rq) and np.array_equal(ns.view(np.uint32), rs.view(np.uint32))
    c.free()


# ------------------------------------------------------------------ GQA decode
@pytest.mark.parametrize("n_keys,nh,nkv,hd", [
    (4096, 16, 4, 256),      # BASELINE config 1
    (1, 16, 4, 256),
    (63, 16, 4, 256),
    (1000, 8, 8, 128),
    (777, 32, 4, 128),
    (513, 8, 4, 256),
])
def test_gqa_decode(hip, orc, n_keys, nh, nkv, hd):
    say("[case] gqa_decode", n_keys, nh, nkv, hd)
    c = synth.cfg1_gqa_decode(n_keys, nh, nkv, hd, seed=100 + n_keys)
    cache = hip.KVCache(n_keys + 7, nkv, hd)
    cache.write(0, c["k"].reshape(n_keys, -1), c["v"].reshape(n_keys, -1))
    got = hip.gqa_decode(cache, n_keys, c["q"], c["scale"])
    ref = orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"])
    assert_close(got, ref, "gqa_decode %d keys %d/%d/%d" % (n_keys, nh, nkv, hd))
    cache.free()


# ------------------------------------------------------------------ GQA prefill
@pytest.mark.parametrize("pos0,n,nh,nkv", [
    (0, 300, 16, 4),         # BASELINE config 2 geometry, reduced length
    (0, 1, 16, 4),
    (100, 77, 16, 4),        # chunk appended to a prefix, ragged length
    (0, 130, 8, 8),          # group 1
    (5, 200, 16, 2),         # group 8
    (0, 64, 4, 2),           # group 2
    # beyond 1024 keys the kernel leaves its two-term-weight variant for the pipelined one:
    (2100, 150, 16, 4),      # every position block on the long-prefix path, ragged tiles
    (0, 2300, 8, 2),         # one launch that crosses the boundary between the two variants
    (1990, 200, 4, 4),       # group 1
    (1000, 100, 8, 4),       # the boundary between the variants inside a chunk
    (3000, 40, 16, 2),       # group 8, a chunk shorter than one position block
    (1500, 260, 4, 2),       # group 2, two position blocks and a ragged third
])
def test_gqa_prefill(hip, orc, pos0, n, nh, nkv):
    say("[case] gqa_prefill", pos0, n, nh, nkv)
    c = synth.cfg2_gqa_prefill(n, nh, nkv, 256, pos0, seed=200 + n)
    cache = hip.KVCache(pos0 + n, nkv, 256)
    cache.write(0, c["k"].reshape(pos0 + n, -1), c["v"].reshape(pos0 + n, -1))
    got = hip.gqa_prefill(cache, pos0, c["q"], c["scale"])
    ref = orc.gqa_prefill(c["q"], c["k"], c["v"], pos0, c["scale"], nthreads=0)
    assert_close(got, ref, "gqa_prefill pos0 %d n %d %d/%d" % (pos0, n, nh, nkv))
    # row t of a prefill is the decode at position pos0+t
    t = n - 1
    dec = hip.gqa_decode(cache, pos0 + t + 1, c["q"][t], c["scale"])
    assert_close(got[t], dec, "gqa_prefill last row vs decode kernel")
    cache.free()


@pytest.mark.parametrize("pos0,n,start,slope", [
    (0, 300, 0, 0.5),        # short prefix: the two-term-weight variant
    # long prefix: the pipelined variant leaves its fast loop after a few steps / after many.
    # The slope is smaller there so that the raw scores stay below 2e4 as in the first case:
    # fp32 dot products of 1e5 differ by 1e-3 in the exponent between summation orders.
    (2100, 150, 0, 0.05),
    (2100, 150, 1100, 0.1),
])
def test_gqa_prefill_growing_scores(hip, orc, pos0, n, start, slope):
    """Scores that climb by far more than 2^64 along the keys: the rows must leave the fixed
    softmax reference of their first tile and follow the maximum (rescaling path)."""
    say("[case] gqa_prefill growing scores", pos0, n, start, slope)
    nh, nkv = 16, 4
    nk = pos0 + n
    c = synth.cfg2_gqa_prefill(n, nh, nkv, 256, pos0, seed=777)
    k = synth.bf16_to_f32(c["k"]).reshape(nk, nkv, 256)
    q = synth.bf16_to_f32(c["q"]).reshape(n, nh, 256)
    # a common direction whose weight grows with the key index: q.k gains 8 * slope per key
    k[:, :, 0] = np.maximum(np.arange(nk, dtype=np.float32) - start, 0.0)[:, None] * slope
    q[:, :, 0] = 8.0 * 16.0                                   # times scale 1/16 -> 8 * slope * i
    ck = synth.f32_to_bf16(k.reshape(nk, -1)); cq = synth.f32_to_bf16(q.reshape(n, nh, 256))
    cv = c["v"]
    if pos0 + n > 1024:
        # Beyond 1024 keys the weights are single bf16 terms: a softmax that a handful of keys
        # share, as here, is off by 2^-9 of the spread of their values.  Values within +-1.2
        # keep that inside the tolerance; the case is about the moving reference.
        cv = synth.f32_to_bf16(synth.bf16_to_f32(cv) * 0.25)
    cache = hip.KVCache(nk, nkv, 256)
    cache.write(0, ck, cv.reshape(nk, -1))
    got = hip.gqa_prefill(cache, pos0, cq, c["scale"])
    ref = orc.gqa_prefill(cq, ck.reshape(nk, nkv, 256), cv, pos0, c["scale"], nthreads=0)
    assert np.isfinite(got).all()
    assert_close(got, ref, "gqa_prefill growing scores", strict=False)
    cache.free()


def test_gqa_prefill_declines_unsupported(hip):
    say("[case] gqa_prefill declines")
    cache = hip.KVCache(64, 4, 128)                       # head_dim 128: decode only
    q = np.zeros((8, 16, 128), np.uint16)
    rc, out = hip.gqa_prefill(cache, 0, q, 0.1, raw=True)
    assert rc == 0 and "head_dim" in hip.last_error()
    cache.free()
    cache = hip.KVCache(64, 4, 256)
    q = np.zeros((8, 12, 256), np.uint16)                 # group 3
    rc, out = hip.gqa_prefill(cache, 0, q, 0.1, raw=True)
    assert rc == 0 and "group" in hip.last_error()
    rc, out = hip.gqa_prefill(cache, 60, q[:, :4], 0.1, raw=True)   # past the capacity
    assert rc == 0 and "capacity" in hip.last_error()
    cache.free()


# ------------------------------------------------------------------ MLA decode
@pytest.mark.parametrize("n_keys,nh", [
    (32768, 128),            # BASELINE config 3
    (1, 128),
    (65, 128),
    (2051, 64),              # the reference's released geometry (src/attention.c:341-343)
    (700, 16),
    (300, 40),
])
def test_mla_decode_dense(hip, orc, n_keys, nh):
    say("[case] mla_decode dense", n_keys, nh)
    c = synth.cfg3_mla_decode(n_keys, nh, seed=300 + n_keys)
    cache = hip.LatentCache(1, n_keys)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_decode(cache, 0, c["q"], c["scale"], n_list=n_keys)
    ref = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=0)
    # with a handful of keys the output IS (nearly) a latent value of magnitude O(1)
    assert_close(got, ref, "mla_decode dense %d keys %d heads" % (n_keys, nh), strict=n_keys >= 256)
    cache.free()


@pytest.mark.parametrize("n_keys,gain", [(4096, 32.0), (32768, 32.0), (3000, 8.0)])
def test_mla_decode_large_values(hip, orc, n_keys, gain):
    """Latent values `gain` times larger with the query's latent part as much smaller: the same
    scores, outputs `gain` times larger.  The split partials cross HBM as 16-bit fixed point with
    one scale per head and 128 dims, good to 2^-16 of the largest of those outputs, so the
    elementwise tolerance holds while that largest output stays below about a hundred.  The
    second value block is made another 16 times smaller: small outputs next to no large one."""
    say("[case] mla_decode large values", n_keys, gain)
    c = synth.cfg3_mla_decode(n_keys, 128, seed=900 + n_keys)
    scales = c["scales"].copy()
    scales[:, :4] *= np.float32(gain)
    scales[:, 1] *= np.float32(1.0 / 16.0)
    qf = synth.bf16_to_f32(c["q"]).copy()
    qf[:, :512] *= np.float32(1.0 / gain)                  # powers of two: exact in bf16
    qf[:, 128:256] *= np.float32(16.0)
    q = synth.f32_to_bf16(qf)
    cache = hip.LatentCache(1, n_keys)
    cache.write(0, 0, c["rows"], scales)
    got = hip.mla_decode(cache, 0, q, c["scale"], n_list=n_keys)
    ref = orc.mla_decode(q, c["rows"], scales, c["scale"], nthreads=0)
    assert np.abs(ref).max() < 100.0
    assert_close(got, ref, "mla_decode values x%g, %d keys" % (gain, n_keys), strict=False)
    blk = np.abs(got[:, 128:256] - ref[:, 128:256]).max()
    say("[parity] small block: max-abs %.3e of max |ref| %.3e" % (blk, np.abs(ref[:, 128:256]).max()))
    cache.free()


def test_mla_decode_sel(hip, orc):
    say("[case] mla_decode sel")
    n_rows, nh = 5000, 128
    c = synth.cfg3_mla_decode(n_rows, nh, seed=77)
    g = synth.rng(78)
    sel = g.permutation(n_rows)[:2048].astype(np.int32)     # any order, as the selector emits
    sel[[3, 500, 2047]] = -1                                 # -1 padding is skipped
    cache = hip.LatentCache(2, n_rows)
    cache.write(1, 0, c["rows"], c["scales"])
    got = hip.mla_decode(cache, 1, c["q"], c["scale"], sel=sel)
    ref = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=sel, nthreads=0)
    assert_close(got, ref, "mla_decode sel 2048 of 5000")
    # order of the list does not matter beyond rounding
    got2 = hip.mla_decode(cache, 1, c["q"], c["scale"], sel=np.sort(sel))
    assert_close(got2, ref, "mla_decode sel sorted")
    # a list entry outside the cache is refused on the host, outputs untouched
    bad = sel.copy()
    bad[0] = n_rows
    rc, _ = hip.mla_decode(cache, 1, c["q"], c["scale"], sel=bad, raw=True)
    assert rc == 0 and "outside" in hip.last_error()
    cache.free()


# ------------------------------------------------------------------ MLA prefill
@pytest.mark.parametrize("pos0,n,nh", [(0, 70, 128), (200, 33, 64), (1000, 5, 16), (4000, 20, 128), (63, 130, 96),
                                       (129, 64, 128), (0, 1, 128)])
def test_mla_prefill_chunk(hip, orc, pos0, n, nh):
    say("[case] mla_prefill_chunk", pos0, n, nh)
    c = synth.cfg4_mla_prefill(n, pos0, nh, seed=400 + n)
    cache = hip.LatentCache(1, pos0 + n)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_prefill_chunk(cache, 0, pos0, c["q"], c["scale"])
    ref = orc.mla_prefill_chunk(c["q"], c["rows"], c["scales"], pos0, c["scale"], nthreads=0)
    assert_close(got, ref, "mla_prefill pos0 %d n %d heads %d" % (pos0, n, nh), strict=pos0 >= 200)
    cache.free()


@pytest.mark.parametrize("nh,gain", [(128, 6.0), (128, 12.0), (64, 12.0)])
def test_mla_prefill_chunk_peaked_scores(hip, orc, nh, gain):
    """Queries scaled up so that the scores spread over tens of log2 units: the softmax reference of
    a head moves many times along the keys (64 heads per workgroup move it inside the scoring wave,
    32 reconcile the key blocks a step later), single keys carry whole rows, and both kernels must
    still agree with the oracle.  (The score error of Q as two E4M3 terms grows with the score: at
    gain 12 the scores have a standard deviation of 30 log2 units and near-ties of the two best keys
    are still resolved inside the tolerance; far beyond that they would not be.)"""
    say("[case] mla_prefill_chunk peaked", nh, gain)
    pos0, n = 700, 40
    c = synth.cfg4_mla_prefill(n, pos0, nh, seed=4400 + nh)
    q = synth.f32_to_bf16(synth.bf16_to_f32(c["q"]) * np.float32(gain))
    cache = hip.LatentCache(1, pos0 + n)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_prefill_chunk(cache, 0, pos0, q, c["scale"])
    ref = orc.mla_prefill_chunk(q, c["rows"], c["scales"], pos0, c["scale"], nthreads=0)
    assert_close(got, ref, "mla_prefill peaked heads %d gain %g" % (nh, gain), strict=False)
    cache.free()


def test_mla_prefill_wide_equals_the_decode_kernel(hip, orc):
    """The 64-head prefill kernel against the decode kernel run query by query through the same
    ABI (same operands, two different kernels, both with fp16 weights: up to 6e-4 each against
    the exact result): the difference between them stays inside the tolerance against the oracle."""
    say("[case] mla_prefill wide vs decode per query")
    pos0, n, nh = 300, 9, 128
    c = synth.cfg4_mla_prefill(n, pos0, nh, seed=4500)
    cache = hip.LatentCache(1, pos0 + n)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_prefill_chunk(cache, 0, pos0, c["q"], c["scale"])
    for t in range(n):
        one = hip.mla_decode(cache, 0, c["q"][t], c["scale"], n_list=pos0 + t + 1)
        assert np.abs(got[t] - one).max() <= 1.5e-3, "query %d: %g" % (t, np.abs(got[t] - one).max())
    cache.free()


# ------------------------------------------------------------------ indexer + top-k
@pytest.mark.parametrize("n_keys,ih", [(65536, 64), (1, 64), (1000, 32), (257, 7)])
def test_indexer_scores_bit_exact(hip, orc, n_keys, ih):
    say("[case] indexer_scores", n_keys, ih)
    g = synth.rng(500 + n_keys)
    keys, ks = synth.index_keys(g, n_keys)
    q = synth.normal_bf16(g, (ih, synth.IDIM))
    w = (g.standard_normal(ih, dtype=np.float32) / np.float32(np.sqrt(128.0 * ih))).astype(np.float32)
    cache = hip.IndexKeys(1, n_keys)
    cache.write(0, 0, keys, ks)
    got = hip.indexer_scores(cache, 0, n_keys, q, w)
    ref = orc.indexer_scores(q, w, keys, ks, nthreads=0)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "indexer scores differ in %d of %d places" % ((got != ref).sum(), n_keys)
    cache.free()


@pytest.mark.parametrize("n_keys,ih,kind", [
    (65536, 64, "normal"), (20000, 64, "positive_w"), (5000, 7, "normal"), (40000, 33, "wide"),
])
def test_indexer_approx_within_its_bound(hip, orc, n_keys, ih, kind):
    """The matrix-core scores of the fused select and the bound that comes with them: every key's
    approximate score must lie within the bound of the exact one (the selection relies on it),
    and the bound must be small against the spread of the scores (or the band holds everything).
    Measured against the oracle's exact scores, which the exact kernel reproduces bit for bit."""
    say("[case] indexer approx bound", n_keys, ih, kind)
    g = synth.rng(520 + n_keys + ih)
    keys, ks = synth.index_keys(g, n_keys)
    q = synth.normal_bf16(g, (ih, synth.IDIM))
    w = (g.standard_normal(ih, dtype=np.float32) / np.float32(np.sqrt(128.0 * ih))).astype(np.float32)
    if kind == "positive_w":
        w = np.abs(w)
    if kind == "wide":                              # scales and queries over many binades
        ks = (ks * np.exp2(g.integers(-20, 20, n_keys)).astype(np.float32)).astype(np.float32)
        q = synth.f32_to_bf16(synth.bf16_to_f32(q) * np.exp2(g.integers(-8, 8, (ih, 1))).astype(np.float32))
    cache = hip.IndexKeys(1, n_keys)
    cache.write(0, 0, keys, ks)
    approx, bound = hip.indexer_scores_approx(cache, 0, n_keys, q, w)
    ref = orc.indexer_scores(q, w, keys, ks, nthreads=0)
    err = np.abs(approx.astype(np.float64) - ref.astype(np.float64))
    say("[bound] max error %.3e, bound %.3e (error/bound %.3f), score std %.3e" %
        (err.max(), bound, err.max() / bound, ref.std()))
    assert np.isfinite(bound) and bound > 0
    assert err.max() <= bound, "approximate scores leave their bound: %.3e > %.3e" % (err.max(), bound)
    if kind != "wide":
        assert bound < 1e-2 * ref.std(), "the bound is useless: %.3e against a spread of %.3e" % (bound, ref.std())
    cache.free()


TOPK_KNOWN = [
    ([5, 5, 7], 2, [0, 2]),                      # ds_topk_scores returns {1,2} here
    ([3, 9, 3, 3, 8, 3], 4, [0, 1, 2, 4]),       # ... and {1,2,3,4} here
    ([1, 1, 1, 1, 1], 3, [0, 1, 2]),
    ([2, 1], 5, [0, 1]),
    ([0.0, -0.0, 1.0, -0.0], 3, [0, 1, 2]),
    ([-np.inf, 1, -np.inf, 2], 3, [0, 1, 3]),
]


@pytest.mark.parametrize("sc,k,want", TOPK_KNOWN)
def test_topk_known_answers(hip, orc, sc, k, want):
    say("[case] topk known", sc, k)
    sc = np.array(sc, np.float32)
    assert list(orc.topk_contract(sc, k)) == want
    assert list(hip.topk(sc, k)) == want


@pytest.mark.parametrize("n,k,kind", [
    (65536, 2048, "normal"), (65536, 2048, "ties"), (65536, 2048, "const"),
    (100000, 512, "normal"), (5000, 5000, "normal"), (3000, 4096, "ties"),
    (1 << 20, 2048, "ties"), (777, 1, "normal"), (4097, 2048, "inf"),
    # 16 K .. 128 K scores take the many-workgroup kernels:
    (40000, 1000, "ties"),           # ragged last workgroup, ties across workgroup borders
    (131072, 70, "const"),           # the largest such row; every score ties
    (16384, 16384, "normal"),        # the smallest; k = n
    (20000, 4096, "inf"), (131073, 2048, "normal"),
])
def test_topk_bit_exact(hip, orc, n, k, kind):
    say("[case] topk", n, k, kind)
    g = synth.rng(600 + n + k)
    if kind == "normal":
        sc = g.standard_normal(n, dtype=np.float32)
    elif kind == "ties":
        sc = g.integers(-20, 20, n).astype(np.float32) * np.float32(0.25)
    elif kind == "const":
        sc = np.full(n, 1.5, np.float32)
    else:
        sc = g.standard_normal(n, dtype=np.float32)
        sc[g.random(n) < 0.7] = -np.inf
    got = hip.topk(sc, k)
    ref = orc.topk_contract(sc, k)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("n_keys,topk,ih", [
    (3000, 256, 64),     # every key scored exactly; one workgroup per query in the top-k
    (20000, 512, 64),    # approximate scores + exact band, many workgroups per query, batched
    (65536, 2048, 64),   # BASELINE config 5 geometry (batch 3)
    (17000, 300, 22),    # fewer index heads than the kernels' blocks of 32 and groups of 4
])
def test_dsa_decode_small(hip, orc, n_keys, topk, ih):
    say("[case] dsa_decode small", n_keys, topk, ih)
    c = synth.cfg5_dsa(n_keys=n_keys, batch=3, ih=ih, topk=topk, nh=128, seed=909)
    ik = hip.IndexKeys(3, n_keys)
    lat = hip.LatentCache(3, n_keys)
    for b in range(3):
        ik.write(b, 0, c["ikeys"][b], c["ikscale"][b])
        lat.write(b, 0, c["rows"][b], c["scales"][b])
    out, sel = hip.dsa_decode(ik, lat, 0, 1, n_keys, c["q_idx"], c["w"], topk, c["q"], c["scale"])
    for b in range(3):
        sc = orc.indexer_scores(c["q_idx"][b], c["w"][b], c["ikeys"][b], c["ikscale"][b], nthreads=0)
        rsel = orc.topk_contract(sc, topk)
        assert np.array_equal(sel[b], rsel), "query %d: selected rows differ" % b
        ref = orc.mla_decode(c["q"][b], c["rows"][b], c["scales"][b], c["scale"], sel=rsel, nthreads=0)
        assert_close(out[b], ref, "dsa_decode query %d" % b)
    ik.free()
    lat.free()


@pytest.mark.parametrize("n_keys,topk,copies,take,batch", [(20000, 512, 9, 4, 2), (65536, 2048, 40, 1, 2), (20000, 512, 6, 6, 2),
                                                             (20000, 512, 1400, 200, 8)])
def test_dsa_select_ties_at_the_threshold(hip, orc, n_keys, topk, copies, take, batch):
    """The key that closes the selection exists `copies` times (identical rows: identical exact
    scores) and only `take` of the copies fit: the banded path has to rank its candidates by
    score and then by index, as the reference does.  The last case makes the candidate list of
    each of eight rows longer than one round of the rescoring kernel covers."""
    say("[case] dsa select ties at the threshold", n_keys, topk, copies, take, batch)
    c = synth.cfg5_dsa(n_keys=n_keys, batch=batch, ih=64, topk=topk, nh=128, seed=1300 + copies)
    ikeys = c["ikeys"].copy(); ikscale = c["ikscale"].copy()
    g = synth.rng(77 + copies)
    for b in range(batch):
        sc = orc.indexer_scores(c["q_idx"][b], c["w"][b], ikeys[b], ikscale[b], nthreads=0)
        order = np.lexsort((np.arange(n_keys), -sc.astype(np.float64)))
        # rank topk - take (0-based) is the first copy's rank: `take` copies end the selection
        src = order[topk - take]
        # overwrite keys that rank below the selection, at indices on both sides of src
        dst = g.choice(order[topk + 50:], size=copies - 1, replace=False)
        ikeys[b, dst] = ikeys[b, src]
        ikscale[b, dst] = ikscale[b, src]
    ik = hip.IndexKeys(batch, n_keys)
    lat = hip.LatentCache(batch, n_keys)
    for b in range(batch):
        ik.write(b, 0, ikeys[b], ikscale[b])
        lat.write(b, 0, c["rows"][b], c["scales"][b])
    out, sel = hip.dsa_decode(ik, lat, 0, 1, n_keys, c["q_idx"], c["w"], topk, c["q"], c["scale"])
    for b in range(batch):
        sc = orc.indexer_scores(c["q_idx"][b], c["w"][b], ikeys[b], ikscale[b], nthreads=0)
        rsel = orc.topk_contract(sc, topk)
        T = np.sort(sc)[::-1][topk - 1]
        tied = int((sc == T).sum())
        inside = int((sc[rsel[rsel >= 0]] == T).sum())
        say("[parity] query %d: %d keys tie at the threshold, %d of them selected" % (b, tied, inside))
        assert tied >= copies and inside < tied or take == copies
        assert np.array_equal(sel[b], rsel), "query %d: selected rows differ" % b
        ref = orc.mla_decode(c["q"][b], c["rows"][b], c["scales"][b], c["scale"], sel=rsel, nthreads=0)
        assert_close(out[b], ref, "dsa_decode with ties, query %d of %d" % (b, batch))
    ik.free()
    lat.free()


def test_dsa_decode_as_benchmarked(hip, orc):
    """BASELINE config 5 exactly as bench.py times it: eight independent queries with caches of
    their own, 65536 keys, 64 index heads, top-2048, 128 heads.  The batch sets the number of key
    slices per query (and with it the merge path), so this is not the batch-3 case above: selected
    rows bit for bit and the outputs of all eight queries."""
    say("[case] dsa_decode as benchmarked: batch 8, 65536 keys, top-2048")
    c = synth.cfg5_dsa()
    B, N, K = c["batch"], c["n_keys"], c["topk"]
    assert (B, N, K, c["ih"], c["nh"]) == (8, 65536, 2048, 64, 128)
    ik = hip.IndexKeys(B, N)
    lat = hip.LatentCache(B, N)
    for b in range(B):
        ik.write(b, 0, c["ikeys"][b], c["ikscale"][b])
        lat.write(b, 0, c["rows"][b], c["scales"][b])
    out, sel = hip.dsa_decode(ik, lat, 0, 1, N, c["q_idx"], c["w"], K, c["q"], c["scale"])
    for b in range(B):
        sc = orc.indexer_scores(c["q_idx"][b], c["w"][b], c["ikeys"][b], c["ikscale"][b], nthreads=0)
        rsel = orc.topk_contract(sc, K)
        assert np.array_equal(sel[b], rsel), "query %d: selected rows differ" % b
        ref = orc.mla_decode(c["q"][b], c["rows"][b], c["scales"][b], c["scale"], sel=rsel, nthreads=0)
        assert_close(out[b], ref, "dsa_decode as benchmarked, query %d" % b)
    ik.free()
    lat.free()


@pytest.mark.parametrize("kind", ["same", "two", "zero_w"])
def test_dsa_select_degenerate(hip, orc, kind):
    """Selections where the error band of the approximate scores holds most keys (identical or
    nearly identical scores): the exact kernel has to take over, the indices stay the
    reference's (lowest index first among ties)."""
    say("[case] dsa select degenerate", kind)
    n_keys, topk = 20000, 512
    c = synth.cfg5_dsa(n_keys=n_keys, batch=2, ih=64, topk=topk, nh=128, seed=911)
    ikeys = c["ikeys"].copy(); ikscale = c["ikscale"].copy(); w = c["w"].copy()
    if kind == "same":
        ikeys[:] = ikeys[:, :1]; ikscale[:] = ikscale[:, :1]          # every key the same
    elif kind == "two":
        ikeys[:, 1::2] = ikeys[:, :1]; ikscale[:, 1::2] = ikscale[:, :1]
        ikeys[:, 0::2] = ikeys[:, 1:2]; ikscale[:, 0::2] = ikscale[:, 1:2]
    else:
        w[:] = 0.0                                                     # all scores zero
    ik = hip.IndexKeys(2, n_keys)
    lat = hip.LatentCache(2, n_keys)
    for b in range(2):
        ik.write(b, 0, ikeys[b], ikscale[b])
        lat.write(b, 0, c["rows"][b], c["scales"][b])
    out, sel = hip.dsa_decode(ik, lat, 0, 1, n_keys, c["q_idx"], w, topk, c["q"], c["scale"])
    for b in range(2):
        sc = orc.indexer_scores(c["q_idx"][b], w[b], ikeys[b], ikscale[b], nthreads=0)
        rsel = orc.topk_contract(sc, topk)
        assert np.array_equal(sel[b], rsel), "query %d: selected rows differ" % b
    ik.free()
    lat.free()


# ------------------------------------------------------------------ the two prefill configurations at their full shape
def test_gqa_prefill_full_shape_sampled(hip, orc):
    """BASELINE config 2 as benchmarked: 8192 tokens, 16/4/256, one launch of 512 workgroups
    (128 position blocks, cost-ordered grid, 256 key tiles in the longest rows).  The CPU cannot
    redo 0.55 TFLOP, so rows are sampled: row t of a prefill is the decode at position t (the
    oracle's decode, 33 MFLOP a row), at the first and last rows, on both sides of every kind of
    boundary the kernel has (position blocks of 64, the 1024-key switch between its two variants,
    32-key tiles) and at random places; two whole 128-query tiles, the first and the last, go
    through the oracle's prefill itself."""
    say("[case] gqa_prefill full shape 8192")
    c = synth.cfg2_gqa_prefill()
    n, nh, nkv, hd = c["n"], c["nh"], c["nkv"], c["hd"]
    cache = hip.KVCache(n, nkv, hd)
    cache.write(0, c["k"].reshape(n, -1), c["v"].reshape(n, -1))
    got = hip.gqa_prefill(cache, 0, c["q"], c["scale"])
    assert np.isfinite(got).all()
    g = synth.rng(2024)
    rows = sorted(set([0, 1, 31, 32, 63, 64, 65, 127, 128, 1023, 1024, 1025, 1087, 1088, 4095, 4096,
                       8127, 8128, 8190, 8191] + [int(x) for x in g.integers(0, n, 24)]))
    worst = 0.0
    for t in rows:
        ref = orc.gqa_decode(c["q"][t], c["k"][:t + 1], c["v"][:t + 1], c["scale"], nthreads=0)
        d = np.abs(got[t] - ref).max()
        worst = max(worst, d)
        assert d <= 2e-3 and d / np.abs(ref).max() <= 1e-2, "row %d: max-abs %.3e" % (t, d)
    say("[parity] gqa_prefill 8192: %d sampled rows, worst max-abs %.3e" % (len(rows), worst))
    for tile in (0, 63):
        ref = orc.gqa_prefill(c["q"], c["k"], c["v"], 0, c["scale"], tiles=(tile, tile + 1, 1), nthreads=0)
        sl = slice(128 * tile, 128 * tile + 128)
        assert_close(got[sl], ref[sl], "gqa_prefill 8192, query tile %d" % tile)
    cache.free()


def test_mla_prefill_chunk_full_shape_sampled(hip, orc):
    """BASELINE config 4 as benchmarked: 4096 queries appended to 28672 rows, 128 heads, causal
    over 32768 positions.  Sampled queries (first, last, around the middle and the 64-key tile
    edges, random ones) against the oracle's chunk prefill restricted to those queries."""
    say("[case] mla_prefill_chunk full shape 4096 + 28672")
    c = synth.cfg4_mla_prefill()
    n, pos0, nh = c["n"], c["pos0"], c["nh"]
    cache = hip.LatentCache(1, pos0 + n)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_prefill_chunk(cache, 0, pos0, c["q"], c["scale"])
    cache.free()
    assert np.isfinite(got).all()
    g = synth.rng(4044)
    qs = sorted(set([0, 1, 62, 63, 64, 2047, 2048, 4094, 4095] + [int(x) for x in g.integers(0, n, 5)]))
    ref = np.zeros((n, nh, synth.VDIM), np.float32)
    worst = 0.0
    for t in qs:
        orc.mla_prefill_chunk(c["q"], c["rows"], c["scales"], pos0, c["scale"], queries=(t, t + 1, 1),
                              nthreads=0, out=ref)
        d = np.abs(got[t] - ref[t]).max()
        worst = max(worst, d)
        assert d <= 2e-3 and d / np.abs(ref[t]).max() <= 1e-2, "query %d: max-abs %.3e" % (t, d)
    say("[parity] mla_prefill 4096+28672: %d sampled queries, worst max-abs %.3e" % (len(qs), worst))


# ------------------------------------------------------------------ cache appends from fp32, read-back
def test_kv_write_f32_and_read_back(hip, orc):
    """q35_narrow_rows / q35_widen_rows (src/q35_model.c:1543-1575): fp32 rows narrowed to bf16 on
    the device with round-to-nearest-even, bit-equal to the numpy and the oracle's recipe
    (ties, subnormals and large values included); read back as stored and widened."""
    say("[case] kv write_f32 / read")
    g = synth.rng(31)
    n, nkv, hd = 37, 4, 256
    k = g.standard_normal((n, nkv * hd), dtype=np.float32)
    v = g.standard_normal((n, nkv * hd), dtype=np.float32) * np.float32(1e3)
    k[0, :8] = np.array([1.00390625, 1.01171875, -1.00390625, 0.0, -0.0, 1e-40, 3.3e38, 1.0], np.float32)  # ties up/down
    cache = hip.KVCache(64, nkv, hd)
    cache.write_f32(0, k, v)
    cache.write_f32(40, k[:10], v[:10])                   # an append further along
    kb, vb = cache.read(0, n)
    assert np.array_equal(kb, synth.f32_to_bf16(k)) and np.array_equal(vb, synth.f32_to_bf16(v))
    k40, v40 = cache.read(40, 10)
    assert np.array_equal(k40, kb[:10]) and np.array_equal(v40, vb[:10])
    L = orc.lib()
    assert all(int(kb[0, i]) == L.orc_f32_to_bf16_rne(float(k[0, i])) for i in range(8))
    kf, vf = cache.read_f32(0, n)
    assert np.array_equal(kf.view(np.uint32), synth.bf16_to_f32(kb).view(np.uint32))
    assert np.array_equal(vf.view(np.uint32), synth.bf16_to_f32(vb).view(np.uint32))
    rc = hip.lib().cwick_hip_kv_read(cache.h, 60, 10, kb.ctypes.data, vb.ctypes.data)
    assert rc == 0 and "capacity" in hip.last_error()
    # attention over the rows appended this way = the oracle over rows narrowed on the host
    k[0, 6] = 1.0                                          # keep the scores finite
    cache.write_f32(0, k[:1], v[:1])
    kb, vb = cache.read(0, n)
    q = synth.normal_bf16(g, (16, hd))
    got = hip.gqa_decode(cache, n, q, 0.0625)
    ref = orc.gqa_decode(q, synth.f32_to_bf16(k).reshape(n, nkv, hd), synth.f32_to_bf16(v).reshape(n, nkv, hd), 0.0625)
    assert_close(got, ref, "gqa_decode over rows appended as fp32", strict=False)
    cache.free()


def test_ikeys_write_f32_and_read_back(hip, orc):
    say("[case] ikeys write_f32 / read")
    g = synth.rng(32)
    x = g.standard_normal((200, synth.IDIM), dtype=np.float32)
    x[3] = 0.0
    x[4] *= 1e-5
    c = hip.IndexKeys(2, 256)
    c.write_f32(1, 10, x)
    rows, scales = c.read(1, 10, 200)
    rq, rs = orc.quantize_rows_e4m3(x, synth.IDIM)
    assert np.array_equal(rows, rq) and np.array_equal(scales.view(np.uint32), rs[:, 0].view(np.uint32))
    nq, ns = synth.quantize_rows(x, synth.IDIM)
    assert np.array_equal(nq, rq)
    # scores over the keys quantised on the device
    q = synth.normal_bf16(g, (64, synth.IDIM))
    w = (g.standard_normal(64, dtype=np.float32) / np.float32(np.sqrt(128.0 * 64))).astype(np.float32)
    c2 = hip.IndexKeys(1, 256)
    c2.write(0, 0, rows, scales)
    got = hip.indexer_scores(c2, 0, 200, q, w)
    ref = orc.indexer_scores(q, w, rq, rs[:, 0], nthreads=0)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    c.free(); c2.free()


# ------------------------------------------------------------------ backend selection
def test_force_off_declines_and_on_again_works(hip, orc):
    """cwick_hip_force mirrors cwick_metal_force (src/metal.c:60-79): 0 selects the CPU and every
    compute call declines with its outputs untouched, 1 selects the GPU again.  shutdown frees
    the internal workspaces; the next call allocates them anew."""
    say("[case] force(0) / force(1) / shutdown")
    c = synth.cfg3_mla_decode(700, 16, seed=5)
    cache = hip.LatentCache(1, 700)
    cache.write(0, 0, c["rows"], c["scales"])
    ref = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=0)
    assert_close(hip.mla_decode(cache, 0, c["q"], c["scale"], n_list=700), ref, "before force(0)")
    assert hip.force(False) == 0
    assert not hip.ready()
    out = np.full((16, synth.VDIM), 7.0, np.float32)
    q = np.ascontiguousarray(c["q"], np.uint16)
    rc = hip.lib().cwick_hip_mla_decode(cache.h, 0, None, 700, q.ctypes.data, 16, c["scale"], out.ctypes.data)
    assert rc == 0 and (out == 7.0).all()
    assert "not selected" in hip.last_error() or "unavailable" in hip.last_error()
    rc, _ = hip.topk(np.arange(8, dtype=np.float32), 3, raw=True)
    assert rc == 0
    assert hip.force(True) == 0 and hip.ready()
    assert_close(hip.mla_decode(cache, 0, c["q"], c["scale"], n_list=700), ref, "after force(1)")
    hip.shutdown()
    assert hip.ready()
    assert_close(hip.mla_decode(cache, 0, c["q"], c["scale"], n_list=700), ref, "after shutdown")
    assert list(hip.topk(np.array([1, 3, 2, 3], np.float32), 2)) == [1, 3]
    cache.free()


def test_two_handles_on_two_threads(hip, orc):
    """Every handle has its own stream, staging buffer and split-K workspace: calls on different
    handles from different threads (one request slot each, src/metal.c:306-319) do not disturb
    one another."""
    import threading
    say("[case] two handles, two threads")
    cs = [synth.cfg3_mla_decode(4000 + 500 * i, 128, seed=60 + i) for i in range(2)]
    caches = []
    for c in cs:
        h = hip.LatentCache(1, c["n_keys"])
        h.write(0, 0, c["rows"], c["scales"])
        caches.append(h)
    refs = [orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=0) for c in cs]
    errs = [None, None]

    def work(i):
        try:
            for _ in range(30):
                got = hip.mla_decode(caches[i], 0, cs[i]["q"], cs[i]["scale"], n_list=cs[i]["n_keys"])
                d = np.abs(got - refs[i]).max()
                if not d <= 2e-3:
                    errs[i] = "thread %d: max-abs %.3e" % (i, d)
                    return
        except Exception as e:      # noqa: BLE001
            errs[i] = repr(e)
    th = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    [t.start() for t in th]
    [t.join() for t in th]
    assert errs == [None, None], errs
    for h in caches:
        h.free()


# ------------------------------------------------------------------ MLA decode: more edge cases
def test_mla_decode_dev_batched_strides(hip, orc):
    """cwick_hip_mla_decode_dev with a batch of queries that read different caches (batch
    strides), one of them through a list: the form the fused DSA step and the benchmark call."""
    import torch
    say("[case] mla_decode_dev batch strides")
    B, n_rows, nh = 3, 3000, 128
    cs = [synth.cfg3_mla_decode(n_rows, nh, seed=80 + b) for b in range(B)]
    rows = torch.from_numpy(np.stack([c["rows"] for c in cs])).cuda()
    scales = torch.from_numpy(np.stack([c["scales"] for c in cs])).cuda()
    q = torch.from_numpy(np.stack([c["q"] for c in cs]).view(np.int16)).cuda()
    out = torch.empty((B, nh, synth.VDIM), dtype=torch.float32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    hip.mla_decode_dev(rows, scales, n_rows * synth.KDIM, n_rows * synth.NBLK, n_rows, B, None, n_rows,
                       q, nh, cs[0]["scale"], out, s)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for b in range(B):
        ref = orc.mla_decode(cs[b]["q"], cs[b]["rows"], cs[b]["scales"], cs[b]["scale"], nthreads=0)
        assert_close(got[b], ref, "mla_decode_dev dense, batch row %d" % b)
    g = synth.rng(83)
    sel = np.stack([np.sort(g.permutation(n_rows)[:1000]) for _ in range(B)]).astype(np.int32)
    sel[1, 990:] = -1
    dsel = torch.from_numpy(sel).cuda()
    hip.mla_decode_dev(rows, scales, n_rows * synth.KDIM, n_rows * synth.NBLK, n_rows, B, dsel, 1000,
                       q, nh, cs[0]["scale"], out, s)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for b in range(B):
        ref = orc.mla_decode(cs[b]["q"], cs[b]["rows"], cs[b]["scales"], cs[b]["scale"], sel=sel[b], nthreads=0)
        assert_close(got[b], ref, "mla_decode_dev sel, batch row %d" % b)


@pytest.mark.parametrize("n_keys", [32768, 2500])
def test_mla_decode_q_outliers(hip, orc, n_keys):
    """An absorbed query q_abs = W_k^T q has outliers inside its 128-dim blocks.  The kernel
    splits Q into two E4M3 terms under one power-of-two scale per head and block, so an outlier
    sets the scale for its 127 neighbours: elements 256 and 4096 times larger than the rest of
    their block, in every block kind (nope and rope), must still give scores inside tolerance."""
    say("[case] mla_decode with outliers in Q", n_keys)
    c = synth.cfg3_mla_decode(n_keys, 128, seed=1700 + n_keys)
    qf = synth.bf16_to_f32(c["q"]).copy()
    g = synth.rng(17)
    for h in range(128):
        for blk, width in ((0, 128), (2, 128), (4, 64)):
            i = 128 * blk + int(g.integers(0, width))
            # the outlier carries little of the score (small factor on a large element would not
            # be an outlier): scale the rest of the block down instead, keeping the score's size
            qf[h, 128 * blk:128 * blk + width] *= np.float32(1.0 / (256.0 if h % 2 else 4096.0))
            qf[h, i] *= np.float32(256.0 if h % 2 else 4096.0) * np.float32(0.25)
    q = synth.f32_to_bf16(qf)
    cache = hip.LatentCache(1, n_keys)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_decode(cache, 0, q, c["scale"], n_list=n_keys)
    ref = orc.mla_decode(q, c["rows"], c["scales"], c["scale"], nthreads=0)
    assert_close(got, ref, "mla_decode, outliers in Q, %d keys" % n_keys)
    cache.free()


def test_mla_decode_rows_outside_the_list_do_not_leak(hip, orc):
    """Masked positions of a tile (a ragged end, -1 entries) must contribute nothing whatever the
    cache holds elsewhere: row 0 is not in the list and holds NaN bytes and a scale 2^40 times
    the others; a second unlisted row is all NaN bytes."""
    say("[case] mla_decode: unlisted rows with NaN bytes and huge scales")
    n_rows, nh = 3000, 128
    c = synth.cfg3_mla_decode(n_rows, nh, seed=91)
    rows, scales = c["rows"].copy(), c["scales"].copy()
    rows[0, ::3] = 0x7F
    rows[0, 1::3] = 0xFF
    scales[0] *= np.float32(2.0 ** 40)
    rows[1234] = 0x7F
    scales[1234] = np.float32(np.inf)
    g = synth.rng(92)
    pool = np.setdiff1d(np.arange(n_rows), [0, 1234])
    sel = g.choice(pool, size=1000, replace=False).astype(np.int32)
    sel[[0, 63, 64, 500, 999]] = -1
    cache = hip.LatentCache(1, n_rows)
    cache.write(0, 0, rows, scales)
    got = hip.mla_decode(cache, 0, c["q"], c["scale"], sel=sel)
    ref = orc.mla_decode(c["q"], rows, scales, c["scale"], sel=sel, nthreads=0)
    assert_close(got, ref, "mla_decode sel with poisoned unlisted rows")
    # a ragged dense list that stops before the poisoned row 1234
    rows[0] = c["rows"][0]; scales[0] = c["scales"][0]
    cache.write(0, 0, rows[:1], scales[:1])
    got = hip.mla_decode(cache, 0, c["q"], c["scale"], n_list=1201)
    ref = orc.mla_decode(c["q"], rows, scales, c["scale"], nlist=1201, nthreads=0)
    assert_close(got, ref, "mla_decode dense, poisoned row past the end of the list")
    cache.free()


@pytest.mark.parametrize("n_rows,n_sel", [(5000, 2048), (40000, 0), (300, 40)])
def test_mla_decode_sink(hip, orc, n_rows, n_sel):
    """The attention sink of ds_sparse_attn_heads (src/ds_model.c:946): exp(sink[h] - max) in the
    denominator only.  One launch without split-K (short list), one with (merge kernel)."""
    say("[case] mla_decode with sink", n_rows, n_sel)
    nh = 128
    c = synth.cfg3_mla_decode(n_rows, nh, seed=95 + n_rows)
    g = synth.rng(96)
    sel = None
    if n_sel:
        sel = g.permutation(n_rows)[:n_sel].astype(np.int32)
        sel[::97] = -1
    # sinks around the largest score of each head, so that they matter
    base = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=sel, nthreads=0)
    sink = (g.standard_normal(nh) * 2.0 + 5.0).astype(np.float32)
    cache = hip.LatentCache(1, n_rows)
    cache.write(0, 0, c["rows"], c["scales"])
    got = hip.mla_decode(cache, 0, c["q"], c["scale"], sel=sel, n_list=None if n_sel else n_rows, sink=sink)
    ref = orc.sparse_attn_sink(c["q"], c["rows"], c["scales"], c["scale"], sink=sink, sel=sel, nthreads=0)
    assert_close(got, ref, "mla_decode sink %d rows" % n_rows)
    assert np.abs(ref - base).max() > 10 * 2e-3 or n_rows > 10000, "the sink does not show in this case"
    # every entry skipped: zeros, with or without the sink
    none = hip.mla_decode(cache, 0, c["q"], c["scale"], sel=np.full(70, -1, np.int32), sink=sink)
    assert np.array_equal(none, np.zeros_like(none))
    cache.free()


@pytest.mark.parametrize("pos,W,n_cmp,topk", [(50, 128, 0, 64), (127, 128, 31, 64), (1000, 128, 250, 64),
                                              (5000, 128, 1250, 512)])
def test_window_ring_and_compressed_rows_with_sink(hip, orc, pos, W, n_cmp, topk):
    """ds_sparse_attn_heads' key list (src/ds_model.c:917-932, built at :1214-1237): a ring of W
    window rows written at slot pos % W, then the compressed rows; idx[] holds the ring slots of
    the W positions ending at pos (oldest first, -1 where the sequence has not got to), then W + j
    for the compressed rows the indexer kept (-1 padded).  With the store laid out
    [ring | compressed] idx[] is a row list as it stands: the sparse decode with the sink against
    the oracle over a host mirror of the same store."""
    say("[case] window ring + compressed rows + sink", pos, W, n_cmp, topk)
    nh = 128
    g = synth.rng(8800 + pos)
    n_pos = pos + 1
    lat_rows, lat_scales = synth.latent_cache(g, n_pos)             # the window latent of every position so far
    cmp_rows, cmp_scales = synth.latent_cache(g, max(n_cmp, 1))
    q = synth.normal_bf16(g, (nh, synth.KDIM))
    scale = float(1.0 / np.sqrt(192.0))
    cache = hip.LatentCache(1, W + max(n_cmp, 1))
    ring_rows = np.zeros((W, synth.KDIM), np.uint8)
    ring_scales = np.zeros((W, synth.NBLK), np.float32)
    cache.write(0, 0, ring_rows, ring_scales)                        # the reference clears the ring (:714)
    # written in wrap order, one position at a time where the ring wraps (the last 2 W positions),
    # so that slots are overwritten on the device as the engine would
    first_single = max(0, n_pos - 2 * W)
    for pp in range(first_single):
        ring_rows[pp % W] = lat_rows[pp]; ring_scales[pp % W] = lat_scales[pp]
    if first_single:
        cache.write(0, 0, ring_rows, ring_scales)
    for pp in range(first_single, n_pos):
        ring_rows[pp % W] = lat_rows[pp]; ring_scales[pp % W] = lat_scales[pp]
        cache.write(0, pp % W, lat_rows[pp:pp + 1], lat_scales[pp:pp + 1])
    if n_cmp:
        cache.write(0, W, cmp_rows, cmp_scales)
    idx = []
    lo = max(0, pos - W + 1)
    for pp in range(lo, pos + 1):
        idx.append(pp % W)
    idx += [-1] * (W - len(idx))
    ncmp = min(n_cmp, topk)
    kept = np.sort(g.permutation(n_cmp)[:ncmp]) if n_cmp else np.zeros(0, np.int64)
    idx += [W + int(j) for j in kept]
    idx = np.array(idx, np.int32)
    assert idx.size == W + ncmp
    sink = (g.standard_normal(nh) * 2.0 + 4.0).astype(np.float32)
    store_rows = np.concatenate([ring_rows, cmp_rows]); store_scales = np.concatenate([ring_scales, cmp_scales])
    got = hip.mla_decode(cache, 0, q, scale, sel=idx, sink=sink)
    ref = orc.sparse_attn_sink(q, store_rows, store_scales, scale, sink=sink, sel=idx, nthreads=0)
    assert_close(got, ref, "window ring pos %d" % pos)
    # the ring really holds the last W positions: the same output from a list over the positions' own latents
    live = np.arange(lo, pos + 1)
    flat_rows = np.concatenate([lat_rows[live], cmp_rows[kept]]) if ncmp else lat_rows[live]
    flat_scales = np.concatenate([lat_scales[live], cmp_scales[kept]]) if ncmp else lat_scales[live]
    ref2 = orc.sparse_attn_sink(q, flat_rows, flat_scales, scale, sink=sink, sel=None, nthreads=0)
    assert np.abs(ref - ref2).max() <= 1e-5 * max(1.0, np.abs(ref2).max())
    cache.free()


# ------------------------------------------------------------------ the DeepSeek indexer flavour
@pytest.mark.parametrize("n_keys,ih", [(65536, 64), (1000, 32), (257, 7), (1, 64)])
def test_indexer_scores_ds_mode_bit_exact(hip, orc, n_keys, ih):
    """ds_indexer's roundings (src/ds_model.c:1099-1121): serial dot over the dequantised key,
    bf16-rounded dot before the ReLU, bf16-rounded weight: bit for bit."""
    say("[case] indexer_scores DS mode", n_keys, ih)
    g = synth.rng(700 + n_keys)
    keys, ks = synth.index_keys(g, n_keys)
    q = synth.normal_bf16(g, (ih, synth.IDIM))
    w = (g.standard_normal(ih, dtype=np.float32) / np.float32(np.sqrt(128.0 * ih))).astype(np.float32)
    cache = hip.IndexKeys(1, n_keys)
    cache.write(0, 0, keys, ks)
    got = hip.indexer_scores(cache, 0, n_keys, q, w, mode=hip.INDEXER_DS)
    ref = orc.indexer_scores_ds(q, w, keys, ks, nthreads=0)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "DS-mode scores differ in %d of %d places" % ((got != ref).sum(), n_keys)
    glm = hip.indexer_scores(cache, 0, n_keys, q, w, mode=hip.INDEXER_GLM)
    assert np.array_equal(glm.view(np.uint32), hip.indexer_scores(cache, 0, n_keys, q, w).view(np.uint32))
    if n_keys > 100:
        assert (glm != got).any()
    rc, _ = hip.indexer_scores(cache, 0, n_keys, q, w, mode=7, raw=True)
    assert rc == 0 and "mode" in hip.last_error()
    cache.free()


# ------------------------------------------------------------------ the steps around the attention kernels
def test_mla_absorb_decode_expand_chain_on_device(hip, orc):
    """W_k absorb -> MLA decode -> W_v expand with every intermediate in HBM (the absorbed query
    and c_acc never cross the host link): src/attention.c:741-744, :749-811, :812-815.  Each
    device step is compared with the oracle's restatement on its own (absorb and expand to fp32
    rounding: the GPU sums in a different order; tolerance 1e-4 relative to the largest value,
    plus the bf16 rounding of q_abs), and the chain as a whole with the oracle's chain."""
    import torch
    say("[case] absorb -> decode -> expand on the device")
    nh, nope, rope, vdim, kv_lora, n_keys = 128, 128, 64, 128, 512, 3000
    q_dim, kv_dim = nope + rope, nope + vdim
    g = synth.rng(1234)
    kvb = synth.f32_to_bf16(g.standard_normal((nh * kv_dim, kv_lora), dtype=np.float32) * np.float32(kv_lora ** -0.5))
    q = g.standard_normal((nh, q_dim), dtype=np.float32)
    c = synth.cfg3_mla_decode(n_keys, nh, seed=1235)
    s = torch.cuda.current_stream().cuda_stream
    d_kvb = torch.from_numpy(kvb.view(np.int16)).cuda()
    d_q = torch.from_numpy(q).cuda()
    d_qabs = torch.empty((nh, synth.KDIM), dtype=torch.int16, device="cuda")
    d_rows = torch.from_numpy(c["rows"]).cuda(); d_scales = torch.from_numpy(c["scales"]).cuda()
    d_cacc = torch.empty((nh, synth.VDIM), dtype=torch.float32, device="cuda")
    d_out = torch.empty((nh, vdim), dtype=torch.float32, device="cuda")
    hip.mla_absorb_dev(d_kvb, d_q, 0, 1, nh, q_dim, nope, rope, kv_dim, kv_lora, d_qabs, s)
    hip.mla_decode_dev(d_rows, d_scales, 0, 0, n_keys, 1, None, n_keys, d_qabs, nh, c["scale"], d_cacc, s)
    hip.mla_expand_dev(d_kvb, d_cacc, 1, nh, nope, vdim, kv_dim, kv_lora, d_out, s)
    torch.cuda.synchronize()
    # absorb
    qabs_ref = orc.mla_absorb(kvb, q, nope, rope, kv_dim)
    qabs_got = synth.bf16_to_f32(d_qabs.cpu().numpy().view(np.uint16))
    scale_q = np.abs(qabs_ref).max()
    assert np.abs(qabs_got - qabs_ref).max() <= 2.0 ** -8 * scale_q + 1e-4 * scale_q        # bf16 rounding of the output
    assert np.array_equal(qabs_got[:, 512:], synth.bf16_to_f32(synth.f32_to_bf16(q[:, nope:])))
    # decode from the device's own q_abs bits
    qabs_bits = d_qabs.cpu().numpy().view(np.uint16)
    cacc_ref = orc.mla_decode(qabs_bits, c["rows"], c["scales"], c["scale"], nthreads=0)
    cacc_got = d_cacc.cpu().numpy()
    assert_close(cacc_got, cacc_ref, "decode inside the device chain")
    # expand from the device's own c_acc
    out_ref = orc.mla_expand(kvb, cacc_got, nope, vdim, kv_dim)
    out_got = d_out.cpu().numpy()
    assert np.abs(out_got - out_ref).max() <= 1e-4 * np.abs(out_ref).max()
    # the chain against the oracle's chain (q_abs narrowed to bf16 there as well)
    chain = orc.mla_expand(kvb, orc.mla_decode(synth.f32_to_bf16(qabs_ref), c["rows"], c["scales"], c["scale"],
                                               nthreads=0), nope, vdim, kv_dim)
    assert_close(out_got, chain, "absorb -> decode -> expand")
    # a latent width other than 512 is declined
    rc = hip.lib().cwick_hip_mla_absorb_dev(d_kvb.data_ptr(), d_q.data_ptr(), 0, 1, nh, q_dim, nope, rope, kv_dim,
                                            256, d_qabs.data_ptr(), s)
    assert rc == 0 and "kv_lora" in hip.last_error()


@pytest.mark.parametrize("n,pos0,H,KV,HD,rotary,gate", [(1, 4095, 16, 4, 256, 64, True), (300, 100, 16, 4, 256, 64, True),
                                                       (17, 0, 8, 8, 128, 128, False), (5, 9, 4, 2, 256, 0, False)])
def test_gqa_prepare_on_device_then_attention(hip, orc, n, pos0, H, KV, HD, rotary, gate):
    """q/k head norm + RoPE + narrowing + cache append on the device (src/q35_model.c:1627-1652),
    then attention over the rows it appended, queries never leaving HBM.  The prepared values
    agree with the oracle's to one bf16 step (the sum of squares is a wave's tree sum here and a
    serial loop there: tolerance 2^-7 relative per head, stated)."""
    import torch
    say("[case] gqa_prepare", n, pos0, H, KV, HD, rotary, gate)
    g = synth.rng(4321 + n)
    stride = HD * (2 if gate else 1)
    theta, eps = 1e6, 1e-6
    cos_t, sin_t = orc.build_rope(pos0 + n, max(rotary, 2), theta)
    qp = g.standard_normal((n, H, stride), dtype=np.float32)
    kp = g.standard_normal((n, KV * HD), dtype=np.float32)
    vp = g.standard_normal((n, KV * HD), dtype=np.float32)
    qn = (g.standard_normal(HD, dtype=np.float32) * np.float32(0.1))
    kn = (g.standard_normal(HD, dtype=np.float32) * np.float32(0.1))
    cache = hip.KVCache(pos0 + n, KV, HD)
    if pos0:
        past = synth.cfg2_gqa_prefill(pos0, H, KV, HD, 0, seed=99)
        cache.write(0, past["k"].reshape(pos0, -1), past["v"].reshape(pos0, -1))
    s = torch.cuda.current_stream().cuda_stream
    d = lambda a: torch.from_numpy(a).cuda()
    d_q = torch.empty((n, H, HD), dtype=torch.int16, device="cuda")
    hip.gqa_prepare_dev(d(qp), stride, d(kp), d(vp), n, pos0, H, KV, HD, d(qn), d(kn), eps, d(cos_t), d(sin_t),
                        rotary, d_q, cache, s)
    torch.cuda.synchronize()
    q_got = d_q.cpu().numpy().view(np.uint16)
    k_got, v_got = cache.read(pos0, n)
    q_ref, k_ref, v_ref = orc.gqa_prepare(qp, stride, kp, vp, pos0, H, KV, HD, qn, kn, eps, cos_t, sin_t, rotary)
    assert np.array_equal(v_got, v_ref)                           # narrowing only: bit for bit
    for got, ref, heads in ((q_got.reshape(n, H, HD), q_ref.reshape(n, H, HD), H),
                            (k_got.reshape(n, KV, HD), k_ref.reshape(n, KV, HD), KV)):
        gf, rf = synth.bf16_to_f32(got), synth.bf16_to_f32(ref)
        tol = 2.0 ** -7 * np.abs(rf).max(axis=-1, keepdims=True)
        assert (np.abs(gf - rf) <= tol).all(), "prepared heads differ by more than a bf16 step"
        assert (got != ref).mean() < 0.02, "more than 2 %% of the prepared values differ from the oracle's bits"
    if HD == 256 and KV * 4 >= H:
        # attention straight from the prepared queries and the appended rows
        out = torch.empty((n, H, HD), dtype=torch.float32, device="cuda")
        scale = float(HD) ** -0.5
        hip.gqa_prefill_dev(cache.k_dev(), cache.v_dev(), pos0, n, KV, HD, d_q, H, scale, out, s)
        torch.cuda.synchronize()
        k_all, v_all = cache.read(0, pos0 + n)
        ref = orc.gqa_prefill(q_got.reshape(n, H, HD), k_all.reshape(-1, KV, HD), v_all.reshape(-1, KV, HD), pos0, scale,
                              nthreads=0)
        assert_close(out.cpu().numpy(), ref, "gqa_prefill over prepared queries and rows")
    rc = hip.gqa_prepare_dev(d(qp), stride, d(kp), d(vp), n, pos0 + 1, H, KV, HD, d(qn), d(kn), eps, d(cos_t), d(sin_t),
                             rotary, d_q, cache, s, raw=True)
    assert rc == 0 and "capacity" in hip.last_error()
    cache.free()


# ------------------------------------------------------------------ indexer pool, candidate blocks, snapshots
@pytest.mark.parametrize("kp,n_pools", [(4, 301), (1, 5), (8, 64), (3, 2)])
def test_ikeys_pool_append_on_device(hip, orc, kp, n_pools):
    """Closing indexer pools on the device (src/attention.c:486-525): the fp32 keys against the
    oracle's (statistics in double on both sides; expf differs between the device's and the
    host's library, so 1e-5 relative + 1e-6 absolute, stated), and the stored rows bit for bit
    against the oracle's quantiser run over the device's own fp32 keys."""
    import torch
    say("[case] ikeys_pool_append", kp, n_pools)
    g = synth.rng(700 + kp)
    eps = 1e-6
    tk = (g.standard_normal((n_pools, kp, synth.IDIM), dtype=np.float32) * np.float32(2) + np.float32(0.7))
    tg = g.standard_normal((n_pools, kp, synth.IDIM), dtype=np.float32)
    tk[0, 0] = 3.0                                            # a constant row: zero variance, eps carries it
    ape = synth.f32_to_bf16(g.standard_normal((kp, synth.IDIM), dtype=np.float32) * np.float32(0.5))
    w = (1 + 0.1 * g.standard_normal(synth.IDIM, dtype=np.float32)).astype(np.float32)
    b = (0.1 * g.standard_normal(synth.IDIM, dtype=np.float32)).astype(np.float32)
    c = hip.IndexKeys(2, 512)
    d = lambda a: torch.from_numpy(a).cuda()
    d_f32 = torch.empty((n_pools, synth.IDIM), dtype=torch.float32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    c.pool_append_dev(1, 7, n_pools, d(tk), d(tg), d(ape.view(np.int16)), d(w), d(b), eps, kp, d_f32, s)
    torch.cuda.synchronize()
    got = d_f32.cpu().numpy()
    ref = np.stack([orc.indexer_pool_row(tk[i], tg[i], ape, w, b, eps) for i in range(n_pools)])
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)
    rows, scales = c.read(1, 7, n_pools)
    rq, rs = orc.quantize_rows_e4m3(got, synth.IDIM)
    assert np.array_equal(rows, rq) and np.array_equal(scales.view(np.uint32), rs[:, 0].view(np.uint32))
    # against the quantised oracle keys: the same bytes but for values that sit on a rounding edge
    oq, _ = orc.quantize_rows_e4m3(ref, synth.IDIM)
    assert (rows != oq).mean() < 2e-3
    # without the fp32 copy, and declined outside the store
    c.pool_append_dev(0, 0, n_pools, d(tk), d(tg), d(ape.view(np.int16)), d(w), d(b), eps, kp, None, s)
    torch.cuda.synchronize()
    r0, s0 = c.read(0, 0, n_pools)
    assert np.array_equal(r0, rows) and np.array_equal(s0, scales)
    rc = c.pool_append_dev(0, 512 - n_pools + 1, n_pools, d(tk), d(tg), d(ape.view(np.int16)), d(w), d(b), eps, kp,
                           None, s, raw=True)
    assert rc == 0 and "capacity" in hip.last_error()
    rc = c.pool_append_dev(0, 0, n_pools, d(tk), d(tg), d(ape.view(np.int16)), d(w), d(b), eps, 9, None, s, raw=True)
    assert rc == 0 and "kpool" in hip.last_error()
    c.free()


@pytest.mark.parametrize("batch,n,bs,keep", [(1, 65536, 64, 32), (4, 10000, 128, 8), (2, 65, 64, 1), (3, 300, 7, 50),
                                             (1, 5, 64, 3), (2, 131072, 64, 512),
                                             # more than 14336 blocks: the block top-k is the many-workgroup select,
                                             # which keeps a workspace of its own next to this call's block scores
                                             (1, 16000, 1, 100), (2, 31000, 2, 64)])
def test_candidate_blocks_on_device(hip, orc, batch, n, bs, keep):
    """Level one of the two-level selection (src/ds_model.c:1125-1148): the byte mask bit for bit
    against the oracle's, then masked scores -> top-k equal to the oracle's selection over its own
    masked scores."""
    import torch
    say("[case] candidate blocks", batch, n, bs, keep)
    g = synth.rng(n + bs)
    sc = g.standard_normal((batch, n), dtype=np.float32)
    d_sc = torch.from_numpy(sc).cuda()
    d_cand = torch.full((batch, n), 7, dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    hip.candidate_select_dev(d_sc, batch, n, bs, keep, d_cand, s)
    torch.cuda.synchronize()
    cand = d_cand.cpu().numpy()
    for r in range(batch):
        want, k = orc.candidate_mask(sc[r], bs, keep)
        assert np.array_equal(cand[r], want), "row %d" % r
    # a later layer: its own scores, masked by the shared candidates, then the positions
    sc2 = g.standard_normal((batch, n), dtype=np.float32)
    d_sc2 = torch.from_numpy(sc2).cuda()
    hip.candidate_apply_dev(d_sc2, d_cand, batch, n, s)
    torch.cuda.synchronize()
    masked = d_sc2.cpu().numpy()
    kk = min(n, 2048)
    d_idx = torch.empty((batch, kk), dtype=torch.int32, device="cuda")
    hip.topk_dev(d_sc2, batch, n, kk, d_idx, s)
    torch.cuda.synchronize()
    idx = d_idx.cpu().numpy()
    for r in range(batch):
        ref_masked = orc.candidate_apply(sc2[r], cand[r])
        assert np.array_equal(masked[r].view(np.uint32), ref_masked.view(np.uint32))
        n_cand = int(cand[r].sum())
        # the reference selects `cnt` positions and the -inf ones can only come last; positions
        # that are candidates fill the list first
        want = orc.topk_contract(ref_masked, kk)
        got = idx[r][idx[r] >= 0]
        if n_cand >= kk:
            assert np.array_equal(np.sort(got), np.sort(want))
            assert cand[r][got].all()
        else:
            assert cand[r][got].sum() == n_cand
    rc = hip.candidate_select_dev(d_sc, batch, n, 0, keep, d_cand, s, raw=True)
    assert rc == 0 and "block" in hip.last_error()


def test_candidate_select_declines_too_many_blocks(hip):
    import torch
    say("[case] candidate blocks: too many blocks")
    sc = torch.zeros((1, 20000), dtype=torch.float32, device="cuda")
    cand = torch.zeros((1, 20000), dtype=torch.uint8, device="cuda")
    rc = hip.candidate_select_dev(sc, 1, 20000, 1, 4, cand, torch.cuda.current_stream().cuda_stream, raw=True)
    assert rc == 0 and "16383" in hip.last_error()


def test_snapshot_reads_dequantised_rows_and_restores_them(hip, orc):
    """Prefix snapshots hold fp32 (src/pfx.h:63-67, filled by src/engine.c:3626-3666): rows read
    back dequantised equal byte value x block scale exactly; writing them into another store
    reproduces the bytes, and the scales to one unit in the last place; attention over the
    restored store equals attention over the original."""
    say("[case] snapshot read_f32 / restore")
    c3 = synth.cfg3_mla_decode(700, 16, seed=77)
    lat = hip.LatentCache(2, 1024)
    lat.write(1, 5, c3["rows"], c3["scales"])
    f = lat.read_f32(1, 5, 700)
    lut = orc.e4m3_lut()
    want = lut[c3["rows"]] * np.repeat(c3["scales"], 128, axis=1)[:, :synth.KDIM]
    assert np.array_equal(f.view(np.uint32), want.astype(np.float32).view(np.uint32))
    lat2 = hip.LatentCache(1, 700)
    lat2.write_f32(0, 0, f)
    r2, s2 = lat2.read(0, 0, 700)
    assert np.array_equal(r2, c3["rows"])
    assert np.abs(s2.view(np.int32) - c3["scales"].view(np.int32)).max() <= 1
    a = hip.mla_decode(lat, 1, c3["q"], c3["scale"], sel=np.arange(5, 705, dtype=np.int32))
    b = hip.mla_decode(lat2, 0, c3["q"], c3["scale"], n_list=700)
    assert_close(b, a, "attention over the restored latent store")
    # indexer keys
    g = synth.rng(78)
    x = g.standard_normal((300, synth.IDIM), dtype=np.float32)
    x[9] = 0.0
    ik = hip.IndexKeys(1, 512)
    ik.write_f32(0, 100, x)
    rows, scales = ik.read(0, 100, 300)
    fx = ik.read_f32(0, 100, 300)
    assert np.array_equal(fx.view(np.uint32), (lut[rows] * scales[:, None]).astype(np.float32).view(np.uint32))
    ik2 = hip.IndexKeys(1, 300)
    ik2.write_f32(0, 0, fx)
    rr, ss = ik2.read(0, 0, 300)
    assert np.array_equal(rr, rows) and np.abs(ss.view(np.int32) - scales.view(np.int32)).max() <= 1
    rc = hip.lib().cwick_hip_latent_read_f32(lat.h, 1, 1000, 100, f.ctypes.data)
    assert rc == 0 and "capacity" in hip.last_error()
    lat.free(); lat2.free(); ik.free(); ik2.free()


# ------------------------------------------------------------------ block-sparse GQA decode
@pytest.mark.parametrize("n_rows,nh,nkv,hd,bs,keep", [(4096, 16, 4, 256, 64, 8), (700, 8, 8, 128, 16, 5), (3000, 64, 8, 128, 128, 4),
                                                      (64, 16, 4, 256, 64, 1)])
def test_gqa_decode_over_selected_blocks(hip, orc, n_rows, nh, nkv, hd, bs, keep):
    """The attention of the block-sparse decode (src/mm_model.c:1962-2047) over positions expanded
    from selected blocks as the reference expands them (:1966-1973: whole blocks in the order of
    selection, clipped to the positions written).  Checked against the oracle's decode over the
    gathered rows (the same softmax and sums over the same set)."""
    import torch
    say("[case] gqa_decode_sel", n_rows, nh, nkv, hd, bs, keep)
    g = synth.rng(9000 + n_rows)
    c = synth.cfg2_gqa_prefill(n_rows, nh, nkv, hd, 0, seed=900 + n_rows)
    cache = hip.KVCache(n_rows, nkv, hd)
    cache.write(0, c["k"].reshape(n_rows, -1), c["v"].reshape(n_rows, -1))
    nblk = -(-n_rows // bs)
    blocks = g.permutation(nblk)[:keep]
    if nblk - 1 not in blocks:
        blocks[-1] = nblk - 1                                # the newest block, always (:1752-1757)
    sel = np.concatenate([np.arange(b * bs, min((b + 1) * bs, n_rows)) for b in blocks]).astype(np.int32)
    q = c["q"][n_rows - 1]
    got = hip.gqa_decode_sel(cache, sel, q, c["scale"])
    ref = orc.gqa_decode(q, c["k"][sel], c["v"][sel], c["scale"])
    assert_close(got, ref, "gqa_decode_sel %d rows, %d positions" % (n_rows, sel.size))
    # entries that name no row carry no weight; the order of the list does not matter
    padded = np.concatenate([[-1, n_rows, -7], sel[::-1], [2 ** 31 - 1]]).astype(np.int32)
    got2 = hip.gqa_decode_sel(cache, padded, q, c["scale"])
    assert_close(got2, ref, "gqa_decode_sel padded and reversed")
    # the whole cache as a list equals the dense decode
    full = hip.gqa_decode_sel(cache, np.arange(n_rows, dtype=np.int32), q, c["scale"])
    dense = hip.gqa_decode(cache, n_rows, q, c["scale"])
    assert np.abs(full - dense).max() <= 1e-6
    # device operands
    d_sel = torch.from_numpy(sel).cuda()
    d_q = torch.from_numpy(q.view(np.int16)).cuda()
    d_out = torch.empty((nh, hd), dtype=torch.float32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    hip.gqa_decode_sel_dev(cache.k_dev(), cache.v_dev(), n_rows, nkv, hd, d_sel, sel.size, d_q, nh, c["scale"], d_out, s)
    torch.cuda.synchronize()
    assert np.array_equal(d_out.cpu().numpy().view(np.uint32), got.view(np.uint32))
    # nothing valid: zeros
    none = hip.gqa_decode_sel(cache, np.array([-1, -1, n_rows], np.int32), q, c["scale"])
    assert np.all(none == 0.0)
    cache.free()


@pytest.mark.parametrize("limit0,batch,ih,idim,bs,keep,max_sel", [
    (8192, 1, 4, 128, 128, 16, 4096),      # the reference's geometry (src/mm_model.c:1011-1012), a full last block
    (8000, 1, 4, 128, 128, 16, 4096),      # a partly filled newest block
    (1020, 8, 4, 128, 128, 3, 4096),       # a chunk whose queries cross a block border (1024)
    (70, 3, 1, 8, 7, 4, 64),
    (1, 2, 4, 128, 128, 16, 4096),         # the first positions of a sequence
    (40000, 2, 8, 64, 64, 20, 1000),       # the list cut at max_sel
    (300, 1, 2, 512, 128, 16, 4096),       # more blocks asked for than exist
    (70000, 1, 4, 128, 64, 16, 4096),      # more than 1024 blocks: the streaming row select inside the one-workgroup step
    (9000, 3, 4, 128, 192, 5, 4096),       # blocks of three scoring groups
    (45000, 2, 2, 64, 3, 16, 4096),        # 15000 blocks of a size the scoring groups do not divide: block maxima,
                                           # the many-workgroup top-k (its own workspace), expansion
])
def test_mm_select_blocks_on_device(hip, orc, limit0, batch, ih, idim, bs, keep, max_sel):
    """The block selection of the block-sparse decode (src/mm_model.c:1764-1780, :1733-1761,
    :1969-1976) for a chunk of consecutive queries: position scores bit for bit, the kept blocks
    and the position list equal to the oracle's."""
    import torch
    say("[case] mm select", limit0, batch, ih, idim, bs, keep, max_sel)
    g = synth.rng(limit0 + 31 * batch + ih)
    n = limit0 + batch - 1
    keys = synth.normal_bf16(g, (n, idim))
    iq = g.standard_normal((batch, ih, idim)).astype(np.float32)
    stride = n + 5
    d_keys = torch.from_numpy(keys.view(np.int16)).cuda()
    d_iq = torch.from_numpy(iq).cuda()
    d_sc = torch.full((batch, stride), float("nan"), dtype=torch.float32, device="cuda")
    d_blk = torch.full((batch, keep + 1), 77, dtype=torch.int32, device="cuda")
    d_sel = torch.full((batch, max_sel), 77, dtype=torch.int32, device="cuda")
    d_ns = torch.full((batch,), 77, dtype=torch.int32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    hip.mm_select_dev(d_keys, d_iq, batch, limit0, ih, idim, bs, keep, d_sc, stride, d_blk, d_sel, max_sel, d_ns, s)
    torch.cuda.synchronize()
    sc, blk, sel, ns = d_sc.cpu().numpy(), d_blk.cpu().numpy(), d_sel.cpu().numpy(), d_ns.cpu().numpy()
    for t in range(batch):
        limit = limit0 + t
        ref_sc = orc.mm_index_scores(iq[t], keys, limit)
        assert np.array_equal(sc[t, :limit].view(np.uint32), ref_sc.view(np.uint32)), "query %d: scores differ" % t
        assert np.isnan(sc[t, limit:]).all(), "query %d: scores written past the limit" % t
        rblk, rpos = orc.mm_select_blocks(ref_sc, limit, bs, keep, max_sel)
        assert list(blk[t, :rblk.size]) == list(rblk) and (blk[t, rblk.size:] == -1).all(), "query %d: blocks" % t
        assert ns[t] == rpos.size
        assert list(sel[t, :rpos.size]) == list(rpos) and (sel[t, rpos.size:] == -1).all(), "query %d: positions" % t
    # blk_out and n_sel may be left out
    d_sel2 = torch.full((batch, max_sel), 77, dtype=torch.int32, device="cuda")
    hip.mm_select_dev(d_keys, d_iq, batch, limit0, ih, idim, bs, keep, d_sc, stride, None, d_sel2, max_sel, None, s)
    torch.cuda.synchronize()
    assert torch.equal(d_sel, d_sel2)
    rc = hip.mm_select_dev(d_keys, d_iq, batch, limit0, 9, idim, bs, keep, d_sc, stride, None, d_sel2, max_sel, None, s,
                           raw=True)
    assert rc == 0 and "index heads" in hip.last_error()


@pytest.mark.parametrize("n_rows,nh,nkv,hd", [(5000, 64, 4, 128), (2304, 32, 2, 256)])
def test_mm_block_sparse_decode_chain(hip, orc, n_rows, nh, nkv, hd):
    """Selection and attention of the block-sparse decode chained on the device with nothing
    crossing to the host in between, sixteen query heads per kv head (the reference's 64/4,
    src/mm_model.c:1962-2047): against the oracle's selection and its decode over the gathered rows."""
    import torch
    say("[case] mm chain", n_rows, nh, nkv, hd)
    g = synth.rng(4100 + n_rows)
    ih, idim, bs, keep = 4, 128, 128, 16
    c = synth.cfg1_gqa_decode(n_rows, nh, nkv, hd, seed=4200 + n_rows)
    keys = synth.normal_bf16(g, (n_rows, idim))
    iq = g.standard_normal((1, ih, idim)).astype(np.float32)
    cache = hip.KVCache(n_rows, nkv, hd)
    cache.write(0, c["k"].reshape(n_rows, -1), c["v"].reshape(n_rows, -1))
    max_sel = (keep + 1) * bs
    d_keys = torch.from_numpy(keys.view(np.int16)).cuda()
    d_iq = torch.from_numpy(iq).cuda()
    d_sc = torch.empty((1, n_rows), dtype=torch.float32, device="cuda")
    d_sel = torch.empty((1, max_sel), dtype=torch.int32, device="cuda")
    d_q = torch.from_numpy(c["q"].view(np.int16)).cuda()
    d_out = torch.empty((nh, hd), dtype=torch.float32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    hip.mm_select_dev(d_keys, d_iq, 1, n_rows, ih, idim, bs, keep, d_sc, n_rows, None, d_sel, max_sel, None, s)
    hip.gqa_decode_sel_dev(cache.k_dev(), cache.v_dev(), n_rows, nkv, hd, d_sel, max_sel, d_q, nh, c["scale"], d_out, s)
    torch.cuda.synchronize()
    _, rpos = orc.mm_select_blocks(orc.mm_index_scores(iq[0], keys), n_rows, bs, keep, max_sel)
    sel = d_sel.cpu().numpy()[0]
    assert list(sel[:rpos.size]) == list(rpos)
    ref = orc.gqa_decode(c["q"], c["k"][rpos], c["v"][rpos], c["scale"])
    assert_close(d_out.cpu().numpy(), ref, "mm chain %d rows, %d positions, %d/%d heads" % (n_rows, rpos.size, nh, nkv))
    # the dense decode with sixteen heads per kv head
    dense = hip.gqa_decode(cache, n_rows, c["q"], c["scale"])
    assert_close(dense, orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"], nthreads=0), "gqa decode group 16")
    cache.free()


def test_mm_select_host_operands(hip, orc):
    """The block selection for an engine whose state is in host memory: index keys kept as the K
    side of a one-head cache handle, everything else host pointers, then the attention over the
    returned positions (src/mm_model.c:1962-2047)."""
    say("[case] mm select, host operands")
    n, ih, idim, bs, keep, nh, nkv, hd = 3000, 4, 128, 128, 16, 64, 4, 128
    g = synth.rng(5150)
    keys = synth.normal_bf16(g, (n, idim))
    iq = g.standard_normal((ih, idim)).astype(np.float32)
    idx = hip.KVCache(n, 1, idim)
    idx.write(0, keys, keys)
    for limit in (n, 2944, 1):                      # a partly filled newest block, a full one, a single position
        blk, pos = hip.mm_select(idx, limit, iq, bs, keep, 4096)
        rblk, rpos = orc.mm_select_blocks(orc.mm_index_scores(iq, keys, limit), limit, bs, keep, 4096)
        assert list(blk) == list(rblk) and list(pos) == list(rpos), limit
    blk, pos = hip.mm_select(idx, n, iq, bs, keep, 4096)
    c = synth.cfg1_gqa_decode(n, nh, nkv, hd, seed=5151)
    kv = hip.KVCache(n, nkv, hd)
    kv.write(0, c["k"].reshape(n, -1), c["v"].reshape(n, -1))
    got = hip.gqa_decode_sel(kv, pos.astype(np.int32), c["q"], c["scale"])
    ref = orc.gqa_decode(c["q"], c["k"][pos], c["v"][pos], c["scale"])
    assert_close(got, ref, "block-sparse decode, host operands, %d positions" % pos.size)
    with pytest.raises(hip.Declined):
        hip.mm_select(kv, n, iq, bs, keep, 4096)    # four heads per position: not an index-key cache
    idx.free()
    kv.free()


# ------------------------------------------------------------------ the GLM selector behind the pool scores
@pytest.mark.parametrize("n_comp,kp,topk,tail,strict,batch,kind", [
    (5, 4, 8, 0, False, 1, "traced"),          # the hand-traced case: the query's position twice
    (600, 4, 2048, 3, False, 3, "normal"),     # the GLM geometry (kpool 4, top-2048 -> 512 pools), a tail of three
    (600, 4, 2048, 0, False, 3, "normal"),     # no tail: the self rule decides
    (600, 4, 2048, 0, True, 2, "normal"),      # strict
    (20000, 4, 2048, 1, False, 2, "normal"),   # the many-workgroup top-k under it
    (3000, 1, 512, 0, False, 2, "ties"),       # kpool 1, ties at the threshold
    (300, 4, 2048, 2, False, 2, "normal"),     # no more pools than wanted: the whole prefix
    (5000, 8, 100, 5, False, 1, "last_high"),  # the last pool far above the threshold
])
def test_glm_select_on_device(hip, orc, n_comp, kp, topk, tail, strict, batch, kind):
    """The rest of indexer_select (src/attention.c:585-620) on the device: pools by the contract,
    the reference's list order, tail and self rule, against the oracle entry for entry; then the
    list straight into the sparse MLA decode."""
    import torch
    say("[case] glm select", n_comp, kp, topk, tail, strict, batch, kind)
    g = synth.rng(9100 + n_comp + tail)
    npos = n_comp * kp + tail
    want = (topk + kp - 1) // kp
    max_sel = (want + 1) * kp + 7
    if kind == "traced":
        sc = np.array([[3, 1, 4, 1, 5]], np.float32)
    elif kind == "ties":
        sc = g.integers(0, 40, (batch, n_comp)).astype(np.float32)
    else:
        sc = g.standard_normal((batch, n_comp), dtype=np.float32)
        if kind == "last_high":
            sc[:, -1] = 50.0
    d_sc = torch.from_numpy(sc).cuda()
    d_sel = torch.full((batch, max_sel), 77, dtype=torch.int32, device="cuda")
    d_n = torch.full((batch,), 77, dtype=torch.int32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    hip.glm_select_dev(d_sc, batch, n_comp, npos, kp, topk, strict, d_sel, max_sel, d_n, s)
    torch.cuda.synchronize()
    sel, ns = d_sel.cpu().numpy(), d_n.cpu().numpy()
    for b in range(batch):
        ref = orc.glm_select(sc[b], npos, kp, topk, strict=strict, faithful=False)
        if ref is None:
            assert ns[b] == -1 and list(sel[b, :npos]) == list(range(npos)) and (sel[b, npos:] == -1).all()
            continue
        assert ns[b] == ref.size, "query %d: %d positions, the oracle %d" % (b, ns[b], ref.size)
        assert list(sel[b, :ref.size]) == list(ref), "query %d" % b
        assert (sel[b, ref.size:] == -1).all()
        if kind == "traced":
            assert list(ref) == [16, 17, 18, 19, 8, 9, 10, 11, 19]
        took = len(orc.topk_quickselect(sc[b], want))
        if took == want:          # the reference's own threshold is the lowest of its top set: the same list
            assert list(orc.glm_select(sc[b], npos, kp, topk, strict=strict, faithful=True)) == list(ref)
    # the list as it stands into the sparse decode (a repeated position counts twice, as in the reference)
    if npos >= 64:
        c = synth.cfg3_mla_decode(npos, 128, seed=9200 + n_comp)
        rows, scales = torch.from_numpy(c["rows"]).cuda(), torch.from_numpy(c["scales"]).cuda()
        q = torch.from_numpy(np.repeat(c["q"][None], batch, 0).view(np.int16)).cuda()
        out = torch.empty((batch, 128, synth.VDIM), dtype=torch.float32, device="cuda")
        hip.mla_decode_dev(rows, scales, 0, 0, npos, batch, d_sel, max_sel, q, 128, c["scale"], out, s)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        for b in range(batch):
            ref = orc.glm_select(sc[b], npos, kp, topk, strict=strict, faithful=False)
            rsel = np.arange(npos, dtype=np.int32) if ref is None else ref
            want_out = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=rsel, nthreads=0)
            assert_close(got[b], want_out, "glm select -> sparse decode, query %d" % b)
    rc = hip.glm_select_dev(d_sc, batch, n_comp, npos + kp, kp, topk, strict, d_sel, max_sel, d_n, s, raw=True)
    assert rc == 0 and "pools" in hip.last_error()
    rc = hip.glm_select_dev(d_sc, batch, n_comp, npos, kp, topk, strict, d_sel, want * kp, d_n, s, raw=True)
    assert rc == 0 and "max_sel" in hip.last_error()
