"""Pins the CPU oracle (oracle/cwick_oracle.c) before anything trusts it.

Each oracle function is checked against evidence that does not share its
formula: closed forms, brute force in double precision, invariants of the
mathematics, the reference's own compiled object code (oracle/_ref, built from
/root/reference where present) and the golden vectors that object code wrote
(tests/golden/ref_vectors.npz, which travel where the reference cannot).
"""
import math
import os

import numpy as np
import pytest

from cwick_amd import synth

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


def bits(x):
    return np.asarray(x, np.float32).view(np.uint32)


# ------------------------------------------------------------------ E4M3
def e4m3_closed_form(b):
    """Independent of both reference decoders: exact rational arithmetic."""
    s, e, m = b >> 7, (b >> 3) & 15, b & 7
    if e == 15 and m == 7:
        return float("nan")
    v = m * 2.0 ** -9 if e == 0 else (8 + m) * 2.0 ** (e - 10)
    return -v if s else v


def test_e4m3_decode_all_256(orc, gold):
    lut = orc.e4m3_lut()
    for b in range(256):
        want = e4m3_closed_form(b)
        a = float(orc.lib().orc_e4m3_to_f32(b))
        if math.isnan(want):
            assert math.isnan(a) and math.isnan(lut[b])
        else:
            assert a == want and float(lut[b]) == want, b
    # landmarks the reference documents (src/tensor.c:344-353)
    assert lut[0x7E] == 448.0 and lut[0x07] == 0.013671875 and lut[0x08] == 2.0 ** -6
    assert np.isnan(lut[0x7F]) and np.isnan(lut[0xFF])
    # the reference's own object code, as golden vectors and (where built) live
    g = gold["e4m3_table"]
    assert np.array_equal(np.isnan(g), np.isnan(lut))
    assert np.array_equal(bits(g[~np.isnan(g)]), bits(lut[~np.isnan(lut)]))
    if orc.ref() is not None:
        for b in range(256):
            r = float(orc.ref().cwick_fp8_e4m3_to_f32(b))
            assert (math.isnan(r) and math.isnan(lut[b])) or r == float(lut[b])
    # numpy table used by the input generator
    t = synth.e4m3_table()
    assert np.array_equal(bits(t[~np.isnan(t)]), bits(lut[~np.isnan(lut)]))


def test_e4m3_encode_is_nearest_even(orc):
    lut = orc.e4m3_lut()
    grid = np.sort(lut[:0x7F].astype(np.float64))          # 0 .. 448, all finite positives
    g = synth.rng(1)
    xs = np.concatenate([
        g.uniform(-448, 448, 20000), g.standard_normal(20000) * 0.01,
        g.standard_normal(5000) * 1e-3, grid, -grid,
        (grid[:-1] + grid[1:]) / 2, -(grid[:-1] + grid[1:]) / 2,   # exact ties
        [0.0, -0.0, 448.0, -448.0, 2.0 ** -10, 2.0 ** -10 * 1.0001, 2.0 ** -11],
    ]).astype(np.float32)
    f = orc.lib().orc_f32_to_e4m3_rne
    enc = np.array([f(float(x)) for x in xs], np.uint8)
    dec = lut[enc].astype(np.float64)
    for x, b, d in zip(xs.astype(np.float64), enc, dec):
        a = abs(x)
        i = np.searchsorted(grid, a)
        cands = grid[max(i - 1, 0):i + 1]
        best = np.abs(cands - a).min()
        assert abs(abs(d) - a) <= best + 1e-300, (x, b, d)
        if len(cands) == 2 and abs(cands[0] - a) == abs(cands[1] - a):   # tie -> even mantissa
            assert (b & 1) == 0, (x, b)
        if a != 0 and d != 0:
            assert (d < 0) == (x < 0)
    # idempotence on every finite byte, saturation past 448
    for b in range(256):
        if not np.isnan(lut[b]) and (b & 0x7F) != 0:
            assert f(float(lut[b])) == b
    assert f(1e9) == 0x7E and f(-1e9) == 0xFE and f(449.0) == 0x7E
    # the input generator's numpy encoder agrees bit for bit
    assert np.array_equal(synth.f32_to_e4m3(xs), enc)
    # the reference's encoder as written (src/ds_quant.c:102-128) is the same function
    # except for the carry it loses just below 2^-6 (`mm & 7u`, :127)
    fr = orc.lib().orc_f32_to_e4m3
    ref_enc = np.array([fr(float(x)) for x in xs], np.uint8)
    differ = ref_enc != enc
    ax = np.abs(xs[differ])
    assert np.all((ax >= 0.0146484375) & (ax < 2.0 ** -6)) and np.all((ref_enc[differ] & 0x7F) == 0)
    assert fr(0.015623) == 0x00 and f(0.015623) == 0x08 and fr(-0.015623) == 0x80


def test_quantize_rows_numpy_equals_oracle(orc):
    g = synth.rng(2)
    x = g.standard_normal((64, 576), dtype=np.float32)
    x[3] = 0
    x[4, 128:256] = 0
    x[5] *= 1e-5
    q1, s1 = orc.quantize_rows_e4m3(x, 128)
    q2, s2 = synth.quantize_rows(x, 128)
    assert np.array_equal(q1, q2) and np.array_equal(bits(s1), bits(s2))
    assert s1.shape == (64, 5)
    # dequantised error is at most half a grid step of the block's scale
    lut = orc.e4m3_lut()
    deq = lut[q1] * np.repeat(s1, 128, axis=1)[:, :576]
    assert np.abs(deq - x).max() <= 0.0625 * np.abs(x).max() + 1e-12


# ------------------------------------------------------------------ bf16
def test_bf16(orc, gold):
    L = orc.lib()
    # tests/test_cwick.c:72-83 values and tolerance
    for v in [0.0, -0.0, 0.5, 1.0, 1.5, -2.0, 3.5, 123.25, 1e-5]:
        for enc in (L.orc_f32_to_bf16_rne, L.orc_f32_to_bf16_cwick):
            r = L.orc_bf16_to_f32(enc(v))
            assert abs(r - v) <= max(1e-3, abs(v) * 1e-2)
    g = synth.rng(3)
    xs = (g.standard_normal(5000) * 10).astype(np.float32)
    rne = np.array([L.orc_f32_to_bf16_rne(float(x)) for x in xs], np.uint16)
    assert np.array_equal(rne, synth.f32_to_bf16(xs))
    # RNE = nearest representable, ties to even
    lo = (bits(xs) & 0xFFFF0000).view(np.float32).astype(np.float64)
    hi = ((bits(xs) & 0xFFFF0000) + 0x10000).view(np.float32).astype(np.float64)
    got = synth.bf16_to_f32(rne).astype(np.float64)
    x64 = xs.astype(np.float64)
    assert np.all(np.abs(got - x64) <= np.minimum(np.abs(lo - x64), np.abs(hi - x64)))
    # cwick_f32_to_bf16 (src/util.c:202-210): golden from the reference's object code
    assert np.array_equal(
        np.array([L.orc_f32_to_bf16_cwick(float(x)) for x in gold["bf16_in"]], np.uint16),
        gold["bf16_cwick"])
    assert np.array_equal(
        bits([L.orc_bf16_round(float(x)) for x in gold["bf16_in"]]), bits(gold["bf16_round"]))


# ------------------------------------------------------------------ softmax
def test_softmax_closed_forms(orc, gold):
    n = 1000
    assert np.allclose(orc.softmax(np.full(n, 3.25, np.float32)), 1.0 / n, rtol=1e-6)
    x = np.zeros(50, np.float32)
    x[7] = 100.0
    p = orc.softmax(x)
    assert p[7] == 1.0 and p.sum() == 1.0
    g = synth.rng(4)
    x = (g.standard_normal(4096) * 3).astype(np.float32)
    p = orc.softmax(x)
    ref = np.exp(x.astype(np.float64) - x.max())
    ref /= ref.sum()
    assert np.abs(p - ref).max() < 1e-7
    assert np.abs(orc.softmax(x + np.float32(5.0)) - p).max() < 1e-6       # shift invariance
    t = x.copy()
    t[100:] = -1e30                                                        # the causal-tail trick
    pt = orc.softmax(t)
    assert np.all(pt[100:] == 0.0) and np.array_equal(bits(pt[:100]), bits(orc.softmax(x[:100])))
    # bit-exact against the reference's own cwick_softmax / ds_softmax
    assert np.array_equal(bits(orc.softmax(gold["softmax_in"])), bits(gold["softmax_out"]))
    assert np.array_equal(bits(orc.softmax(gold["softmax_in"])), bits(gold["ds_softmax_out"]))


# ------------------------------------------------------------------ top-k
KNOWN = [
    ([5, 5, 7], 2, [0, 2], [1, 2]),
    ([3, 9, 3, 3, 8, 3], 4, [0, 1, 2, 4], [1, 2, 3, 4]),
    ([1, 1, 1, 1, 1], 3, [0, 1, 2], None),
    ([2, 1], 5, [0, 1], None),
    ([0.0, -0.0, 1.0, -0.0], 3, [0, 1, 2], None),
    ([-np.inf, 1, -np.inf, 2], 3, [0, 1, 3], None),
]


@pytest.mark.parametrize("sc,k,contract,heap", KNOWN)
def test_topk_known_answers(orc, sc, k, contract, heap):
    sc = np.array(sc, np.float32)
    assert list(orc.topk_contract(sc, k)) == contract
    if k < len(sc):
        assert set(orc.topk_quickselect(sc, k)) <= set(contract)
    if heap is not None:
        # the heap of src/ds_ops.c:310-338 does NOT keep the lower index on these
        assert list(orc.topk_heap(sc, k)) == heap
        if orc.ref() is not None:
            assert list(orc.ref_topk_scores(sc, k)) == heap


# Known answers of the GLM selector, traced by hand through src/attention.c:529-543
# (score_select: Hoare partition around v[(lo+hi)>>1], `k <= j -> hi = j`, `k >= i -> lo = i`,
# else stop) and :588-598 (thr = copy[want-1]; all `> thr` in index order, then `== thr`).
# State of the copy after every partition round:
#   [1,5,2,4,3] want 3: pivot 2 -> [3,5,4,2,1] (i 3, j 2, lo = 3); pivot 2 -> same (i 4, j 2, stop);
#       thr = copy[2] = 4 -> takes 5 and 4 only: the 3 is lost (copy[3] = 2 would take all three)
#   [5,3,4,1,2] want 3: pivot 4 -> [5,4,3,1,2] (lo = 2); pivot 1 -> [5,4,3,2,1] (hi = 3);
#       pivot 3 -> same (lo = 3); thr = 3 -> `> 3`: indices 0, 2, then `== 3`: index 1
#   [3,1,4,1,5] want 2: pivot 4 -> [5,4,1,1,3] (lo = 2); pivot 1 -> [5,4,3,1,1] (hi = 2);
#       thr = 4 -> index 4, then index 2
#   [2,2,1,2,3] want 2: pivot 1 -> [2,2,3,2,1] (hi = 3); pivot 2 -> [2,3,2,2,1] (lo = 2);
#       pivot 2 -> same (hi = 2); thr = copy[1] = 3 -> index 4 alone (the contract: 0 and 4)
QUICKSELECT_TRACED = [
    ([1, 5, 2, 4, 3], 3, [1, 3]),
    ([5, 3, 4, 1, 2], 3, [0, 2, 1]),
    ([3, 1, 4, 1, 5], 2, [4, 2]),
    ([2, 2, 1, 2, 3], 2, [4]),
]


@pytest.mark.parametrize("sc,want,traced", QUICKSELECT_TRACED)
def test_topk_quickselect_hand_traced(orc, sc, want, traced):
    sc = np.array(sc, np.float32)
    assert list(orc.topk_quickselect(sc, want)) == traced
    # reading the threshold one place later (copy[want]) would give the contract's set on the
    # first and the last case: the traced answers tell the two apart
    assert set(traced) <= set(int(i) for i in orc.topk_contract(sc, want))


# The rest of indexer_select (src/attention.c:585-620) on the score vectors traced above, by hand:
# pools -> positions c*kp + r in the reference's order (`> thr` ascending, then `== thr`), the tail
# npos % kp, then npos - 1 unless it is the LAST entry already (:618 looks at sel[n-1] only, so a
# selected last pool that is not the threshold pool is followed by a second copy of npos - 1).
#   (sc, kp, topk, npos, strict) -> faithful list, contract-choice list (None: the same)
GLM_SELECT_TRACED = [
    # want 3; the reference takes pools 1, 3 only (under-selection), the contract 1, 3 then 4 (== thr 3)
    ([1, 5, 2, 4, 3], 2, 6, 10, False, [2, 3, 6, 7, 9], [2, 3, 6, 7, 8, 9]),          # no tail; self pruned / self last already
    ([1, 5, 2, 4, 3], 2, 6, 11, False, [2, 3, 6, 7, 10], [2, 3, 6, 7, 8, 9, 10]),      # tail of one position, which is the query
    ([1, 5, 2, 4, 3], 2, 5, 10, True, [2, 3, 6, 7], [2, 3, 6, 7, 8, 9]),               # topk 5 -> want 3 as well; strict
    # want 3; both take pools 0, 2 (> 3) then 1 (== 3)
    ([5, 3, 4, 1, 2], 2, 5, 10, False, [0, 1, 4, 5, 2, 3, 9], None),                   # self pruned: appended
    ([5, 3, 4, 1, 2], 2, 5, 10, True, [0, 1, 4, 5, 2, 3], None),
    # want 2, kp 4: pool 4 (> 4) then pool 2 (== 4); the last pool is selected but not last in the list
    ([3, 1, 4, 1, 5], 4, 8, 20, False, [16, 17, 18, 19, 8, 9, 10, 11, 19], None),      # the query twice
    ([3, 1, 4, 1, 5], 4, 8, 22, False, [16, 17, 18, 19, 8, 9, 10, 11, 20, 21], None),  # tail of two, the query among them
    ([3, 1, 4, 1, 5], 1, 2, 5, False, [4, 2, 4], None),                                # kp 1
    ([3, 1, 4, 1, 5], 1, 2, 5, True, [4, 2], None),
]


@pytest.mark.parametrize("sc,kp,topk,npos,strict,faithful,contract", GLM_SELECT_TRACED)
def test_glm_select_hand_traced(orc, sc, kp, topk, npos, strict, faithful, contract):
    sc = np.array(sc, np.float32)
    assert list(orc.glm_select(sc, npos, kp, topk, strict=strict, faithful=True)) == faithful
    assert list(orc.glm_select(sc, npos, kp, topk, strict=strict, faithful=False)) == (contract or faithful)


def test_glm_select_whole_prefix_and_agreement(orc):
    # no more pools than wanted: "the whole prefix" (src/attention.c:558-559)
    assert orc.glm_select(np.array([1, 2], np.float32), 9, 4, 8) is None
    assert orc.glm_select(np.array([1, 2, 3], np.float32), 6, 2, 6, faithful=True) is None
    # tie-free scores: whenever the reference's threshold is the smallest of its top set the two
    # pool choices give the same list, entry for entry
    g = synth.rng(77)
    same = 0
    for _ in range(300):
        n_comp, kp = int(g.integers(5, 60)), int(g.integers(1, 5))
        topk = int(g.integers(1, (n_comp - 1) * kp))
        npos = n_comp * kp + int(g.integers(0, kp))
        sc = g.permutation(n_comp).astype(np.float32)
        a = orc.glm_select(sc, npos, kp, topk, faithful=True)
        b = orc.glm_select(sc, npos, kp, topk, faithful=False)
        want = (topk + kp - 1) // kp
        took = len(orc.topk_quickselect(sc, want))
        if took == want:
            assert list(a) == list(b)
            same += 1
        else:
            assert set(a) <= set(b) | {npos - 1}
    assert same > 50


def brute_topk(sc, k):
    order = sorted(range(len(sc)), key=lambda i: (-float(sc[i]), i))
    return sorted(order[:min(k, len(sc))])


def test_topk_contract_vs_brute_force(orc):
    g = synth.rng(5)
    for n, k in [(1, 1), (17, 5), (100, 100), (100, 7), (1000, 64), (513, 512)]:
        for kind in range(3):
            if kind == 0:
                sc = g.standard_normal(n).astype(np.float32)
            elif kind == 1:
                sc = g.integers(-3, 3, n).astype(np.float32)
            else:
                sc = np.where(g.random(n) < 0.5, -np.inf, g.integers(0, 4, n)).astype(np.float32)
            want = brute_topk(sc, k)
            assert list(orc.topk_contract(sc, k)) == want
            # the GLM selector (src/attention.c:585-598) takes `> thr` then `== thr` in
            # index order, so what it takes follows the same rule -- but its threshold is
            # v[want-1] after a quickselect that only fixes position `want`
            # (src/attention.c:529-543), i.e. some member of the top set rather than
            # its minimum, so it may take fewer than `want`: always a subset.
            if k < n:
                qs = list(orc.topk_quickselect(sc, k))
                assert set(qs) <= set(want) and len(qs) == len(set(qs)) >= 1
                lo = min(float(sc[i]) for i in qs)
                assert all(float(sc[i]) <= lo for i in range(n) if i not in qs)
            # the heap agrees whenever no tie straddles the k-th value
            if kind == 0:
                assert list(orc.topk_heap(sc, k)) == want


def test_topk_heap_golden(orc, gold):
    """orc_topk_heap against ds_topk_scores compiled from the reference, ties included."""
    n_cases = int(gold["topk_ncases"])
    for c in range(n_cases):
        sc, k, want = gold["topk_sc_%d" % c], int(gold["topk_k_%d" % c]), gold["topk_out_%d" % c]
        assert np.array_equal(orc.topk_heap(sc, k), want), c
        if orc.ref() is not None:
            assert np.array_equal(orc.ref_topk_scores(sc, k), want)


def test_order_key_is_monotone(orc):
    f = orc.lib().orc_topk_order_key
    vals = [-np.inf, -3.0, -1e-30, -0.0, 0.0, 1e-30, 2.0, np.inf]
    keys = [f(float(v)) for v in vals]
    assert keys[3] == keys[4]
    ks = keys[:3] + keys[4:]
    assert all(a < b for a, b in zip(ks, ks[1:]))
    assert f(float("nan")) == 0 < keys[0]


# ------------------------------------------------------------------ dots
def test_dot_f32_order(orc):
    # (s0+s1)+(s2+s3) with s_j over i = j mod 4: a case where the order shows
    a = np.array([1e8, 1.0, -1e8, 1.0, 1.0, 1.0, 1.0, 1.0, 3.0], np.float32)
    b = np.ones(9, np.float32)
    s0 = np.float32(np.float32(np.float32(1e8) + np.float32(1.0)) + np.float32(3.0))
    s1, s2, s3 = np.float32(2.0), np.float32(np.float32(-1e8) + np.float32(1.0)), np.float32(2.0)
    want = np.float32(np.float32(s0 + s1) + np.float32(s2 + s3))
    assert orc.dot_f32(a, b) == float(want)
    g = synth.rng(6)
    x, y = g.standard_normal(576).astype(np.float32), g.standard_normal(576).astype(np.float32)
    assert abs(orc.dot_f32(x, y) - float(x.astype(np.float64) @ y.astype(np.float64))) < 1e-3


# ------------------------------------------------------------------ MiniMax block selection
def _bf16(x):
    return synth.f32_to_bf16(np.asarray(x, np.float32))


def test_mm_index_scores_known_answers(orc):
    """src/mm_model.c:1764-1780.  Each case fails for one plausible mistake."""
    one = _bf16([1.0])[0]
    # fused multiply-add: the low bit of the second product survives only when it is not rounded
    # before the addition (multiply-then-add gives 0)
    q = np.array([[-(1.0 + 2.0 ** -7 + 2.0 ** -23), 1.0 + 2.0 ** -23]], np.float32)
    k = np.array([[one, _bf16([1.0 + 2.0 ** -7])[0]]], np.uint16)
    assert orc.mm_index_scores(q, k)[0] == np.float32(2.0 ** -30)
    # serial order from zero: 2^24 + 1 + 1 stays 2^24, then -2^24 + 4 leaves 4 (pairwise 5, exact 6)
    q = np.array([[2.0 ** 24, 1.0, 1.0, -(2.0 ** 24) + 4.0]], np.float32)
    k = np.full((1, 4), one, np.uint16)
    assert orc.mm_index_scores(q, k)[0] == np.float32(4.0)
    # ReLU per head before the sum, heads added in head order, no weights
    q = np.array([[2.0 ** 24], [-5.0], [1.0]], np.float32)
    k = np.array([[one]], np.uint16)
    assert orc.mm_index_scores(q, k)[0] == np.float32(2.0 ** 24)
    q = np.array([[1.0], [1.0], [2.0 ** 24]], np.float32)
    assert orc.mm_index_scores(q, k)[0] == np.float32(2.0 ** 24 + 2.0)
    # the key is bf16 bits widened by a shift; a negative dot scores zero
    k = np.array([[0xC000], [0x3F80], [0x4040]], np.uint16)             # -2, 1, 3
    q = np.array([[1.5]], np.float32)
    assert list(orc.mm_index_scores(q, k)) == [0.0, 1.5, 4.5]
    # only the first `limit` positions are scored
    assert orc.mm_index_scores(q, k, limit=2).shape == (2,)


def test_mm_index_scores_vs_double(orc):
    g = synth.rng(81)
    for n, ih, idim in [(300, 4, 128), (17, 1, 8), (64, 8, 64)]:
        q = g.standard_normal((ih, idim)).astype(np.float32)
        kb = synth.normal_bf16(g, (n, idim))
        kf = synth.bf16_to_f32(kb).astype(np.float64)
        want = np.maximum(kf @ q.astype(np.float64).T, 0.0).sum(axis=1)
        got = orc.mm_index_scores(q, kb)
        assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max())


def test_mm_select_blocks_known_answers(orc):
    """Traced by hand through src/mm_model.c:1733-1761 and :1969-1976 (block size 4)."""
    a = np.array([0.1, 0.9, 0.2, 0.3, 0.5, 0.4, 0.6, 0.2, 0.05, 0.07], np.float32)
    # block maxima 0.9, 0.6, 0.07; two kept: 0 and 1; the newest block, 10 / 4 = 2, is added
    blk, pos = orc.mm_select_blocks(a, 10, 4, 2)
    assert list(blk) == [0, 1, 2] and list(pos) == list(range(10))
    # a limit that is a multiple of the block size: the added block is 8 / 4 = 2, which holds no
    # written position, so the list is block 0 alone (positions 4..7 are NOT attended)
    blk, pos = orc.mm_select_blocks(a, 8, 4, 1)
    assert list(blk) == [0, 2] and list(pos) == [0, 1, 2, 3]
    # the newest block already among the kept ones: nothing is added
    b = a.copy(); b[8] = 5.0
    blk, pos = orc.mm_select_blocks(b, 10, 4, 2)
    assert list(blk) == [0, 2] and list(pos) == [0, 1, 2, 3, 8, 9]
    # at most max_sel positions, cut in block order
    blk, pos = orc.mm_select_blocks(a, 10, 4, 2, max_sel=6)
    assert list(blk) == [0, 1, 2] and list(pos) == [0, 1, 2, 3, 4, 5]
    # more blocks asked for than exist
    blk, pos = orc.mm_select_blocks(a, 10, 4, 5)
    assert list(blk) == [0, 1, 2] and list(pos) == list(range(10))
    # a single position
    blk, pos = orc.mm_select_blocks(a, 1, 4, 2)
    assert list(blk) == [0] and list(pos) == [0]
    # scores past the limit are not read: block 1's 0.6 at position 6 is outside limit 6
    blk, pos = orc.mm_select_blocks(a, 6, 4, 1)
    assert list(blk) == [0, 1] and list(pos) == [0, 1, 2, 3, 4, 5]


def test_mm_select_blocks_vs_brute_force(orc):
    g = synth.rng(82)
    for limit, bs, keep in [(1000, 128, 3), (4096, 128, 16), (4097, 128, 16), (70, 7, 4), (129, 128, 16), (5000, 64, 20)]:
        sc = np.abs(g.standard_normal(limit)).astype(np.float32)
        nblk = -(-limit // bs)
        bmax = np.array([sc[b * bs:min((b + 1) * bs, limit)].max() for b in range(nblk)])
        assert len(set(bmax.tolist())) == nblk                          # tie-free
        want = set(np.argsort(-bmax, kind="stable")[:keep].tolist()) | {limit // bs}
        blk, pos = orc.mm_select_blocks(sc, limit, bs, keep, max_sel=1 << 20)
        assert list(blk) == sorted(want)
        wpos = [s for b in sorted(want) for s in range(b * bs, min((b + 1) * bs, limit))]
        assert list(pos) == wpos
