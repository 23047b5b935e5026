"""Pins the attention functions of the CPU oracle with mathematics that a plausible
mistake (a dropped term, a wrong sign or index, a transposed operand, a wrong head
map, an off-by-one in the causal limit) would break: brute force in double precision
written independently in numpy, and the identities the reference itself relies on."""
import numpy as np
import pytest

from cwick_amd import synth


def f32(b):
    return synth.bf16_to_f32(b).astype(np.float64)


def softmax64(s, axis=-1):
    s = s - s.max(axis=axis, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=axis, keepdims=True)


def dequant(rows, scales, lut):
    return lut[rows].astype(np.float64) * np.repeat(scales.astype(np.float64), 128, axis=1)[:, :rows.shape[1]]


# ------------------------------------------------------------------ GQA
def brute_gqa(q, k, v, scale, limit=None):
    """q [nh,hd], k/v [keys,nkv,hd] float64; head h reads kv head h // group."""
    nh, hd = q.shape
    keys, nkv, _ = k.shape
    group = nh // nkv
    out = np.zeros((nh, hd))
    n = keys if limit is None else limit
    for h in range(nh):
        g = h // group
        p = softmax64(scale * (k[:n, g] @ q[h]))
        out[h] = p @ v[:n, g]
    return out


@pytest.mark.parametrize("keys,nh,nkv,hd", [(300, 16, 4, 256), (1, 4, 4, 64), (97, 8, 2, 128)])
def test_gqa_decode_vs_brute_force(orc, keys, nh, nkv, hd):
    c = synth.cfg1_gqa_decode(keys, nh, nkv, hd, seed=keys)
    got = orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"])
    want = brute_gqa(f32(c["q"]), f32(c["k"]), f32(c["v"]), c["scale"])
    assert np.abs(got - want).max() < 2e-5
    # slicing and threading only reorder the fp32 sums
    for ns, nt in [(1, 1), (7, 3), (16, 0)]:
        assert np.abs(orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"], ns, nt) - want).max() < 2e-5


def test_gqa_decode_attnbench_inputs(orc):
    """The deterministic fixture of tools/attnbench.c:142-149."""
    keys, nkv, hd, nh = 257, 4, 256, 16
    i = np.arange(keys * nkv * hd, dtype=np.int64)
    kf = ((i * 37) % 101 - 50).astype(np.float32) * np.float32(0.02)
    k = (kf.view(np.uint32) >> 16).astype(np.uint16).reshape(keys, nkv, hd)      # truncation, as there
    v = synth.f32_to_bf16(((i * 13) % 89 - 44).astype(np.float32) * np.float32(0.01)).reshape(keys, nkv, hd)
    j = np.arange(nh * hd, dtype=np.int64)
    q = synth.f32_to_bf16(((j * 17) % 67 - 33).astype(np.float32) * np.float32(0.03)).reshape(nh, hd)
    got = orc.gqa_decode(q, k, v, 0.0625)
    assert np.abs(got - brute_gqa(f32(q), f32(k), f32(v), 0.0625)).max() < 2e-5


@pytest.mark.parametrize("pos0,n", [(0, 150), (37, 40)])
def test_gqa_prefill_vs_brute_force_and_decode(orc, pos0, n):
    nh, nkv, hd = 8, 2, 64
    c = synth.cfg2_gqa_prefill(n, nh, nkv, hd, pos0, seed=n)
    got = orc.gqa_prefill(c["q"], c["k"], c["v"], pos0, c["scale"], tile_q=64)
    q, k, v = f32(c["q"]), f32(c["k"]), f32(c["v"])
    for t in range(n):
        want = brute_gqa(q[t], k, v, c["scale"], limit=pos0 + t + 1)
        assert np.abs(got[t] - want).max() < 2e-5, t
    # prefill row t == decode at position pos0+t (the reference runs either, n == 1 or not)
    for t in (0, n // 2, n - 1):
        dec = orc.gqa_decode(c["q"][t], c["k"][:pos0 + t + 1], c["v"][:pos0 + t + 1], c["scale"])
        assert np.abs(got[t] - dec).max() < 2e-5
    # the -1e30 rectangle equals the triangle: tile size must not matter
    other = orc.gqa_prefill(c["q"], c["k"], c["v"], pos0, c["scale"], tile_q=7, nthreads=0)
    assert np.abs(got - other).max() < 2e-5
    # tile sub-sampling touches only the chosen tiles
    part = orc.gqa_prefill(c["q"], c["k"], c["v"], pos0, c["scale"], tile_q=16, tiles=(1, 0, 3))
    for tile in range((n + 15) // 16):
        rows = slice(tile * 16, min(n, tile * 16 + 16))
        if tile >= 1 and (tile - 1) % 3 == 0:
            assert np.abs(part[rows] - got[rows]).max() < 2e-5
        else:
            assert not part[rows].any()


# ------------------------------------------------------------------ MLA
def brute_mla(q, lat, scale, sel=None):
    """q [nh,576] f64, lat [rows,576] f64: K = all 576 dims, V = first 512."""
    rows = lat if sel is None else lat[[t for t in sel if t >= 0]]
    p = softmax64(scale * (q @ rows.T), axis=1)
    return p @ rows[:, :512]


@pytest.mark.parametrize("n,nh", [(1, 4), (200, 16), (1000, 128)])
def test_mla_decode_vs_brute_force(orc, n, nh):
    c = synth.cfg3_mla_decode(n, nh, seed=n)
    lut = orc.e4m3_lut()
    lat = dequant(c["rows"], c["scales"], lut)
    want = brute_mla(f32(c["q"]), lat, c["scale"])
    got = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"])
    assert np.abs(got - want).max() < 1e-5
    assert np.abs(orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=0) - want).max() < 1e-5
    # dense == sel = 0..n-1, bit for bit (same order of operations)
    same = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=np.arange(n, dtype=np.int32))
    assert np.array_equal(got.view(np.uint32), same.view(np.uint32))


def test_mla_decode_sel_gather_and_padding(orc):
    n, nh = 700, 32
    c = synth.cfg3_mla_decode(n, nh, seed=5)
    lat = dequant(c["rows"], c["scales"], orc.e4m3_lut())
    g = synth.rng(6)
    sel = g.permutation(n)[:256].astype(np.int32)
    want = brute_mla(f32(c["q"]), lat, c["scale"], sel)
    got = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=sel)
    assert np.abs(got - want).max() < 1e-5
    # softmax is order-free: a permuted list changes only rounding
    assert np.abs(orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=np.sort(sel)) - want).max() < 1e-5
    # -1 slots contribute nothing (src/ds_model.c:929/:940/:950)
    padded = np.concatenate([sel[:100], [-1, -1], sel[100:], [-1]]).astype(np.int32)
    assert np.abs(orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=padded) - want).max() < 1e-5
    assert not orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"],
                              sel=np.full(4, -1, np.int32)).any()


def test_mla_absorption_identity(orc):
    """The check the reference runs on itself (src/attention.c:838-893): the absorbed
    form over the latent equals classic attention over k_t = W_k c_t, v_t = W_v c_t."""
    g = synth.rng(7)
    nh, dim, nope, vdim, n = 4, 32, 16, 24, 50
    lat = g.standard_normal((n, dim)).astype(np.float32)
    q = g.standard_normal((nh, nope)).astype(np.float32)
    wk = g.standard_normal((nh, nope, dim)).astype(np.float32)
    wv = g.standard_normal((nh, vdim, dim)).astype(np.float32)
    scale = 1.0 / np.sqrt(nope)
    q_abs = np.einsum("hi,hic->hc", q, wk).astype(np.float32)             # :741-744
    c_acc = orc.mla_decode_f32(q_abs, lat, scale)
    absorbed = np.einsum("hvc,hc->hv", wv.astype(np.float64), c_acc.astype(np.float64))   # :812-815
    for h in range(nh):
        k = lat.astype(np.float64) @ wk[h].astype(np.float64).T
        v = lat.astype(np.float64) @ wv[h].astype(np.float64).T
        p = softmax64(scale * (k @ q[h].astype(np.float64)))
        assert np.abs(absorbed[h] - p @ v).max() < 1e-4


def test_mla_prefill_is_a_loop_of_decodes(orc):
    pos0, n, nh = 90, 20, 16
    c = synth.cfg4_mla_prefill(n, pos0, nh, seed=8)
    got = orc.mla_prefill_chunk(c["q"], c["rows"], c["scales"], pos0, c["scale"])
    lat = dequant(c["rows"], c["scales"], orc.e4m3_lut())
    for t in range(n):
        dec = orc.mla_decode(c["q"][t], c["rows"], c["scales"], c["scale"], nlist=pos0 + t + 1)
        assert np.array_equal(got[t].view(np.uint32), dec.view(np.uint32))
        want = brute_mla(f32(c["q"][t]), lat[:pos0 + t + 1], c["scale"])
        assert np.abs(got[t] - want).max() < 1e-5
    part = orc.mla_prefill_chunk(c["q"], c["rows"], c["scales"], pos0, c["scale"], queries=(2, 0, 5))
    for t in range(n):
        if t >= 2 and (t - 2) % 5 == 0:
            assert np.array_equal(part[t], got[t])
        else:
            assert not part[t].any()


# ------------------------------------------------------------------ indexer
def test_indexer_scores_vs_brute_force(orc):
    g = synth.rng(9)
    n, ih = 500, 64
    keys, ks = synth.index_keys(g, n)
    q = synth.normal_bf16(g, (ih, 128))
    w = (g.standard_normal(ih) / np.sqrt(128.0 * ih)).astype(np.float32)
    got = orc.indexer_scores(q, w, keys, ks)
    lut = orc.e4m3_lut().astype(np.float64)
    d = (lut[keys] * ks[:, None].astype(np.float64)) @ f32(q).T           # [n, ih]
    want = (np.maximum(d, 0.0) * w.astype(np.float64)).sum(axis=1)        # ReLU BEFORE the weight
    assert np.abs(got - want).max() < 1e-5
    wrong = np.maximum(d * w.astype(np.float64), 0.0).sum(axis=1)         # ReLU after: a different function
    assert np.abs(got - wrong).max() > 1e-2
    # threads do not change a single bit (each key's sum is private)
    assert np.array_equal(got.view(np.uint32), orc.indexer_scores(q, w, keys, ks, nthreads=0).view(np.uint32))
    # a positive per-token scale commutes with the ReLU: scaling a key's scale by 4
    # (exact in fp32) scales its score by 4
    ks2 = ks.copy()
    ks2[10] *= np.float32(4.0)
    assert orc.indexer_scores(q, w, keys, ks2)[10] == np.float32(4.0) * got[10]


# ------------------------------------------------------------------ DeepSeek flavours
def test_sparse_attn_sink_vs_brute_force(orc):
    """ds_sparse_attn_heads (src/ds_model.c:917-966): the sink joins the denominator and nothing
    else.  Brute force in double; the closed form for a single key; sink = -inf reduces to the
    plain sparse decode; -1 entries are skipped; a wrong sign, a sink added to the numerator or
    a sink scaled like a score would each fail one of these."""
    n_rows, nh = 400, 12
    c = synth.cfg3_mla_decode(n_rows, nh, seed=41)
    lut = orc.e4m3_lut()
    lat = dequant(c["rows"], c["scales"], lut)
    g = synth.rng(42)
    sel = g.permutation(n_rows)[:150].astype(np.int32)
    sel[[4, 77]] = -1
    sink = g.standard_normal(nh).astype(np.float32) * 2.0
    got = orc.sparse_attn_sink(c["q"], c["rows"], c["scales"], c["scale"], sink=sink, sel=sel)
    live = sel[sel >= 0]
    q = f32(c["q"])
    s = c["scale"] * (q @ lat[live].T)                                 # [nh, n]
    m = s.max(axis=1, keepdims=True)
    e = np.exp(s - m)
    den = e.sum(axis=1) + np.exp(sink.astype(np.float64) - m[:, 0])
    want = (e @ lat[live][:, :512]) / den[:, None]
    assert np.abs(got - want).max() < 2e-5
    # without the sink the denominators differ visibly on this data (the test has teeth)
    assert np.abs(want - (e @ lat[live][:, :512]) / e.sum(axis=1)[:, None]).max() > 1e-3
    # sink = -inf: the plain sparse decode
    no = orc.sparse_attn_sink(c["q"], c["rows"], c["scales"], c["scale"],
                              sink=np.full(nh, -np.inf, np.float32), sel=sel)
    plain = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], sel=sel)
    assert np.abs(no - plain).max() < 2e-5
    assert np.array_equal(no, orc.sparse_attn_sink(c["q"], c["rows"], c["scales"], c["scale"], sel=sel))
    # one key: out = v / (1 + exp(sink - score))
    one = orc.sparse_attn_sink(c["q"], c["rows"], c["scales"], c["scale"], sink=sink,
                               sel=np.array([7], np.int32))
    s7 = c["scale"] * (q @ lat[7])
    assert np.abs(one - lat[7][None, :512] / (1.0 + np.exp(sink - s7))[:, None]).max() < 2e-5
    # nothing selected: zeros, as `oh[i] = 0` times 1/inf gives (src/ds_model.c:947-958)
    none = orc.sparse_attn_sink(c["q"], c["rows"], c["scales"], c["scale"], sink=sink,
                                sel=np.array([-1, -1], np.int32))
    assert np.array_equal(none, np.zeros_like(none))


def test_indexer_scores_ds_roundings(orc):
    """ds_indexer's loop (src/ds_model.c:1099-1121): the dot is rounded to bf16 before the ReLU,
    the weight is rounded to bf16, the dot is serial.  Each known answer below separates one of
    these from the GLM flavour."""
    hd = 128
    lut = orc.e4m3_lut()
    one = int(np.where(lut == 1.0)[0][0]); v1125 = int(np.where(lut == 1.125)[0][0])

    def run(qrow, keyrow, ks, w):
        q = synth.f32_to_bf16(np.asarray(qrow, np.float32)[None, :])
        return float(orc.indexer_scores_ds(q, np.array([w], np.float32), np.asarray(keyrow, np.uint8)[None, :],
                                           np.array([ks], np.float32))[0])
    # (1) the dot is rounded to bf16: 1.125 * (1 + 2^-8) = 1.12939453125 -> 1.1328125 (145/128)
    q = np.zeros(hd); q[0] = 1.0
    k = np.zeros(hd, np.uint8); k[0] = v1125
    assert run(q, k, 1.0 + 2.0 ** -8, 1.0) == 1.1328125
    # (2) the weight is rounded to bf16: 1 + 2^-9 rounds to 1 (ties to even), 1 + 3 * 2^-9 to 1 + 2^-7
    k[0] = one
    assert run(q, k, 1.0, 1.0 + 2.0 ** -9) == 1.0
    assert run(q, k, 1.0, 1.0 + 3 * 2.0 ** -9) == 1.0 + 2.0 ** -7
    # (3) the ReLU comes after the rounding and before the weight: a negative dot contributes nothing
    q[0] = -1.0
    assert run(q, k, 1.0, -5.0) == 0.0
    # (4) serial order: 2^24 + 1 + 1 + 1 + 1 - 2^24 is 0 added one by one (each 1 is lost) and 4 when
    #     the four partial lanes of dot_f32 are used; the bf16 rounding keeps both exactly
    q = np.zeros(hd); k = np.zeros(hd, np.uint8)
    q[0] = 2.0 ** 24; q[1:5] = 1.0; q[5] = -2.0 ** 24
    k[:6] = one
    assert run(q, k, 1.0, 1.0) == 0.0
    glm = float(orc.indexer_scores(synth.f32_to_bf16(np.asarray(q, np.float32)[None, :]), np.array([1.0], np.float32),
                                   k[None, :], np.array([1.0], np.float32))[0])
    assert glm != 0.0


def test_indexer_scores_ds_vs_brute_force(orc):
    g = synth.rng(43)
    n, ih = 500, 32
    keys, ks = synth.index_keys(g, n)
    q = synth.normal_bf16(g, (ih, 128))
    w = (g.standard_normal(ih) / np.sqrt(128.0 * ih)).astype(np.float32)
    got = orc.indexer_scores_ds(q, w, keys, ks)
    lut = orc.e4m3_lut().astype(np.float64)
    kt = lut[keys] * ks.astype(np.float64)[:, None]
    d = kt @ f32(q).T                                                    # [n, ih]
    wb = synth.bf16_to_f32(synth.f32_to_bf16(w)).astype(np.float64)
    want = (np.maximum(d, 0.0) * wb[None, :]).sum(axis=1)
    # the bf16 rounding of every dot (2^-9 relative) dominates the error
    bound = (np.abs(d) * np.abs(wb)[None, :]).sum(axis=1) * 2.0 ** -8 + 1e-6
    assert (np.abs(got - want) <= bound).all()
    assert np.abs(got - want).max() > 1e-5            # ... and is really there
    # threads only split the keys
    assert np.array_equal(got, orc.indexer_scores_ds(q, w, keys, ks, nthreads=0))


# ------------------------------------------------------------------ the steps around the kernels
def test_mla_absorb_expand_vs_brute_force(orc):
    """gemv_bf16_t / gemv_bf16_n per head (src/attention.c:741-744, :812-815).  Brute force in
    double with the weight slices taken independently; the absorption identity the reference
    itself checks (:838-893): scores of q_abs against the latent equal scores of q against the
    keys expanded through W_k."""
    g = synth.rng(51)
    nh, nope, rope, vdim, kv_lora = 6, 40, 8, 24, 512
    q_dim, kv_dim = nope + rope, nope + vdim
    kvb = synth.normal_bf16(g, (nh * kv_dim, kv_lora))
    q = g.standard_normal((nh, q_dim)).astype(np.float32)
    q[2, 5] = 0.0                                            # a skipped row
    W = f32(kvb).reshape(nh, kv_dim, kv_lora)
    got = orc.mla_absorb(kvb, q, nope, rope, kv_dim)
    want = np.einsum("hr,hrc->hc", q[:, :nope].astype(np.float64), W[:, :nope])
    assert got.shape == (nh, 576)
    assert np.abs(got[:, :512] - want).max() < 1e-4
    assert np.array_equal(got[:, 512:512 + rope], q[:, nope:]) and not got[:, 512 + rope:].any()
    # transposed or mis-sliced weights would give something else entirely
    assert np.abs(want - np.einsum("hr,hrc->hc", q[:, :nope].astype(np.float64), W[:, vdim:vdim + nope])).max() > 1.0
    c = g.standard_normal((nh, kv_lora)).astype(np.float32)
    ex = orc.mla_expand(kvb, c, nope, vdim, kv_dim)
    assert np.abs(ex - np.einsum("hrc,hc->hr", W[:, nope:], c.astype(np.float64))).max() < 1e-4
    # absorption identity: (W_k^T q) . c == q . (W_k c)
    lat = g.standard_normal((9, kv_lora))
    s_abs = got[:, :512].astype(np.float64) @ lat.T
    s_exp = np.einsum("hr,thr->ht", q[:, :nope].astype(np.float64), np.einsum("hrc,tc->thr", W[:, :nope], lat))
    assert np.abs(s_abs - s_exp).max() < 1e-3


def test_gqa_prepare_closed_forms_and_brute_force(orc):
    """rms_norm_w with (1 + w) weights, rotate-half RoPE on the first rotary dims, bf16 narrowing
    (src/q35_model.c:1627-1652)."""
    H, KV, HD, rotary, theta, eps = 4, 2, 64, 32, 10000.0, 1e-6
    cos_t, sin_t = orc.build_rope(50, rotary, theta)
    inv = 1.0 / theta ** (2 * np.arange(rotary // 2) / rotary)
    assert np.allclose(cos_t[7], np.cos(7 * inv), atol=1e-7) and np.allclose(sin_t[7], np.sin(7 * inv), atol=1e-7)
    assert (cos_t[0] == 1).all() and (sin_t[0] == 0).all()
    g = synth.rng(52)
    n, pos0 = 5, 3
    stride = 2 * HD                                            # a gate behind every head's query
    qp = g.standard_normal((n, H, stride)).astype(np.float32)
    kp = g.standard_normal((n, KV * HD)).astype(np.float32)
    vp = g.standard_normal((n, KV * HD)).astype(np.float32)
    qn = (g.standard_normal(HD) * 0.1).astype(np.float32)
    kn = (g.standard_normal(HD) * 0.1).astype(np.float32)
    qo, ko, vo = orc.gqa_prepare(qp, stride, kp, vp, pos0, H, KV, HD, qn, kn, eps, cos_t, sin_t, rotary)

    def brute(x, w, p):
        x = x.astype(np.float64)
        y = x / np.sqrt((x * x).mean() + eps) * (1.0 + w.astype(np.float64))
        half = rotary // 2
        a, b = y[:half].copy(), y[half:rotary].copy()
        c, s_ = np.cos(p * inv), np.sin(p * inv)
        y[:half], y[half:rotary] = a * c - b * s_, b * c + a * s_
        return y
    for t in range(n):
        for h in range(H):
            want = brute(qp[t, h, :HD], qn, pos0 + t)
            assert np.abs(synth.bf16_to_f32(qo[t, h]) - want).max() < 2.0 ** -7 * np.abs(want).max()
        for h in range(KV):
            want = brute(kp[t, h * HD:(h + 1) * HD], kn, pos0 + t)
            assert np.abs(synth.bf16_to_f32(ko[t, h * HD:(h + 1) * HD]) - want).max() < 2.0 ** -7 * np.abs(want).max()
    assert np.array_equal(vo, synth.f32_to_bf16(vp))
    # closed forms: a constant head normalises to +-1 (times 1 + w); the gate half is never read
    one = np.full((1, 1, stride), 3.0, np.float32)
    one[0, 0, HD:] = 1e9
    z = np.zeros((1, HD), np.float32)
    q1, _, _ = orc.gqa_prepare(one, stride, z, z, 0, 1, 1, HD, None, None, 0.0, cos_t, sin_t, rotary)
    assert np.array_equal(synth.bf16_to_f32(q1[0, 0]), np.ones(HD, np.float32))
    # a quarter turn: with cos = 0, sin = 1 the two halves swap with a sign
    c0 = np.zeros((1, rotary // 2), np.float32); s1 = np.ones((1, rotary // 2), np.float32)
    x = np.zeros((1, 1, HD), np.float32); x[0, 0, :HD] = np.arange(1, HD + 1)
    q2, _, _ = orc.gqa_prepare(x, HD, z, z, 0, 1, 1, HD, None, None, 0.0, c0, s1, rotary)
    y = x[0, 0] / np.sqrt((x[0, 0] ** 2).mean())
    want = y.copy(); want[:rotary // 2] = -y[rotary // 2:rotary]; want[rotary // 2:rotary] = y[:rotary // 2]
    assert np.abs(synth.bf16_to_f32(q2[0, 0]) - want).max() < 2.0 ** -7 * np.abs(want).max()


# ------------------------------------------------------------------ indexer pool, candidate blocks
def _pool_inputs(rng, kp, hd=128):
    k = (rng.standard_normal((kp, hd)) * 2 + 0.7).astype(np.float32)
    g = rng.standard_normal((kp, hd)).astype(np.float32)
    ape = synth.f32_to_bf16(rng.standard_normal((kp, hd)).astype(np.float32) * 0.5)
    w = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)
    b = (0.1 * rng.standard_normal(hd)).astype(np.float32)
    return k, g, ape, w, b


def _layer_norm64(k, w, b, eps):
    k = k.astype(np.float64)
    mu = k.mean(axis=-1, keepdims=True)
    var = ((k - mu) ** 2).mean(axis=-1, keepdims=True)
    return (k - mu) / np.sqrt(var + eps) * w + b


@pytest.mark.parametrize("kp", [1, 3, 4, 8])
def test_indexer_pool_row_closed_forms_and_brute_force(orc, kp):
    rng = np.random.default_rng(90 + kp)
    eps = 1e-6
    k, g, ape, w, b = _pool_inputs(rng, kp)
    got = orc.indexer_pool_row(k, g, ape, w, b, eps)
    normed = _layer_norm64(k, w, b, eps)                                   # [kp, hd]
    p = softmax64(g.astype(np.float64) + f32(ape), axis=0)                  # over the pool's slots
    want = (p * normed).sum(axis=0)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6)
    # a slot-transposed gate or a softmax over the wrong axis would pass none of these:
    # equal gates and no position bias -> the plain mean of the normalised rows
    z = np.zeros_like(ape)
    np.testing.assert_allclose(orc.indexer_pool_row(k, np.zeros_like(g), z, w, b, eps), normed.mean(axis=0),
                               rtol=2e-5, atol=2e-6)
    # one slot's gate far above the rest -> that slot's normalised row
    g1 = np.zeros_like(g)
    g1[kp - 1] = 60.0
    np.testing.assert_allclose(orc.indexer_pool_row(k, g1, z, w, b, eps), normed[kp - 1], rtol=2e-5, atol=2e-6)
    # the same through the position bias alone (60 is exact in bf16)
    a1 = synth.f32_to_bf16(g1)
    np.testing.assert_allclose(orc.indexer_pool_row(k, np.zeros_like(g), a1, w, b, eps), normed[kp - 1],
                               rtol=2e-5, atol=2e-6)
    # a constant added to every gate of a dimension changes nothing
    shift = rng.standard_normal((1, 128)).astype(np.float32)
    np.testing.assert_allclose(orc.indexer_pool_row(k, g + shift, ape, w, b, eps), got, rtol=1e-5, atol=1e-6)
    if kp == 1:
        np.testing.assert_allclose(got, normed[0], rtol=2e-5, atol=2e-6)


def _brute_candidates(sc, bs, keep):
    n = sc.size
    nblk = -(-n // bs)
    bmax = np.array([sc[b * bs:(b + 1) * bs].max() for b in range(nblk)], np.float64)
    bmax[(n - 1) // bs] = np.inf
    order = sorted(range(nblk), key=lambda b: (-bmax[b], b))[:keep]
    cand = np.zeros(n, np.uint8)
    for b in order:
        cand[b * bs:(b + 1) * bs] = 1
    return cand, len(order)


@pytest.mark.parametrize("n,bs,keep", [(1000, 64, 4), (64, 64, 4), (65, 64, 1), (4096, 128, 8), (300, 7, 50), (5, 64, 3)])
def test_candidate_mask_vs_brute_force(orc, n, bs, keep):
    rng = np.random.default_rng(n * 31 + bs)
    sc = rng.standard_normal(n).astype(np.float32)
    cand, k = orc.candidate_mask(sc, bs, keep)
    want, wk = _brute_candidates(sc, bs, keep)
    assert k == wk == min(keep, -(-n // bs))
    assert np.array_equal(cand, want)
    assert cand[n - 1] == 1                                    # the partly filled block is always kept
    assert cand.sum() <= keep * bs
    masked = orc.candidate_apply(sc, cand)
    assert np.array_equal(masked[cand == 1], sc[cand == 1])
    assert np.all(np.isneginf(masked[cand == 0]))
    # the best position overall survives whenever a block besides the last may be kept
    if keep >= 2:
        assert cand[int(np.argmax(sc))] == 1
