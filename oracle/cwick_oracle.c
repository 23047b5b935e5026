/* cwick_oracle.c -- CPU restatement of the reference's attention hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the "port" CPU baseline that bench.py times beside the
 * GPU.  Nothing in the shipped library links, loads or calls it.
 *
 * Every function restates one piece of the reference (landpai/cwick) in plain
 * C and cites the file:line it follows.  Operation order is the reference's
 * wherever the reference fixes one (softmax: float max, expf, double sum,
 * float reciprocal; dots: the four-partial-sum grouping; position-outer
 * accumulation).  Where BASELINE's storage format has no counterpart in the
 * reference (FP8-E4M3 latent with one fp32 scale per 128-element block, FP8
 * indexer keys with one fp32 scale per token) the row is decoded on load and
 * the reference algorithm runs on the decoded floats.
 *
 * Pinning status (what independent evidence each function is checked against
 * in tests/).  oracle/_ref is the reference's ds_ops.c, tensor.c, util.c, pool.c
 * and log.c compiled as they lie; src/attention.c (needs the Metal bridge) and
 * src/q35_model.c, src/mm_model.c, src/ds_quant.c (NEON only) do not build on
 * this host, so nothing below is checked against object code of those files.
 *   orc_e4m3_to_f32, orc_e4m3_lut      closed form over all 256 bytes, the two
 *                                      reference decoders against each other,
 *                                      oracle/_ref (tensor.c)
 *   orc_f32_to_e4m3                    the reference's encoder as written, lost carry
 *                                      below 2^-6 included (known-answer test)
 *   orc_f32_to_e4m3_rne                nearest-grid-point brute force, idempotence,
 *                                      saturation (tools/ds_verify.c:48-63 property)
 *   orc_bf16_*, orc_f32_to_bf16_*      tests/test_cwick.c:72-83 values, bit recipe,
 *                                      oracle/_ref (util.c, ds_ops.c)
 *   orc_softmax                        closed forms, double brute force, oracle/_ref
 *                                      (cwick_softmax and ds_softmax, bit for bit)
 *   orc_dot_f32                        a constructed case where the four-lane order
 *                                      shows, double brute force
 *   orc_topk_heap                      oracle/_ref (ds_topk_scores), golden vectors,
 *                                      ties included
 *   orc_topk_contract                  brute-force sort, known answers
 *   orc_topk_quickselect               known answers traced by hand through
 *                                      src/attention.c:529-543 and :585-598 (they
 *                                      separate the threshold at want-1 from want and
 *                                      show the under-selection), subset-of-contract
 *                                      property
 *   orc_glm_select                     known answers traced by hand through
 *                                      src/attention.c:585-620 (tail present and absent, the
 *                                      query kept already / pruned / repeated, the strict flag,
 *                                      no more pools than wanted), on the score vectors of the
 *                                      quickselect traces; the contract's pool choice against the
 *                                      reference's where the two agree and where they do not
 *   orc_gqa_decode / orc_gqa_prefill   double brute force, decode==prefill row,
 *                                      rectangle==triangle: PARITY UNPINNED against a
 *                                      reference build, pinned by mathematics only
 *   orc_mla_decode[_f32]               double brute force over the dequantised latent,
 *                                      dense == sel 0..n-1, permutation invariance,
 *                                      the absorption identity of src/attention.c:838-893:
 *                                      PARITY UNPINNED against a reference build
 *   orc_mla_prefill_chunk              loop-of-decodes identity, bit for bit: PARITY
 *                                      UNPINNED against a reference build
 *   orc_mla_absorb, orc_mla_expand     double brute force (a transposed or mis-sliced weight
 *                                      fails), the absorption identity: scores from q_abs over
 *                                      the latent equal scores from q over W_k-expanded keys
 *   orc_gqa_prepare, orc_build_rope    closed forms (norm of a constant head, rotation by a
 *                                      quarter turn, position 0 is the identity), double
 *                                      brute force, norm preserved by the rotation:
 *                                      PARITY UNPINNED against a reference build
 *   orc_indexer_pool_row               closed forms (one slot: plain layer norm; equal gates:
 *                                      the mean of the normalised rows; one dominant gate: that
 *                                      row), invariance to a constant added to the gates,
 *                                      double brute force: PARITY UNPINNED against a reference
 *                                      build
 *   orc_candidate_mask / _apply        brute force in numpy, last block always kept, number of
 *                                      blocks kept; the block choice is orc_topk_heap's, which
 *                                      is pinned against oracle/_ref
 *   orc_mm_index_scores                known answers that separate the fused multiply-add from
 *                                      multiply-then-add, the serial order from a pairwise one,
 *                                      ReLU-before-sum and the head order; double brute force:
 *                                      PARITY UNPINNED against a reference build (the file is
 *                                      NEON-only, and whether the reference fuses is its
 *                                      compiler's choice)
 *   orc_mm_select_blocks               known answers traced by hand through src/mm_model.c:
 *                                      1733-1761 (newest block present, absent, and not yet
 *                                      written), brute force in numpy on tie-free scores; the
 *                                      block choice is orc_topk_heap's, pinned against oracle/_ref
 *   orc_indexer_scores[_ds]            double brute force, ReLU-before-weight, thread
 *                                      count invariance: PARITY UNPINNED against a
 *                                      reference build
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* codecs                                                              */
/* ------------------------------------------------------------------ */

/* src/util.h:55-60 (cwick_bf16_fast): the 16-bit left shift, nothing else. */
ORC_API float orc_bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* src/ds_ops.c:89-96 (ds_bf16_round) and src/q35_model.c:1154 (f2bf): true
 * round-to-nearest-even onto the bf16 grid. */
ORC_API uint16_t orc_f32_to_bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

ORC_API float orc_bf16_round(float f) {
    return orc_bf16_to_f32(orc_f32_to_bf16_rne(f));
}

/* src/util.c:202-210 (cwick_f32_to_bf16): adds bit15 + lsb (0..2), not
 * 0x7FFF + lsb, so it is in effect truncation.  Restated because it is the
 * reference's behaviour; the harness never feeds its output to one side only. */
ORC_API uint16_t orc_f32_to_bf16_cwick(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    uint32_t lsb = (u >> 16) & 1u;
    uint32_t round = ((u >> 15) & 1u) + lsb;
    uint32_t r = u + round;
    return (uint16_t)(r >> 16);
}

/* src/tensor.c:354-368 (cwick_fp8_e4m3_to_f32): E4M3fn, bias 7, subnormal step
 * 2^-9, no infinity, 0x7F / 0xFF are the only NaNs. */
ORC_API float orc_e4m3_to_f32(uint8_t b) {
    int sign = (b >> 7) & 1;
    int exp = (b >> 3) & 0xF;
    int man = b & 0x7;
    float v;
    if (exp == 0) v = (float)man * 0x1p-9f;
    else if (exp == 15 && man == 7) v = NAN;
    else v = (1.0f + (float)man / 8.0f) * ldexpf(1.0f, exp - 7);
    return sign ? -v : v;
}

/* src/ds_quant.c:59-72 (DS_E4M3_LUT recipe): the second, independent decoder;
 * (8 + m) * 2^(e - 10) for normals. */
ORC_API void orc_e4m3_lut(float *lut256) {
    for (int b = 0; b < 256; b++) {
        uint32_t sign = (uint32_t)(b >> 7) & 1u;
        uint32_t e = ((uint32_t)b >> 3) & 0xFu;
        uint32_t m = (uint32_t)b & 0x7u;
        float v;
        if (e == 0) v = ldexpf((float)m, -9);
        else if (e == 15 && m == 7) v = NAN;
        else v = ldexpf((float)(8u + m), (int)e - 10);
        lut256[b] = sign ? -v : v;
    }
}

/* src/ds_quant.c:102-128 (ds_f32_to_e4m3): round-to-nearest-even into e4m3fn;
 * the caller clamps to +-448 first, values past it saturate to 0x7E. */
ORC_API uint8_t orc_f32_to_e4m3(float v) {
    if (v == 0.0f) return 0;
    uint32_t u;
    memcpy(&u, &v, sizeof u);
    uint32_t sign = u >> 31;
    int32_t exp = (int32_t)((u >> 23) & 0xFFu) - 127;
    uint32_t m24 = (1u << 23) | (u & 0x7FFFFFu);
    if (exp >= -6) {
        uint32_t keep = m24 >> 20;
        uint32_t rem = m24 & 0xFFFFFu;
        const uint32_t half = 0x80000u;
        if (rem > half || (rem == half && (keep & 1u))) keep++;
        int32_t e = exp;
        if (keep == 16u) { keep >>= 1; e++; }
        if (e > 8) { keep = 14u; e = 8; }
        return (uint8_t)((sign << 7) | ((uint32_t)(e + 7) << 3) | (keep & 7u));
    }
    if (exp < -10) return (uint8_t)(sign << 7);
    int32_t sh = 14 - exp;
    uint32_t mm = m24 >> sh;
    uint32_t rem = m24 & ((1u << sh) - 1u);
    uint32_t half = 1u << (sh - 1);
    if (rem > half || (rem == half && (mm & 1u))) mm++;
    return (uint8_t)((sign << 7) | (mm & 7u));
}

/* The contract the reference states for its encoder (tools/ds_verify.c:48-63:
 * "dequant(quant(v)) must be the nearest e4m3 to v"): round to nearest, ties
 * to even, saturating at 448.  It differs from orc_f32_to_e4m3 in one corner:
 * in the subnormal branch above a round-up out of mantissa 7 carries into the
 * first normal (byte 0x08 = 2^-6); the reference masks the carry away
 * (`mm & 7u`, src/ds_quant.c:127) and returns +-0 for 0.01465 <= |v| < 2^-6.
 * The cache-append path and the input generator use this contract form. */
ORC_API uint8_t orc_f32_to_e4m3_rne(float v) {
    if (v == 0.0f) return 0;
    uint32_t u;
    memcpy(&u, &v, sizeof u);
    int32_t exp = (int32_t)((u >> 23) & 0xFFu) - 127;
    if (exp >= -6 || exp < -10) return orc_f32_to_e4m3(v);
    uint32_t sign = u >> 31;
    uint32_t m24 = (1u << 23) | (u & 0x7FFFFFu);
    int32_t sh = 14 - exp;
    uint32_t mm = m24 >> sh;
    uint32_t rem = m24 & ((1u << sh) - 1u);
    uint32_t half = 1u << (sh - 1);
    if (rem > half || (rem == half && (mm & 1u))) mm++;
    return (uint8_t)((sign << 7) | mm);          /* mm == 8 is byte 0x08 */
}

/* BASELINE storage format (no reference counterpart; the reference's own FP8
 * producer is the per-32 power-of-two scale of src/ds_ops.c:235-252): one fp32
 * scale = amax/448 per `block` consecutive elements of a row, amax == 0 -> 1. */
ORC_API void orc_quantize_rows_e4m3(const float *x, int64_t rows, int64_t cols,
                                    int64_t block, uint8_t *q, float *scales) {
    const int64_t nb = (cols + block - 1) / block;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t b = 0; b < nb; b++) {
            const int64_t c0 = b * block;
            const int64_t c1 = c0 + block < cols ? c0 + block : cols;
            float amax = 0.0f;
            for (int64_t c = c0; c < c1; c++) {
                float a = fabsf(x[r * cols + c]);
                if (a > amax) amax = a;
            }
            float s = amax > 0.0f ? amax / 448.0f : 1.0f;
            scales[r * nb + b] = s;
            for (int64_t c = c0; c < c1; c++) {
                float v = x[r * cols + c] / s;
                if (v > 448.0f) v = 448.0f;
                if (v < -448.0f) v = -448.0f;
                q[r * cols + c] = orc_f32_to_e4m3_rne(v);
            }
        }
}

/* ------------------------------------------------------------------ */
/* softmax and dots                                                    */
/* ------------------------------------------------------------------ */

/* src/tensor.c:793-803 (cwick_softmax) == src/ds_ops.c:100-107 (ds_softmax). */
ORC_API void orc_softmax(float *s, int64_t n) {
    float mx = s[0];
    for (int64_t i = 1; i < n; i++) if (s[i] > mx) mx = s[i];
    double sum = 0.0;
    for (int64_t i = 0; i < n; i++) {
        s[i] = expf(s[i] - mx);
        sum += s[i];
    }
    float inv = (float)(1.0 / sum);
    for (int64_t i = 0; i < n; i++) s[i] *= inv;
}

/* src/attention.c:249-258 (dot_f32, portable branch): four partial sums,
 * combined as (s0+s1)+(s2+s3). */
ORC_API float orc_dot_f32(const float *a, const float *b, int64_t n) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int64_t i = 0;
    for (; i + 4 <= n; i += 4) {
        s0 += a[i + 0] * b[i + 0];
        s1 += a[i + 1] * b[i + 1];
        s2 += a[i + 2] * b[i + 2];
        s3 += a[i + 3] * b[i + 3];
    }
    for (; i < n; i++) s0 += a[i] * b[i];
    return (s0 + s1) + (s2 + s3);
}

static int orc_threads(int nthreads) {
#ifdef _OPENMP
    if (nthreads <= 0) nthreads = omp_get_max_threads();
    return nthreads < 1 ? 1 : nthreads;
#else
    (void)nthreads;
    return 1;
#endif
}

ORC_API int orc_max_threads(void) { return orc_threads(0); }

/* ------------------------------------------------------------------ */
/* GQA decode (BASELINE config 1)                                      */
/* ------------------------------------------------------------------ */
/* src/q35_model.c:1460-1518 and :1656-1701.  The cache is bf16 and is widened
 * to f32 exactly as q35_widen_rows does (:1543-1555); q arrives bf16 and is
 * widened the same way.  Scores walk cache rows (one row serves every head),
 * cwick_softmax per head, AV in `nslice` row slices with private accumulators
 * summed in slice order (:1693-1701).  nslice = 16 is Q35_DEC_SLICES.
 *
 * q35_dot_f32 (:1425-1437) keeps sixteen partial sums (four NEON registers)
 * folded as ((s0+s1)+(s2+s3)) then across lanes pairwise; restated here
 * lane for lane.  NEON's vfmaq is a fused multiply-add; products of two bf16
 * values are exact in fp32, so fused and unfused agree bit for bit. */
static float q35_dot16(const float *a, const float *b, int n) {
    float s[16];
    for (int j = 0; j < 16; j++) s[j] = 0.0f;
    int i = 0;
    for (; i + 16 <= n; i += 16)
        for (int j = 0; j < 16; j++) s[j] += a[i + j] * b[i + j];
    float t[4];
    for (int j = 0; j < 4; j++)
        t[j] = (s[j] + s[4 + j]) + (s[8 + j] + s[12 + j]);
    float r = (t[0] + t[1]) + (t[2] + t[3]);
    for (; i < n; i++) r += a[i] * b[i];
    return r;
}

ORC_API void orc_gqa_decode(const uint16_t *q_bf16,   /* [nh][hd] */
                            const uint16_t *k_bf16,   /* [keys][nkv*hd] */
                            const uint16_t *v_bf16,   /* [keys][nkv*hd] */
                            int64_t keys, int nh, int nkv, int hd, float scale,
                            int nslice, int nthreads,
                            float *out /* [nh][hd] */) {
    const int group = nh / nkv;
    const int64_t kv = (int64_t)nkv * hd;
    if (nslice <= 0) nslice = 16;
    nthreads = orc_threads(nthreads);
    float *q = malloc(sizeof(float) * (size_t)nh * hd);
    float *s = malloc(sizeof(float) * (size_t)nh * keys);
    float *buf = malloc(sizeof(float) * (size_t)nslice * nh * hd);
    for (int i = 0; i < nh * hd; i++) q[i] = orc_bf16_to_f32(q_bf16[i]);

    /* dec_scores: split over positions */
#pragma omp parallel num_threads(nthreads)
    {
        float *row = malloc(sizeof(float) * (size_t)kv);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < keys; t++) {
            for (int64_t c = 0; c < kv; c++) row[c] = orc_bf16_to_f32(k_bf16[t * kv + c]);
            for (int g = 0; g < nkv; g++)
                for (int j = 0; j < group; j++) {
                    const int h = g * group + j;
                    s[(size_t)h * keys + t] =
                        q35_dot16(q + (size_t)h * hd, row + (size_t)g * hd, hd) * scale;
                }
        }
        free(row);
    }
    /* dec_softmax: split over heads */
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int h = 0; h < nh; h++) orc_softmax(s + (size_t)h * keys, keys);
    /* dec_out_slices */
#pragma omp parallel num_threads(nthreads)
    {
        float *row = malloc(sizeof(float) * (size_t)kv);
#pragma omp for schedule(static)
        for (int sl = 0; sl < nslice; sl++) {
            const int64_t lo = keys * sl / nslice, hi = keys * (sl + 1) / nslice;
            float *o = buf + (size_t)sl * nh * hd;
            memset(o, 0, sizeof(float) * (size_t)nh * hd);
            for (int64_t t = lo; t < hi; t++) {
                for (int64_t c = 0; c < kv; c++) row[c] = orc_bf16_to_f32(v_bf16[t * kv + c]);
                for (int h = 0; h < nh; h++) {
                    const float w = s[(size_t)h * keys + t];
                    if (w == 0.0f) continue;
                    const float *vr = row + (size_t)(h / group) * hd;
                    float *oh = o + (size_t)h * hd;
                    for (int i = 0; i < hd; i++) oh[i] += w * vr[i];
                }
            }
        }
        free(row);
    }
    for (int h = 0; h < nh; h++) {
        float *dst = out + (size_t)h * hd;
        memcpy(dst, buf + (size_t)h * hd, sizeof(float) * (size_t)hd);
        for (int sl = 1; sl < nslice; sl++) {
            const float *src = buf + ((size_t)sl * nh + h) * hd;
            for (int i = 0; i < hd; i++) dst[i] += 1.0f * src[i];
        }
    }
    free(buf); free(s); free(q);
}

/* ------------------------------------------------------------------ */
/* GQA causal prefill (BASELINE config 2)                              */
/* ------------------------------------------------------------------ */
/* src/q35_model.c:1713-1746: per head, per tile of `tile_q` queries
 * (Q35_ATTN_Q, src/q35.h:82 = 128): S = scale * Q K^T over the rectangle of
 * kk = pos0 + t0 + nq keys with the naive GEMM of :1586-1599 (one serial
 * accumulator per output), the tail past each row's own position set to -1e30
 * (:1529-1537), cwick_softmax over the whole row, O = S V.
 *
 * t_begin/t_end/t_step select which query tiles are computed (the CPU baseline
 * sub-samples tiles at the full shape); rows of skipped tiles are left
 * untouched. */
ORC_API void orc_gqa_prefill(const uint16_t *q_bf16,  /* [n][nh*hd] */
                             const uint16_t *k_bf16,  /* [pos0+n][nkv*hd] */
                             const uint16_t *v_bf16,
                             int64_t pos0, int64_t n, int nh, int nkv, int hd,
                             float scale, int tile_q,
                             int64_t tile_begin, int64_t tile_end, int64_t tile_step,
                             int nthreads, float *out /* [n][nh*hd] */) {
    const int group = nh / nkv;
    const int64_t kv = (int64_t)nkv * hd, qdim = (int64_t)nh * hd;
    if (tile_q <= 0) tile_q = 128;
    const int64_t ntiles = (n + tile_q - 1) / tile_q;
    if (tile_end <= 0 || tile_end > ntiles) tile_end = ntiles;
    if (tile_step <= 0) tile_step = 1;
    if (tile_begin < 0) tile_begin = 0;
    nthreads = orc_threads(nthreads);
    const int64_t keys_all = pos0 + n;

    for (int g = 0; g < nkv; g++) {
        /* the widened K/V slice of this kv head (q35_widen_rows) */
        float *kf = malloc(sizeof(float) * (size_t)keys_all * hd);
        float *vf = malloc(sizeof(float) * (size_t)keys_all * hd);
        for (int64_t t = 0; t < keys_all; t++)
            for (int i = 0; i < hd; i++) {
                kf[t * hd + i] = orc_bf16_to_f32(k_bf16[t * kv + (int64_t)g * hd + i]);
                vf[t * hd + i] = orc_bf16_to_f32(v_bf16[t * kv + (int64_t)g * hd + i]);
            }
        const int64_t nitems = (int64_t)group * ((tile_end - tile_begin + tile_step - 1) / tile_step);
#pragma omp parallel num_threads(nthreads)
        {
            float *S = malloc(sizeof(float) * (size_t)tile_q * keys_all);
            float *qf = malloc(sizeof(float) * (size_t)tile_q * hd);
#pragma omp for schedule(dynamic, 1)
            for (int64_t item = 0; item < nitems; item++) {
                const int h = g * group + (int)(item % group);
                const int64_t tile = tile_begin + (item / group) * tile_step;
                const int64_t t0 = tile * tile_q;
                const int64_t nq = n - t0 < tile_q ? n - t0 : tile_q;
                const int64_t kk = pos0 + t0 + nq;
                for (int64_t i = 0; i < nq; i++)
                    for (int d = 0; d < hd; d++)
                        qf[i * hd + d] = orc_bf16_to_f32(q_bf16[(t0 + i) * qdim + (int64_t)h * hd + d]);
                /* Q35_MM(nq, kk, HD, scale, q, ., K, ., btrans=1, beta=0, S, kk) */
                for (int64_t i = 0; i < nq; i++)
                    for (int64_t j = 0; j < kk; j++) {
                        float acc = 0.0f;
                        const float *a = qf + i * hd, *b = kf + j * hd;
                        for (int d = 0; d < hd; d++) acc += a[d] * b[d];
                        S[i * kk + j] = scale * acc;
                    }
                /* softmax_items */
                for (int64_t i = 0; i < nq; i++) {
                    const int64_t lim = pos0 + t0 + i + 1;
                    float *row = S + i * kk;
                    for (int64_t j = lim; j < kk; j++) row[j] = -1e30f;
                    orc_softmax(row, kk);
                }
                /* Q35_MM(nq, HD, kk, 1, S, kk, V, ., btrans=0, beta=0, o, qdim) */
                for (int64_t i = 0; i < nq; i++) {
                    float *o = out + (t0 + i) * qdim + (int64_t)h * hd;
                    for (int d = 0; d < hd; d++) {
                        float acc = 0.0f;
                        for (int64_t j = 0; j < kk; j++) acc += S[i * kk + j] * vf[j * hd + d];
                        o[d] = 1.0f * acc;
                    }
                }
            }
            free(S); free(qf);
        }
        free(kf); free(vf);
    }
}

/* ------------------------------------------------------------------ */
/* absorbed-latent MLA decode (BASELINE configs 3 and 5)               */
/* ------------------------------------------------------------------ */
/* Decode one FP8 latent row into fp32: e4m3 value times the fp32 scale of its
 * block.  `block` is 128 for BASELINE's layout, giving 5 scales per 576-wide
 * row (4 x 128 nope + 1 x 64 rope). */
static void latent_row_f32(const uint8_t *row, const float *scales, int64_t dim,
                           int64_t block, const float *lut, float *dst) {
    for (int64_t i = 0; i < dim; i++) dst[i] = lut[row[i]] * scales[i / block];
}

/* src/attention.c:749-811 (mla_latent_decode's two reductions) on BASELINE's
 * inputs: q is already absorbed (q_abs, :741-744 is outside the config) and
 * arrives bf16; the output is c_acc, the latent-space accumulator (:779-811),
 * before the W_v expansion (:812-815).
 *
 *   scores[h][i] = dot_f32(q_abs[h], c[sel[i]], kdim) * scale     position-outer
 *   cwick_softmax(scores[h])                                      per head
 *   c_acc[h]    += p[h][i] * c[sel[i]][0 .. vdim)                 position-outer,
 *                                                                 i ascending
 * kdim = 576 (nope + rope) feeds the score, vdim = 512 the value: the rope
 * tail carries position only.  The reference's latent is rope-free
 * (kdim == vdim == kv_lora, :107); with kdim == vdim this is exactly its loop.
 * sel == NULL means every position 0..nlist-1 (:759).  Entries sel[i] < 0 are
 * skipped the way src/ds_model.c:929/:940/:950 skips its -1 padding: the slot
 * contributes nothing to max, sum or output.
 *
 * nthreads <= 1 keeps the reference's serial order.  nthreads > 1 (CPU
 * baseline timing only) splits the score loop over positions, as
 * scores_range does (:418-433), and the accumulation over row slices with
 * private accumulators summed in slice order, as q35's decode AV does. */
ORC_API void orc_mla_decode(const uint16_t *q_bf16,    /* [nh][kdim] */
                            const uint8_t *lat,        /* [cap][kdim] e4m3 */
                            const float *lat_scales,   /* [cap][nblk] */
                            int64_t kdim, int64_t vdim, int64_t block,
                            const int32_t *sel, int64_t nlist,
                            int nh, float scale, int nthreads,
                            float *out /* [nh][vdim] */) {
    float lut[256];
    orc_e4m3_lut(lut);
    const int64_t nblk = (kdim + block - 1) / block;
    nthreads = orc_threads(nthreads);
    float *q = malloc(sizeof(float) * (size_t)nh * kdim);
    float *scores = malloc(sizeof(float) * (size_t)nh * (nlist > 0 ? nlist : 1));
    for (int64_t i = 0; i < (int64_t)nh * kdim; i++) q[i] = orc_bf16_to_f32(q_bf16[i]);

    /* compact away skipped slots first so softmax sees only live entries */
    int64_t *live = malloc(sizeof(int64_t) * (size_t)(nlist > 0 ? nlist : 1));
    int64_t nl = 0;
    for (int64_t i = 0; i < nlist; i++) {
        int64_t t = sel ? sel[i] : i;
        if (t >= 0) live[nl++] = t;
    }
    if (nl == 0) {
        memset(out, 0, sizeof(float) * (size_t)nh * vdim);
        free(live); free(scores); free(q);
        return;
    }

#pragma omp parallel num_threads(nthreads)
    {
        float *c = malloc(sizeof(float) * (size_t)kdim);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < nl; i++) {
            const int64_t t = live[i];
            latent_row_f32(lat + t * kdim, lat_scales + t * nblk, kdim, block, lut, c);
            for (int h = 0; h < nh; h++)
                scores[(size_t)h * nl + i] = orc_dot_f32(q + (size_t)h * kdim, c, kdim) * scale;
        }
        free(c);
    }
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int h = 0; h < nh; h++) orc_softmax(scores + (size_t)h * nl, nl);

    const int nslice = nthreads > 1 ? nthreads : 1;
    float *buf = nslice > 1 ? malloc(sizeof(float) * (size_t)nslice * nh * vdim) : out;
#pragma omp parallel num_threads(nthreads)
    {
        float *c = malloc(sizeof(float) * (size_t)kdim);
#pragma omp for schedule(static)
        for (int sl = 0; sl < nslice; sl++) {
            const int64_t lo = nl * sl / nslice, hi = nl * (sl + 1) / nslice;
            float *acc = buf + (size_t)sl * nh * vdim;
            memset(acc, 0, sizeof(float) * (size_t)nh * vdim);
            for (int64_t i = lo; i < hi; i++) {
                const int64_t t = live[i];
                latent_row_f32(lat + t * kdim, lat_scales + t * nblk, kdim, block, lut, c);
                for (int h = 0; h < nh; h++) {
                    const float p = scores[(size_t)h * nl + i];
                    float *a = acc + (size_t)h * vdim;
                    for (int64_t j = 0; j < vdim; j++) a[j] += p * c[j];
                }
            }
        }
        free(c);
    }
    if (nslice > 1) {
        memcpy(out, buf, sizeof(float) * (size_t)nh * vdim);
        for (int sl = 1; sl < nslice; sl++) {
            const float *src = buf + (size_t)sl * nh * vdim;
            for (int64_t i = 0; i < (int64_t)nh * vdim; i++) out[i] += src[i];
        }
        free(buf);
    }
    free(live); free(scores); free(q);
}

/* The reference's own precisions, for checks against oracle/_ref: the latent
 * is fp32 (src/attention.c:806-807) or bf16 (:802-803), kdim == vdim. */
ORC_API void orc_mla_decode_f32(const float *q_abs,    /* [nh][dim] */
                                const float *lat,      /* [cap][dim] */
                                int64_t dim, const int64_t *sel, int64_t nlist,
                                int nh, float scale, float *out /* [nh][dim] */) {
    float *scores = malloc(sizeof(float) * (size_t)nh * nlist);
    for (int64_t i = 0; i < nlist; i++) {
        const int64_t t = sel ? sel[i] : i;
        for (int h = 0; h < nh; h++)
            scores[(size_t)h * nlist + i] =
                orc_dot_f32(q_abs + (size_t)h * dim, lat + t * dim, dim) * scale;
    }
    for (int h = 0; h < nh; h++) orc_softmax(scores + (size_t)h * nlist, nlist);
    memset(out, 0, sizeof(float) * (size_t)nh * dim);
    for (int64_t i = 0; i < nlist; i++) {
        const int64_t t = sel ? sel[i] : i;
        const float *c = lat + t * dim;
        for (int h = 0; h < nh; h++) {
            const float p = scores[(size_t)h * nlist + i];
            float *a = out + (size_t)h * dim;
            for (int64_t j = 0; j < dim; j++) a[j] += p * c[j];
        }
    }
    free(scores);
}

/* ------------------------------------------------------------------ */
/* MLA chunked prefill (BASELINE config 4)                             */
/* ------------------------------------------------------------------ */
/* src/attention.c:1010-1019: the reference's chunk path is n sequential
 * mla_latent_decode calls at positions pos0 + t, each over npos = pos + 1
 * keys (:662); causality is that prefix length.  The latent rows of the whole
 * chunk are already in the cache (:988-1007).  q_begin/q_end/q_step select
 * which queries are computed (CPU baseline sub-sampling); others untouched. */
ORC_API void orc_mla_prefill_chunk(const uint16_t *q_bf16,   /* [n][nh][kdim] */
                                   const uint8_t *lat, const float *lat_scales,
                                   int64_t kdim, int64_t vdim, int64_t block,
                                   int64_t pos0, int64_t n, int nh, float scale,
                                   int64_t q_begin, int64_t q_end, int64_t q_step,
                                   int nthreads, float *out /* [n][nh][vdim] */) {
    if (q_end <= 0 || q_end > n) q_end = n;
    if (q_step <= 0) q_step = 1;
    if (q_begin < 0) q_begin = 0;
    for (int64_t t = q_begin; t < q_end; t += q_step)
        orc_mla_decode(q_bf16 + t * nh * kdim, lat, lat_scales, kdim, vdim, block,
                       NULL, pos0 + t + 1, nh, scale, nthreads,
                       out + t * nh * vdim);
}

/* ------------------------------------------------------------------ */
/* lightning indexer scores (BASELINE config 5)                        */
/* ------------------------------------------------------------------ */
/* src/attention.c:573-582 (indexer_select's score loop) with the ReLU-then-
 * weight form shared by src/ds_model.c:1110-1121:
 *
 *     sc[t] = sum_h relu(q_h . k_t) * w[h]          h ascending, fp32
 *
 * Keys are FP8-E4M3 with one fp32 scale per token (BASELINE's format).  The
 * scale is positive, so it commutes with the ReLU; it is applied once to the
 * finished per-head dot rather than to every element:
 *
 *     d   = dot_f32(q_h, e_t)         e_t = raw e4m3 values; every product of a
 *                                     bf16 and an e4m3 value is exact in fp32,
 *                                     so only the fixed 4-lane summation order
 *                                     of dot_f32 rounds
 *     d   = d * kscale[t]
 *     if (d < 0) d = 0
 *     s  += d * w[h]                  one multiply, one add (not fused)
 *
 * This order is what the exact HIP kernel mirrors instruction for
 * instruction, which is what makes the selected indices bit-exact.  The head
 * weights arrive already folded with 1/sqrt(hd*ih) (:564-565). */
ORC_API void orc_indexer_scores(const uint16_t *q_bf16,  /* [ih][hd] */
                                const float *w,          /* [ih] */
                                const uint8_t *keys,     /* [n][hd] e4m3 */
                                const float *kscale,     /* [n] */
                                int64_t n, int ih, int hd, int nthreads,
                                float *sc /* [n] */) {
    float lut[256];
    orc_e4m3_lut(lut);
    nthreads = orc_threads(nthreads);
    float *q = malloc(sizeof(float) * (size_t)ih * hd);
    for (int i = 0; i < ih * hd; i++) q[i] = orc_bf16_to_f32(q_bf16[i]);
#pragma omp parallel num_threads(nthreads)
    {
        float *e = malloc(sizeof(float) * (size_t)hd);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < n; t++) {
            for (int i = 0; i < hd; i++) e[i] = lut[keys[t * hd + i]];
            float s = 0.0f;
            for (int h = 0; h < ih; h++) {
                float d = orc_dot_f32(e, q + (size_t)h * hd, hd);
                d = d * kscale[t];
                if (d < 0.0f) d = 0.0f;
                s += d * w[h];       /* built with -ffp-contract=off: mul, then add */
            }
            sc[t] = s;
        }
        free(e);
    }
    free(q);
}

/* src/ds_model.c:1099-1121 (ds_indexer's score loop) on BASELINE's FP8 keys: the key the
 * reference holds in fp32 is the dequantised one, e4m3(byte) * kscale[t]; the dot is serial
 * over i (`d += qh[i] * kt[i]`, :1115), rounded to bf16 (`ds_bf16_round(d)`, :1116), kept when
 * positive and weighted by iw[h], which is itself rounded to bf16 (:1101; the caller passes
 * w[h] = weights_proj * IH^-1/2 * NH^-1/2 and the rounding happens here). */
ORC_API void orc_indexer_scores_ds(const uint16_t *q_bf16,  /* [ih][hd] */
                                   const float *w,          /* [ih] */
                                   const uint8_t *keys,     /* [n][hd] e4m3 */
                                   const float *kscale,     /* [n] */
                                   int64_t n, int ih, int hd, int nthreads,
                                   float *sc /* [n] */) {
    float lut[256];
    orc_e4m3_lut(lut);
    nthreads = orc_threads(nthreads);
    float *q = malloc(sizeof(float) * (size_t)ih * hd);
    float *iw = malloc(sizeof(float) * (size_t)ih);
    for (int i = 0; i < ih * hd; i++) q[i] = orc_bf16_to_f32(q_bf16[i]);
    for (int h = 0; h < ih; h++) iw[h] = orc_bf16_round(w[h]);
#pragma omp parallel num_threads(nthreads)
    {
        float *kt = malloc(sizeof(float) * (size_t)hd);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < n; t++) {
            for (int i = 0; i < hd; i++) kt[i] = lut[keys[t * hd + i]] * kscale[t];
            float acc = 0.0f;
            for (int h = 0; h < ih; h++) {
                const float *qh = q + (size_t)h * hd;
                float d = 0.0f;
                for (int i = 0; i < hd; i++) d += qh[i] * kt[i];
                d = orc_bf16_round(d);
                if (d > 0.0f) acc += d * iw[h];
            }
            sc[t] = acc;
        }
        free(kt);
    }
    free(iw);
    free(q);
}

/* src/ds_model.c:917-966 (ds_sparse_attn_heads) on BASELINE's FP8 latent: per head, scores
 * over idx[] with a serial dot (`d += qh[i] * kt[i]`, then `d *= scale`, :933-934), entries < 0
 * skipped, running maximum from -1e30 (:926), float sum of expf(score - max) (:939-944), the
 * sink term expf(sink[h] - max) added to the sum only (:946), values accumulated in list order
 * and scaled by 1/sum at the end (:948-958).  The reference's key and value are the same 512
 * floats (HD); here the score uses kdim, the value the first vdim of the same row, as
 * orc_mla_decode does.  idx == NULL means 0..nlist-1.  An entry of the reference's list
 * addresses the window ring below W and compressed row t - W from there (:930-931): one cache
 * whose first W rows are the ring. */
ORC_API void orc_sparse_attn_sink(const uint16_t *q_bf16,   /* [nh][kdim] */
                                  const uint8_t *lat, const float *lat_scales,
                                  int64_t kdim, int64_t vdim, int64_t block,
                                  const int32_t *idx, int64_t nlist, int nh, float scale,
                                  const float *sink /* [nh] or NULL */, int nthreads,
                                  float *out /* [nh][vdim] */) {
    float lut[256];
    orc_e4m3_lut(lut);
    const int64_t nblk = (kdim + block - 1) / block;
    nthreads = orc_threads(nthreads);
    /* the rows are decoded once; the reference's caches hold them decoded */
    float *rows = malloc(sizeof(float) * (size_t)(nlist > 0 ? nlist : 1) * kdim);
    for (int64_t j = 0; j < nlist; j++) {
        const int64_t t = idx ? idx[j] : j;
        if (t >= 0) latent_row_f32(lat + t * kdim, lat_scales + t * nblk, kdim, block, lut, rows + j * kdim);
    }
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int h = 0; h < nh; h++) {
        float *qh = malloc(sizeof(float) * (size_t)kdim);
        float *sc = malloc(sizeof(float) * (size_t)(nlist > 0 ? nlist : 1));
        float *oh = out + (size_t)h * vdim;
        for (int64_t i = 0; i < kdim; i++) qh[i] = orc_bf16_to_f32(q_bf16[(size_t)h * kdim + i]);
        float mx = -1e30f;
        for (int64_t j = 0; j < nlist; j++) {
            const int64_t t = idx ? idx[j] : j;
            if (t < 0) { sc[j] = -INFINITY; continue; }
            const float *kt = rows + j * kdim;
            float d = 0.0f;
            for (int64_t i = 0; i < kdim; i++) d += qh[i] * kt[i];
            d *= scale;
            sc[j] = d;
            if (d > mx) mx = d;
        }
        float sum = 0.0f;
        for (int64_t j = 0; j < nlist; j++) {
            const int64_t t = idx ? idx[j] : j;
            if (t < 0) { sc[j] = 0.0f; continue; }
            const float e = expf(sc[j] - mx);
            sc[j] = e;
            sum += e;
        }
        if (sink) sum += expf(sink[h] - mx);
        for (int64_t i = 0; i < vdim; i++) oh[i] = 0.0f;
        for (int64_t j = 0; j < nlist; j++) {
            const int64_t t = idx ? idx[j] : j;
            if (t < 0) continue;
            const float *kt = rows + j * kdim;
            const float wgt = sc[j];
            for (int64_t i = 0; i < vdim; i++) oh[i] += wgt * kt[i];
        }
        const float inv = 1.0f / sum;
        for (int64_t i = 0; i < vdim; i++) oh[i] *= inv;
        free(sc); free(qh);
    }
    free(rows);
}

/* ------------------------------------------------------------------ */
/* the steps around the attention kernels                               */
/* ------------------------------------------------------------------ */
/* src/attention.c:145-177 (gemv_bf16_t, the portable loop at :170-176) applied per head as at
 * :741-744: q_abs[h][c] = sum_r q[h][r] * W_k[h][r][c], row-outer, rows whose q is zero
 * skipped, multiply and add rounded separately.  W_k[h] = rows h*kv_dim .. +nope of kv_b_proj.
 * The `rope` dims that follow the nope dims in q are copied behind the kv_lora outputs (the
 * reference's released model has none, :107); the row is padded to `out_dim` with zeros. */
ORC_API void orc_mla_absorb(const uint16_t *kvb_w, const float *q, int nh, int q_dim, int nope,
                            int rope, int kv_dim, int kv_lora, int out_dim, float *q_abs) {
    for (int h = 0; h < nh; h++) {
        float *out = q_abs + (size_t)h * out_dim;
        const float *in = q + (size_t)h * q_dim;
        const uint16_t *w = kvb_w + (size_t)h * kv_dim * kv_lora;
        for (int c = 0; c < out_dim; c++) out[c] = 0.0f;
        for (int r = 0; r < nope; r++) {
            const float a = in[r];
            if (a == 0.0f) continue;
            const uint16_t *wr = w + (size_t)r * kv_lora;
            for (int c = 0; c < kv_lora; c++) out[c] += a * orc_bf16_to_f32(wr[c]);
        }
        for (int i = 0; i < rope && kv_lora + i < out_dim; i++) out[kv_lora + i] = in[nope + i];
    }
}

/* src/attention.c:184-224 (gemv_bf16_n, the portable loop at :211-223: four partial sums over
 * j mod 4, combined (s0+s1)+(s2+s3)) applied per head as at :812-815:
 * attn_out[h][r] = W_v[h][r] . c_acc[h], W_v[h] = rows h*kv_dim+nope .. +vdim of kv_b_proj. */
ORC_API void orc_mla_expand(const uint16_t *kvb_w, const float *c_acc, int nh, int nope, int vdim,
                            int kv_dim, int kv_lora, float *attn_out) {
    for (int h = 0; h < nh; h++) {
        const float *in = c_acc + (size_t)h * kv_lora;
        for (int r = 0; r < vdim; r++) {
            const uint16_t *wr = kvb_w + ((size_t)h * kv_dim + nope + r) * kv_lora;
            float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
            int j = 0;
            for (; j + 4 <= kv_lora; j += 4) {
                s0 += orc_bf16_to_f32(wr[j + 0]) * in[j + 0];
                s1 += orc_bf16_to_f32(wr[j + 1]) * in[j + 1];
                s2 += orc_bf16_to_f32(wr[j + 2]) * in[j + 2];
                s3 += orc_bf16_to_f32(wr[j + 3]) * in[j + 3];
            }
            for (; j < kv_lora; j++) s0 += orc_bf16_to_f32(wr[j]) * in[j];
            attn_out[(size_t)h * vdim + r] = (s0 + s1) + (s2 + s3);
        }
    }
}

/* src/q35_model.c:459-476 (build_rope): cos/sin of p / theta^(2i/rotary) in double, stored as
 * float, [position][rotary/2]. */
ORC_API void orc_build_rope(int max_pos, int rotary, double theta, float *cos_t, float *sin_t) {
    const int pairs = rotary / 2;
    for (int p = 0; p < max_pos; p++)
        for (int i = 0; i < pairs; i++) {
            const double inv = 1.0 / pow(theta, (double)(2 * i) / (double)rotary);
            const double a = (double)p * inv;
            cos_t[(size_t)p * pairs + i] = (float)cos(a);
            sin_t[(size_t)p * pairs + i] = (float)sin(a);
        }
}

/* src/q35_model.c:111-121 (rms_norm_w: serial sum of squares, rstd = 1/sqrtf(acc/n + eps),
 * out = in * rstd * (1 + w)) followed by :144-153 (rope_apply: index i pairs with i + pairs,
 * rotate-half) on one head, in place; w may be NULL. */
static void orc_head_norm_rope(float *v, int hd, const float *w, float eps, const float *cos_p,
                               const float *sin_p, int rotary) {
    float acc = 0.0f;
    for (int i = 0; i < hd; i++) acc += v[i] * v[i];
    const float rstd = 1.0f / sqrtf(acc / (float)hd + eps);
    if (w) for (int i = 0; i < hd; i++) v[i] = v[i] * rstd * (1.0f + w[i]);
    else for (int i = 0; i < hd; i++) v[i] = v[i] * rstd;
    const int pairs = rotary / 2;
    for (int i = 0; i < pairs; i++) {
        const float c = cos_p[i], s = sin_p[i];
        const float a = v[i], b = v[i + pairs];
        v[i] = a * c - b * s;
        v[i + pairs] = b * c + a * s;
    }
}

/* src/q35_model.c:1627-1652: the per-token loop of mixer_attn between the projections and the
 * attention.  q_proj heads are q_head_stride floats apart (the gate sits behind each head's
 * query when there is one).  Outputs are narrowed to bf16 with round-to-nearest-even (what the
 * device caches and kernels hold): q_out [n][H][HD], k_rows / v_rows [n][KV*HD]. */
ORC_API void orc_gqa_prepare(const float *q_proj, int64_t q_head_stride, const float *k_proj,
                             const float *v_proj, int64_t n, int64_t pos0, int H, int KV, int HD,
                             const float *q_norm, const float *k_norm, float eps,
                             const float *rope_cos, const float *rope_sin, int rotary,
                             uint16_t *q_out, uint16_t *k_rows, uint16_t *v_rows) {
    const int pairs = rotary / 2;
    float *tmp = malloc(sizeof(float) * (size_t)HD);
    for (int64_t t = 0; t < n; t++) {
        const float *cos_p = rope_cos + (size_t)(pos0 + t) * pairs;
        const float *sin_p = rope_sin + (size_t)(pos0 + t) * pairs;
        for (int h = 0; h < H; h++) {
            memcpy(tmp, q_proj + ((size_t)t * H + h) * q_head_stride, sizeof(float) * (size_t)HD);
            orc_head_norm_rope(tmp, HD, q_norm, eps, cos_p, sin_p, rotary);
            for (int i = 0; i < HD; i++) q_out[((size_t)t * H + h) * HD + i] = orc_f32_to_bf16_rne(tmp[i]);
        }
        for (int h = 0; h < KV; h++) {
            memcpy(tmp, k_proj + ((size_t)t * KV + h) * HD, sizeof(float) * (size_t)HD);
            orc_head_norm_rope(tmp, HD, k_norm, eps, cos_p, sin_p, rotary);
            for (int i = 0; i < HD; i++) k_rows[((size_t)t * KV + h) * HD + i] = orc_f32_to_bf16_rne(tmp[i]);
        }
        for (int i = 0; i < KV * HD; i++)
            v_rows[(size_t)t * KV * HD + i] = orc_f32_to_bf16_rne(v_proj[(size_t)t * KV * HD + i]);
    }
    free(tmp);
}

/* ------------------------------------------------------------------ */
/* top-k                                                               */
/* ------------------------------------------------------------------ */
/* The contract of src/ds_ops.h:110-112 ("ties keep the lower index") and of
 * BASELINE ("bit-exact with a lowest-index tie-break"): order by
 * (score descending, index ascending), keep the first k, emit them in
 * ascending index order.  -0.0 equals +0.0.  NaN sorts below -inf.
 * Straightforward O(n log n) sort: this is the definition, not an algorithm. */
typedef struct { uint32_t key; int32_t idx; } orc_pair;

static uint32_t orc_order_key(float f) {
    uint32_t u;
    if (f != f) return 0u;                       /* NaN: below everything */
    if (f == 0.0f) f = 0.0f;                     /* -0.0 -> +0.0 */
    memcpy(&u, &f, sizeof u);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return u == 0u ? 1u : u;                     /* keep 0 for NaN only */
}

ORC_API uint32_t orc_topk_order_key(float f) { return orc_order_key(f); }

static int orc_pair_cmp(const void *a, const void *b) {
    const orc_pair *x = a, *y = b;
    if (x->key != y->key) return x->key > y->key ? -1 : 1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}

static int orc_int_cmp(const void *a, const void *b) {
    int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
    return x < y ? -1 : (x > y ? 1 : 0);
}

ORC_API int64_t orc_topk_contract(const float *sc, int64_t n, int64_t k, int32_t *out) {
    if (k > n) k = n;
    if (k <= 0) return 0;
    orc_pair *p = malloc(sizeof(orc_pair) * (size_t)n);
    for (int64_t i = 0; i < n; i++) { p[i].key = orc_order_key(sc[i]); p[i].idx = (int32_t)i; }
    qsort(p, (size_t)n, sizeof(orc_pair), orc_pair_cmp);
    for (int64_t i = 0; i < k; i++) out[i] = p[i].idx;
    qsort(out, (size_t)k, sizeof(int32_t), orc_int_cmp);
    free(p);
    return k;
}

/* src/ds_ops.c:294-338 (ds_topk_scores + ds_heap_sift) restated: size-k
 * min-heap, `v <= heap[0]` skipped, indices insertion-sorted ascending.  On
 * ties that straddle the k-th value it evicts the earliest-inserted minimum,
 * so it is NOT the lowest-index rule; it agrees with orc_topk_contract on
 * tie-free input. */
static void orc_heap_sift(float *h, int *hi, int size, int i) {
    for (;;) {
        int l = 2 * i + 1, r = l + 1, m = i;
        if (l < size && h[l] < h[m]) m = l;
        if (r < size && h[r] < h[m]) m = r;
        if (m == i) break;
        float tf = h[i]; h[i] = h[m]; h[m] = tf;
        int ti = hi[i]; hi[i] = hi[m]; hi[m] = ti;
        i = m;
    }
}

ORC_API int orc_topk_heap(const float *sc, int n, int k, int *out) {
    if (k <= 0) return 0;
    float *heap = malloc(sizeof(float) * (size_t)k);
    int *hidx = malloc(sizeof(int) * (size_t)k);
    int size = 0;
    for (int t = 0; t < n; t++) {
        float v = sc[t];
        if (size == k) {
            if (v <= heap[0]) continue;
            heap[0] = v; hidx[0] = t;
            orc_heap_sift(heap, hidx, size, 0);
        } else {
            int i = size++;
            heap[i] = v; hidx[i] = t;
            while (i > 0) {
                int p = (i - 1) / 2;
                if (heap[p] <= heap[i]) break;
                float tf = heap[p]; heap[p] = heap[i]; heap[i] = tf;
                int ti = hidx[p]; hidx[p] = hidx[i]; hidx[i] = ti;
                i = p;
            }
        }
    }
    for (int i = 0; i < size; i++) out[i] = hidx[i];
    for (int i = 1; i < size; i++) {
        int v = out[i], j = i - 1;
        while (j >= 0 && out[j] > v) { out[j + 1] = out[j]; j--; }
        out[j + 1] = v;
    }
    free(heap); free(hidx);
    return size;
}

/* src/attention.c:529-543 (score_select, Hoare quickselect on a copy) and
 * :585-598 (threshold, then take `> thr` and `== thr` in ascending order):
 * the GLM selector, which does implement lowest-index ties.  Emits selected
 * indices in the reference's order (all `> thr` ascending, then `== thr`
 * ascending); with kpool == 1 and no tail rule this is the whole selector. */
static void orc_score_select(float *v, int64_t n, int64_t k) {
    int64_t lo = 0, hi = n - 1;
    while (lo < hi) {
        const float pivot = v[(size_t)(lo + hi) >> 1];
        int64_t i = lo, j = hi;
        while (i <= j) {
            while (v[i] > pivot) i++;
            while (v[j] < pivot) j--;
            if (i <= j) { float t = v[i]; v[i] = v[j]; v[j] = t; i++; j--; }
        }
        if (k <= j) hi = j;
        else if (k >= i) lo = i;
        else break;
    }
}

ORC_API int64_t orc_topk_quickselect(const float *sc, int64_t n, int64_t want, int32_t *out) {
    if (want <= 0 || n <= want) {
        for (int64_t i = 0; i < n; i++) out[i] = (int32_t)i;
        return n;
    }
    float *cp = malloc(sizeof(float) * (size_t)n);
    memcpy(cp, sc, sizeof(float) * (size_t)n);
    orc_score_select(cp, n, want);
    const float thr = cp[want - 1];
    int64_t m = 0;
    for (int pass = 0; pass < 2 && m < want; pass++)
        for (int64_t c = 0; c < n && m < want; c++) {
            const int take = pass == 0 ? (sc[c] > thr) : (sc[c] == thr);
            if (take) out[m++] = (int32_t)c;
        }
    free(cp);
    return m;
}

/* src/attention.c:548-622 after the scores (:585-620): which positions a query keeps.  `sc` holds
 * one score per closed pool (n_comp = npos / kp of them).  want = ceil(topk / kp) pools; when there
 * are no more pools than that the answer is "the whole prefix" (-1, :558-559).  Otherwise the pools
 * are chosen, each expands to its kp positions c kp + r (:592-598), the positions behind the last
 * closed pool are always kept (:603-604), and unless `strict` (CWICK_INDEXER_STRICT, :618-620) the
 * query's own position npos - 1 is added when it is not the last entry already.
 * The list keeps the reference's order: the pools above the threshold in ascending order, then
 * the pools that equal it, then the tail, then the query itself -- whose test looks at the last
 * entry only (:618), so a last pool that was selected above the threshold is followed by a second
 * copy of npos - 1; that is the reference's behaviour and it is kept.
 * faithful != 0: the pool choice as the reference makes it (threshold read at want - 1 after
 * score_select fixed position want: it can take fewer than `want` pools, see
 * orc_topk_quickselect).  faithful == 0: the pool choice by the contract (the `want` best by
 * score, ties to the lower index), which is what the device path implements; the two agree
 * whenever the reference's threshold is the smallest of its top set.  Returns the number of
 * positions written to sel, or -1. */
ORC_API int64_t orc_glm_select(const float *sc, int64_t n_comp, int64_t npos, int64_t kp, int64_t topk,
                               int strict, int faithful, int32_t *sel) {
    if (kp < 1) kp = 1;
    const int64_t want = (topk + kp - 1) / kp;
    if (want <= 0 || n_comp <= want) return -1;
    int32_t *pools = malloc(sizeof(int32_t) * (size_t)want);
    int64_t got;
    if (faithful) {
        got = orc_topk_quickselect(sc, n_comp, want, pools);
    } else {
        int32_t *asc = malloc(sizeof(int32_t) * (size_t)want);
        const int64_t m = orc_topk_contract(sc, n_comp, want, asc);
        float thr = INFINITY;
        for (int64_t i = 0; i < m; i++) if (sc[asc[i]] < thr) thr = sc[asc[i]];
        got = 0;
        for (int pass = 0; pass < 2; pass++)
            for (int64_t i = 0; i < m; i++) {
                const float v = sc[asc[i]];
                if (pass == 0 ? (v > thr) : (v == thr)) pools[got++] = asc[i];
            }
        free(asc);
    }
    int64_t n = 0;
    for (int64_t i = 0; i < got; i++)
        for (int64_t r = 0; r < kp; r++) sel[n++] = (int32_t)(pools[i] * kp + r);
    free(pools);
    const int64_t tail = npos % kp;
    for (int64_t r = 0; r < tail; r++) sel[n++] = (int32_t)(npos - tail + r);
    if (!strict && (n == 0 || sel[n - 1] != npos - 1)) sel[n++] = (int32_t)(npos - 1);
    return n;
}

/* src/attention.c:486-525 (indexer_absorb once the pool has closed): one compressed indexer
 * key from the pool's kp raw key rows and gate rows.  Statistics in double, everything else in
 * float, in the reference's order. */
ORC_API void orc_indexer_pool_row(const float *tail_k, const float *tail_g, const uint16_t *ape,
                                  const float *knw, const float *knb, float eps, int kp, int hd,
                                  float *dst) {
    float mean[8], inv[8];
    for (int i = 0; i < kp; i++) {
        const float *row = tail_k + (size_t)i * hd;
        double s = 0.0;
        for (int d = 0; d < hd; d++) s += (double)row[d];
        mean[i] = (float)(s / (double)hd);
        double v = 0.0;
        for (int d = 0; d < hd; d++) {
            double t = (double)row[d] - (double)mean[i];
            v += t * t;
        }
        inv[i] = 1.0f / sqrtf((float)(v / (double)hd) + eps);
    }
    for (int d = 0; d < hd; d++) {
        float mx = -INFINITY;
        for (int i = 0; i < kp; i++) {
            float lg = tail_g[(size_t)i * hd + d] + orc_bf16_to_f32(ape[(size_t)i * hd + d]);
            if (lg > mx) mx = lg;
        }
        float den = 0.0f, acc = 0.0f;
        for (int i = 0; i < kp; i++) {
            float lg = tail_g[(size_t)i * hd + d] + orc_bf16_to_f32(ape[(size_t)i * hd + d]);
            float p = expf(lg - mx);
            den += p;
            float nv = ((tail_k[(size_t)i * hd + d] - mean[i]) * inv[i]) * knw[d] + knb[d];
            acc += p * nv;
        }
        dst[d] = den > 0.0f ? acc / den : 0.0f;
    }
}

/* src/ds_model.c:1125-1144: level one of the two-level selection.  Block maxima, the partly
 * filled last block forced in, the `keep` best blocks by the reference's heap selector, and a
 * byte per position.  Returns the number of blocks kept. */
ORC_API int orc_candidate_mask(const float *scores, int nvis, int bs, int keep, uint8_t *cand) {
    const int nblk = (nvis + bs - 1) / bs;
    float *bsc = malloc(sizeof(float) * (size_t)nblk);
    int *blk = malloc(sizeof(int) * (size_t)(keep > 0 ? keep : 1));
    for (int b = 0; b < nblk; b++) {
        int hi = (b + 1) * bs; if (hi > nvis) hi = nvis;
        float mx = -INFINITY;
        for (int t = b * bs; t < hi; t++) if (scores[t] > mx) mx = scores[t];
        bsc[b] = mx;
    }
    bsc[(nvis - 1) / bs] = INFINITY;
    const int k = orc_topk_heap(bsc, nblk, keep, blk);
    memset(cand, 0, (size_t)nvis);
    for (int i = 0; i < k; i++) {
        int b = blk[i];
        int hi = (b + 1) * bs; if (hi > nvis) hi = nvis;
        for (int t = b * bs; t < hi; t++) cand[t] = 1;
    }
    free(bsc); free(blk);
    return k;
}

/* src/ds_model.c:1145-1148: scores outside the candidate blocks become -inf. */
ORC_API void orc_candidate_apply(float *scores, const uint8_t *cand, int nvis) {
    for (int t = 0; t < nvis; t++) if (!cand[t]) scores[t] = -INFINITY;
}

/* ------------------------------------------------------------------ */
/* MiniMax block selection (the second consumer of the gather decode)  */
/* ------------------------------------------------------------------ */

/* src/mm_model.c:1764-1780 (mm_index_scores): per position the dot of every index head's fp32
 * query with the position's bf16 index key, accumulated serially from 0 in dimension order,
 * ReLU, and the heads summed in head order.  No head weights.  The reference writes
 * `d += qh[i] * k[i]` and leaves contraction to its compiler (clang, which fuses by default);
 * this file is compiled with contraction off, so the fused form is spelled out. */
ORC_API void orc_mm_index_scores(const float *iq, const uint16_t *keys, int64_t limit, int ih, int id,
                                 float *scores) {
    for (int64_t s = 0; s < limit; s++) {
        const uint16_t *k = keys + (size_t)s * (size_t)id;
        float tot = 0.0f;
        for (int h = 0; h < ih; h++) {
            const float *qh = iq + (size_t)h * (size_t)id;
            float d = 0.0f;
            for (int i = 0; i < id; i++) d = fmaf(qh[i], orc_bf16_to_f32(k[i]), d);
            if (d > 0.0f) tot += d;
        }
        scores[s] = tot;
    }
}

/* src/mm_model.c:1733-1761 (mm_select_blocks) and :1969-1976 (the chosen blocks written out as
 * positions): a block scores the largest position score inside it, the `keep` best blocks are
 * taken by the heap selector (mm_topk, :777-814, the same sequence of comparisons and swaps as
 * ds_topk_scores on scores that are not NaN), and block limit / bs is added when it is not among
 * them -- when limit is a multiple of bs that is a block with no position written yet, which
 * then contributes no position.  blk_out holds keep + 1 entries; sel holds at most max_sel
 * positions.  Returns the number of blocks; *n_sel receives the number of positions. */
ORC_API int orc_mm_select_blocks(const float *scores, int64_t limit, int bs, int keep, int *blk_out,
                                 int64_t *sel, int64_t max_sel, int64_t *n_sel) {
    const int64_t nblk = (limit + bs - 1) / bs;
    float *bsc = malloc(sizeof(float) * (size_t)(nblk + 1));
    for (int64_t b = 0; b < nblk; b++) {
        int64_t s0 = b * bs, s1 = s0 + bs;
        if (s1 > limit) s1 = limit;
        float best = -1e30f;
        for (int64_t s = s0; s < s1; s++) best = fmaxf(best, scores[s]);
        bsc[b] = best;
    }
    int nb = orc_topk_heap(bsc, (int)nblk, keep, blk_out);
    const int newest = (int)(limit / bs);
    int have = 0;
    for (int i = 0; i < nb; i++) if (blk_out[i] == newest) have = 1;
    if (!have) blk_out[nb++] = newest;
    int64_t ns = 0;
    for (int b = 0; b < nb && ns < max_sel; b++) {
        int64_t s0 = (int64_t)blk_out[b] * bs, s1 = s0 + bs;
        if (s1 > limit) s1 = limit;
        for (int64_t s = s0; s < s1 && ns < max_sel; s++) sel[ns++] = s;
    }
    *n_sel = ns;
    free(bsc);
    return nb;
}

/* src/prof.c:39-43 (cwick_prof_ns): CLOCK_MONOTONIC in nanoseconds. */
ORC_API int64_t orc_now_ns(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (int64_t)ts.tv_sec * 1000000000ll + (int64_t)ts.tv_nsec;
}
