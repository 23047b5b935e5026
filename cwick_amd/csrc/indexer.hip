// indexer.hip -- lightning-indexer scores with a fixed, documented summation
// order (the score loop of indexer_select, src/attention.c:573-582, and of
// ds_indexer, src/ds_model.c:1108-1121):
//
//     sc[t] = sum_h relu(q_h . k_t) * w[h]
//
// The top-k that follows must be bit-exact against the CPU, which is only
// possible if the scores themselves are bit-identical.  So this kernel does
// not use the matrix cores: their accumulation order is not specified.  It
// runs the dot products on the vector ALU in exactly the order of the
// reference's dot_f32 (src/attention.c:249-258), one key per lane:
//
//     s0..s3 over dims i = 0,4,8,..   s_j = fma(e[i+j], q[h][i+j], s_j)
//     d  = (s0 + s1) + (s2 + s3)
//     d  = d * kscale[t]              per-token FP8 scale (positive: commutes
//                                     with the ReLU)
//     d  = d < 0 ? 0 : d
//     s  = s + (d * w[h])             multiply, then add; not fused
//
// e[] are the raw E4M3 values of the key and q the bf16 query widened to fp32;
// the product of a 4-bit and an 8-bit significand is exact in fp32, so the fma
// rounds exactly like the CPU's multiply-then-add.  This file is compiled with
// -ffp-contract=off so nothing else is fused.
//
// Layout: one key per lane, its 128 E4M3 bytes held as 128 fp32 registers for
// the whole head loop; q[h][i] is wave-uniform: the workgroup widens q to fp32
// in LDS, a lane holds sixteenths of a head in eight registers and each FMA
// picks its value with a DPP row broadcast.
// VALU-bound: ih*hd fused multiply-adds per key, and a SIMD retires one wave-wide
// VALU instruction per four cycles however many waves it holds (the oldest wave
// of a SIMD issues one every five cycles, the others share what is left).
#include "common.hpp"

namespace cwick {

constexpr int IDX_HD = CWICK_HIP_INDEX_DIM;   // 128
constexpr int IDX_THREADS = 256;

__global__ void __launch_bounds__(IDX_THREADS)
indexer_scores_kernel(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                      int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                      const uint16_t *__restrict__ q,  // [batch][ih][128] bf16
                      const float *__restrict__ w,     // [batch][ih]
                      int ih, float *__restrict__ scores,
                      const IndexerBandRow *__restrict__ rows, int cap) {
    const int b = blockIdx.y;
    // after a banded select: only the rows whose band failed are computed
    if (rows && !indexer_band_failed(rows[b], cap)) return;
    const int64_t t = (int64_t)blockIdx.x * IDX_THREADS + threadIdx.x;
    const bool live = t < n_keys;
    const int64_t tc = live ? t : n_keys - 1;
    const uint8_t *krow = keys + (size_t)b * key_bstride + (size_t)tc * IDX_HD;
    const float ks = kscale[(size_t)b * kscale_bstride + tc];
    const uint16_t *qb = q + (size_t)b * ih * IDX_HD;
    const float *wb = w + (size_t)b * ih;

    float e[IDX_HD];
#pragma unroll
    for (int c = 0; c < IDX_HD / 16; c++) {
        const u32x4 v = *(const u32x4 *)(krow + c * 16);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const f32x2 lo = e4m3x2_to_f32<false>(v[j]);
            const f32x2 hi = e4m3x2_to_f32<true>(v[j]);
            e[c * 16 + j * 4 + 0] = lo[0];
            e[c * 16 + j * 4 + 1] = lo[1];
            e[c * 16 + j * 4 + 2] = hi[0];
            e[c * 16 + j * 4 + 3] = hi[1];
        }
    }

    // q[h][i] reaches the FMAs through DPP row broadcasts: lane l holds q[h][16 c + (l & 15)] in
    // register c, and the FMA of element 16 c + n reads lane n of its own row of 16.  The
    // workgroup first widens q to fp32 in LDS, laid out [head][n][c] so that a lane fetches its
    // eight values of a head with two 16-byte reads, one head ahead of their use.  (Scalar loads
    // of q -- one SGPR operand per FMA -- left the waves waiting on the scalar cache for 60 % of
    // their cycles: the eight 64-byte loads of a head cannot be issued far enough ahead within
    // the SGPR budget.  Vector loads from global memory a head ahead still wait: their latency
    // exceeds the 128 FMAs of a head.)
    __shared__ __attribute__((aligned(16))) float qs[64 * IDX_HD];
    for (int idx = threadIdx.x; idx < ih * (IDX_HD / 8); idx += IDX_THREADS) {
        const u32x4 v = *(const u32x4 *)(qb + (size_t)idx * 8);       // dims i0 .. i0+7 of head h
        const int h = idx / (IDX_HD / 8), i0 = (idx % (IDX_HD / 8)) * 8;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = i0 + j;
            const uint32_t pair = v[j >> 1];
            qs[h * IDX_HD + (i & 15) * 8 + (i >> 4)] = (j & 1) ? bf16hi_to_f32(pair) : bf16lo_to_f32(pair);
        }
    }
    __syncthreads();
    const f32x4 *qlane = (const f32x4 *)(qs + (threadIdx.x & 15) * 8);
    // the head weights live in one register (lane h holds w[h]) and are picked by readlane: a
    // scalar load per head would be waited for in full at the end of every head
    float wv = wb[(threadIdx.x & 63) < ih ? (threadIdx.x & 63) : 0];
    float ksr = ks;
    asm volatile("" : "+v"(ksr), "+v"(wv));                       // the scale has arrived before the loop: no full wait inside it
    f32x4 qa[2], qn[2];
    qa[0] = qlane[0];
    qa[1] = qlane[1];
    float s = 0.0f;
    // two heads per trip so that the two register sets alternate without copies (a DPP read of
    // a register that a VALU move has just written needs wait states the compiler cannot see
    // inside inline assembly)
    auto head = [&](int h, const f32x4 (&q)[2], f32x4 (&qnext)[2]) {
        const int hn = h + 1 < ih ? h + 1 : h;
        qnext[0] = qlane[hn * (IDX_HD / 4)];
        qnext[1] = qlane[hn * (IDX_HD / 4) + 1];
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
        for (int c = 0; c < IDX_HD / 16; c++) {
#define CWICK_IDX_FMA(acc, n)                                                                      \
    asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #n " row_mask:0xf bank_mask:0xf"             \
        : "+v"(acc) : "v"(q[c >> 2][c & 3]), "v"(e[16 * c + n]))
            CWICK_IDX_FMA(s0, 0);  CWICK_IDX_FMA(s1, 1);  CWICK_IDX_FMA(s2, 2);  CWICK_IDX_FMA(s3, 3);
            CWICK_IDX_FMA(s0, 4);  CWICK_IDX_FMA(s1, 5);  CWICK_IDX_FMA(s2, 6);  CWICK_IDX_FMA(s3, 7);
            CWICK_IDX_FMA(s0, 8);  CWICK_IDX_FMA(s1, 9);  CWICK_IDX_FMA(s2, 10); CWICK_IDX_FMA(s3, 11);
            CWICK_IDX_FMA(s0, 12); CWICK_IDX_FMA(s1, 13); CWICK_IDX_FMA(s2, 14); CWICK_IDX_FMA(s3, 15);
#undef CWICK_IDX_FMA
        }
        float d = (s0 + s1) + (s2 + s3);
        d = d * ksr;
        d = d < 0.0f ? 0.0f : d;
        const float wh = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), h));
        const float prod = d * wh;
        s = s + prod;
    };
    for (int h = 0; h < ih; h += 2) {
        head(h, qa, qn);
        if (h + 1 < ih) head(h + 1, qn, qa);
    }
    if (live) scores[(size_t)b * n_keys + t] = s;
}

int launch_indexer_scores(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys,
                          const uint16_t *q_idx, const float *w, int n_idx_heads, float *scores,
                          hipStream_t s) {
    CWICK_REQUIRE(keys && kscale && q_idx && w && scores, "indexer_scores: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535, "indexer_scores: batch %d", batch);
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= ((int64_t)1 << 30), "indexer_scores: n_keys %lld",
                  (long long)n_keys);
    CWICK_REQUIRE(n_idx_heads >= 1 && n_idx_heads <= 64, "indexer_scores: n_idx_heads %d (1..64)",
                  n_idx_heads);
    CWICK_REQUIRE((uintptr_t)keys % 16 == 0 && key_bstride % 16 == 0 && (uintptr_t)q_idx % 16 == 0,
                  "indexer_scores: keys and q must be 16-byte aligned");
    dim3 grid((unsigned)((n_keys + IDX_THREADS - 1) / IDX_THREADS), batch);
    {
        ProfScope ps(CWICK_HIP_PROF_INDEXER, s);
        indexer_scores_kernel<<<grid, IDX_THREADS, 0, s>>>(keys, kscale, key_bstride, kscale_bstride,
                                                           n_keys, q_idx, w, n_idx_heads, scores, nullptr, 0);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_indexer_scores_rows(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                               int64_t kscale_bstride, int batch, int64_t n_keys,
                               const uint16_t *q_idx, const float *w, int n_idx_heads, float *scores,
                               const IndexerBandRow *rows, int cap, hipStream_t s) {
    CWICK_REQUIRE(rows, "indexer_scores_rows: null pointer");
    dim3 grid((unsigned)((n_keys + IDX_THREADS - 1) / IDX_THREADS), batch);
    indexer_scores_kernel<<<grid, IDX_THREADS, 0, s>>>(keys, kscale, key_bstride, kscale_bstride,
                                                       n_keys, q_idx, w, n_idx_heads, scores, rows, cap);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
