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
#include "indexer_exact.hpp"

namespace cwick {

__global__ void __launch_bounds__(IDX_THREADS)
indexer_scores_kernel(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                      int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                      const uint16_t *__restrict__ q,  // [batch][ih][128] bf16
                      const float *__restrict__ w,     // [batch][ih]
                      int ih, float *__restrict__ scores) {
    indexer_exact_block(keys, kscale, key_bstride, kscale_bstride, n_keys, q, w, ih, scores, blockIdx.y, blockIdx.x);
}

// The DeepSeek flavour of the same loop (ds_indexer, src/ds_model.c:1099-1121), bit for bit:
//
//     kt[i] = e4m3(key[t][i]) * kscale[t]          the dequantised key the reference holds in fp32
//     d     = 0;  d = d + (q_h[i] * kt[i])         i = 0..127 in order, multiply and add rounded
//                                                  separately (the product of an 8-bit and a
//                                                  24-bit significand is not exact: no fma)
//     d     = bf16_round(d)                        round-to-nearest-even onto the bf16 grid
//     s     = s + d * bf16_round(w[h])  if d > 0   multiply, then add
//
// One key per lane, its 128 dequantised values in registers; q is widened to fp32 in LDS and
// every lane reads the same address (a broadcast).  Twice the vector-ALU work of the kernel
// above and one dependent chain per head: this is the mode for checking against that CPU path,
// not the fast one.
__global__ void __launch_bounds__(IDX_THREADS)
indexer_scores_ds_kernel(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                         int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                         const uint16_t *__restrict__ q, const float *__restrict__ w, int ih,
                         float *__restrict__ scores) {
    __shared__ __attribute__((aligned(16))) float qs[64 * IDX_HD];
    __shared__ float ws[64];
    const int b = blockIdx.y;
    const int64_t t = (int64_t)blockIdx.x * IDX_THREADS + threadIdx.x;
    const bool live = t < n_keys;
    const int64_t tc = live ? t : n_keys - 1;
    const uint8_t *krow = keys + (size_t)b * key_bstride + (size_t)tc * IDX_HD;
    const float ks = kscale[(size_t)b * kscale_bstride + tc];
    const uint16_t *qb = q + (size_t)b * ih * IDX_HD;
    for (int i = threadIdx.x; i < ih * IDX_HD; i += IDX_THREADS) qs[i] = bf16_to_f32(qb[i]);
    if ((int)threadIdx.x < ih)
        ws[threadIdx.x] = __builtin_bit_cast(float, f32_to_bf16_rne(w[(size_t)b * ih + threadIdx.x]) << 16);
    float e[IDX_HD];
#pragma unroll
    for (int c = 0; c < IDX_HD / 16; c++) {
        const u32x4 v = *(const u32x4 *)(krow + c * 16);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const f32x2 lo = e4m3x2_to_f32<false>(v[j]);
            const f32x2 hi = e4m3x2_to_f32<true>(v[j]);
            e[c * 16 + j * 4 + 0] = lo[0] * ks;
            e[c * 16 + j * 4 + 1] = lo[1] * ks;
            e[c * 16 + j * 4 + 2] = hi[0] * ks;
            e[c * 16 + j * 4 + 3] = hi[1] * ks;
        }
    }
    __syncthreads();
    float s = 0.0f;
    for (int h = 0; h < ih; h++) {
        const f32x4 *qh = (const f32x4 *)(qs + h * IDX_HD);
        float d = 0.0f;
#pragma unroll
        for (int c = 0; c < IDX_HD / 4; c++) {
            const f32x4 qv = qh[c];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float prod = qv[j] * e[4 * c + j];
                d = d + prod;
            }
        }
        d = __builtin_bit_cast(float, f32_to_bf16_rne(d) << 16);
        if (d > 0.0f) {
            const float prod = d * ws[h];
            s = s + prod;
        }
    }
    if (live) scores[(size_t)b * n_keys + t] = s;
}

int launch_indexer_scores(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys,
                          const uint16_t *q_idx, const float *w, int n_idx_heads, int mode,
                          float *scores, hipStream_t s) {
    CWICK_REQUIRE(keys && kscale && q_idx && w && scores, "indexer_scores: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535, "indexer_scores: batch %d", batch);
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= ((int64_t)1 << 30), "indexer_scores: n_keys %lld",
                  (long long)n_keys);
    CWICK_REQUIRE(n_idx_heads >= 1 && n_idx_heads <= 64, "indexer_scores: n_idx_heads %d (1..64)",
                  n_idx_heads);
    CWICK_REQUIRE(mode == CWICK_HIP_INDEXER_GLM || mode == CWICK_HIP_INDEXER_DS,
                  "indexer_scores: unknown mode %d", mode);
    CWICK_REQUIRE((uintptr_t)keys % 16 == 0 && key_bstride % 16 == 0 && (uintptr_t)q_idx % 16 == 0,
                  "indexer_scores: keys and q must be 16-byte aligned");
    dim3 grid((unsigned)((n_keys + IDX_THREADS - 1) / IDX_THREADS), batch);
    {
        ProfScope ps(CWICK_HIP_PROF_INDEXER, s);
        if (mode == CWICK_HIP_INDEXER_DS)
            indexer_scores_ds_kernel<<<grid, IDX_THREADS, 0, s>>>(keys, kscale, key_bstride, kscale_bstride,
                                                                  n_keys, q_idx, w, n_idx_heads, scores);
        else
            indexer_scores_kernel<<<grid, IDX_THREADS, 0, s>>>(keys, kscale, key_bstride, kscale_bstride,
                                                               n_keys, q_idx, w, n_idx_heads, scores);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
