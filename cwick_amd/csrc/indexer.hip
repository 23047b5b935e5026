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
// the whole head loop; q[h][i] is wave-uniform and comes in through scalar
// loads from a small fp32 copy of q that a prologue kernel writes.
// VALU-bound: ih*hd fused multiply-adds per key.
#include "common.hpp"

namespace cwick {

constexpr int IDX_HD = CWICK_HIP_INDEX_DIM;   // 128
constexpr int IDX_THREADS = 256;

__global__ void __launch_bounds__(256)
indexer_widen_q_kernel(const uint16_t *__restrict__ q, int n, float *__restrict__ qf) {
    int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) qf[i] = bf16_to_f32(q[i]);
}

__global__ void __launch_bounds__(IDX_THREADS)
indexer_scores_kernel(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                      int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                      const float *__restrict__ qf,   // [batch][ih][128] fp32
                      const float *__restrict__ w,    // [batch][ih]
                      int ih, float *__restrict__ scores) {
    const int b = blockIdx.y;
    const int64_t t = (int64_t)blockIdx.x * IDX_THREADS + threadIdx.x;
    const bool live = t < n_keys;
    const int64_t tc = live ? t : n_keys - 1;
    const uint8_t *krow = keys + (size_t)b * key_bstride + (size_t)tc * IDX_HD;
    const float ks = kscale[(size_t)b * kscale_bstride + tc];
    const float *qb = qf + (size_t)b * ih * IDX_HD;
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

    float s = 0.0f;
    for (int h = 0; h < ih; h++) {
        const float *qh = qb + (size_t)h * IDX_HD;   // wave-uniform address
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
        for (int i = 0; i < IDX_HD; i += 4) {
            s0 = __builtin_fmaf(e[i + 0], qh[i + 0], s0);
            s1 = __builtin_fmaf(e[i + 1], qh[i + 1], s1);
            s2 = __builtin_fmaf(e[i + 2], qh[i + 2], s2);
            s3 = __builtin_fmaf(e[i + 3], qh[i + 3], s3);
        }
        float d = (s0 + s1) + (s2 + s3);
        d = d * ks;
        d = d < 0.0f ? 0.0f : d;
        const float prod = d * wb[h];
        s = s + prod;
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
    CWICK_REQUIRE((uintptr_t)keys % 16 == 0 && key_bstride % 16 == 0,
                  "indexer_scores: keys must be 16-byte aligned");
    const int nq = batch * n_idx_heads * IDX_HD;
    float *qf = (float *)workspace(s, (size_t)nq * sizeof(float));
    CWICK_REQUIRE(qf, "indexer_scores: workspace allocation failed");
    indexer_widen_q_kernel<<<(nq + 255) / 256, 256, 0, s>>>(q_idx, nq, qf);
    CWICK_HIP_CALL(hipGetLastError());
    dim3 grid((unsigned)((n_keys + IDX_THREADS - 1) / IDX_THREADS), batch);
    {
        ProfScope ps(CWICK_HIP_PROF_INDEXER, s);
        indexer_scores_kernel<<<grid, IDX_THREADS, 0, s>>>(keys, kscale, key_bstride, kscale_bstride,
                                                           n_keys, qf, w, n_idx_heads, scores);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
