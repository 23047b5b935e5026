// indexer_exact.hpp -- the exact indexer's work for one block of 256 keys, shared by the
// stand-alone kernel (indexer.hip) and by the banded select's rescoring kernel, which runs it
// for the rows that did not fit the band (indexer_band.hip).  Both files are compiled with
// -ffp-contract=off; indexer.hip says why and describes the arithmetic.
#pragma once
#include "common.hpp"

namespace cwick {

constexpr int IDX_HD = CWICK_HIP_INDEX_DIM;   // 128
constexpr int IDX_THREADS = 256;

// one block of IDX_THREADS keys of batch row b, by a whole workgroup of IDX_THREADS (contains
// a workgroup barrier; a caller that runs it again must put one between the calls: the query
// staged in LDS is read until the end)
__device__ __forceinline__ void indexer_exact_block(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                                                    int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                                                    const uint16_t *__restrict__ q,  // [batch][ih][128] bf16
                                                    const float *__restrict__ w,     // [batch][ih]
                                                    int ih, float *__restrict__ scores, int b, int64_t block) {
    const int64_t t = block * IDX_THREADS + threadIdx.x;
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

}  // namespace cwick
