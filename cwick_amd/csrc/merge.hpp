// merge.hpp -- second pass of split-K flash-decoding: combine the per-slice
// partials (m_s, l_s, acc_s) of one query row into the normalised output
//
//     out[d] = sum_s acc_s[d] e^{m_s - M} / sum_s l_s e^{m_s - M},  M = max_s m_s.
//
// One workgroup per (head, query); the loads of all slices are independent, so
// they overlap instead of paying one memory latency per slice.
#pragma once
#include "common.hpp"

namespace cwick {

constexpr int MERGE_MAX_SPLITS = 1024;

// Every load in flight at once: one workgroup per (head, query), up to 16
// waves; wave w takes slices w, w + n_waves, ... (eight per batch), lane = one float4 of the
// row; the waves meet in LDS.  Which slices exist is uniform per wave.
template <int DIM>
__global__ void __launch_bounds__(1024)
splitk_merge_wide_kernel(const float *__restrict__ part_acc,   // [y][split][head][DIM]
                         const float *__restrict__ part_ml,    // [y][split][head][2]
                         int n_splits, int n_heads, float *__restrict__ out /* [y][head][DIM] */) {
    static_assert(DIM % 4 == 0 && DIM <= 256, "one float4 per lane");
    __shared__ float red_m[16];
    __shared__ float red_l[16];
    __shared__ f32x4 red_a[16][64];
    const int h = blockIdx.x, y = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6), mw = (int)blockDim.x >> 6;
    const bool live = lane < DIM / 4;
    const size_t base = (size_t)y * n_splits;
    const float *ml = part_ml + (base * n_heads + h) * 2;
    const size_t ml_stride = (size_t)n_heads * 2;
    const float *pa = part_acc + (base * n_heads + h) * DIM + (live ? lane : 0) * 4;
    const size_t pa_stride = (size_t)n_heads * DIM;

    f32x4 a0[8];
    f32x2 v0[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int s = wv + mw * j;
        v0[j] = (f32x2){-INFINITY, 0.0f};
        a0[j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        if (s < n_splits) {
            v0[j] = *(const f32x2 *)(ml + s * ml_stride);
            a0[j] = *(const f32x4 *)(pa + s * pa_stride);
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; j++) mx = fmaxf(mx, v0[j][0]);
    for (int s = wv + 8 * mw; s < n_splits; s += mw) mx = fmaxf(mx, ml[s * ml_stride]);
    if (lane == 0) red_m[wv] = mx;
    __syncthreads();
    for (int w = 0; w < mw; w++) mx = fmaxf(mx, red_m[w]);

    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float ls = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float c = v0[j][0] == -INFINITY ? 0.0f : __expf(v0[j][0] - mx);
        ls = __builtin_fmaf(v0[j][1], c, ls);
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] = __builtin_fmaf(a0[j][r], c, acc[r]);
    }
    for (int s0 = wv + 8 * mw; s0 < n_splits; s0 += 8 * mw) {
        f32x4 a[8];
        f32x2 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = s0 + mw * j;
            v[j] = (f32x2){-INFINITY, 0.0f};
            a[j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
            if (s < n_splits) {
                v[j] = *(const f32x2 *)(ml + s * ml_stride);
                a[j] = *(const f32x4 *)(pa + s * pa_stride);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float c = v[j][0] == -INFINITY ? 0.0f : __expf(v[j][0] - mx);
            ls = __builtin_fmaf(v[j][1], c, ls);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = __builtin_fmaf(a[j][r], c, acc[r]);
        }
    }
    if (lane == 0) red_l[wv] = ls;
    red_a[wv][lane] = acc;
    __syncthreads();
    if (wv != 0 || !live) return;
    float l = 0.f;
    f32x4 r4 = {0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < mw; w++) {
        l += red_l[w];
        const f32x4 t = red_a[w][lane];
#pragma unroll
        for (int r = 0; r < 4; r++) r4[r] += t[r];
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) r4[r] *= inv;
    *(f32x4 *)(out + ((size_t)y * n_heads + h) * DIM + lane * 4) = r4;
}

}  // namespace cwick
