// merge.hpp -- second pass of split-K flash-decoding: combine the per-slice
// partials (m_s, l_s, acc_s) of one query row into the normalised output
//
//     out[d] = sum_s acc_s[d] e^{m_s - M} / sum_s l_s e^{m_s - M},  M = max_s m_s.
//
// One workgroup per (head, query).  The slice weights are computed once, in
// parallel over slices, and parked in LDS; the accumulation loop then has
// nothing but independent loads in it, so they overlap instead of paying one
// memory latency per slice.
#pragma once
#include "common.hpp"

namespace cwick {

constexpr int MERGE_MAX_SPLITS = 1024;

template <int DIM>
__global__ void __launch_bounds__(256)
splitk_merge_kernel(const float *__restrict__ part_acc,   // [y][split][head][DIM]
                    const float *__restrict__ part_ml,    // [y][split][head][2]
                    int n_splits, int n_heads, float *__restrict__ out /* [y][head][DIM] */) {
    __shared__ float w[MERGE_MAX_SPLITS];
    __shared__ float red[8];
    const int h = blockIdx.x, y = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const size_t base = (size_t)y * n_splits;

    float mx = -INFINITY;
    for (int s = tid; s < n_splits; s += 256) mx = fmaxf(mx, part_ml[((base + s) * n_heads + h) * 2]);
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

    float ls = 0.0f;
    for (int s = tid; s < n_splits; s += 256) {
        const float ms = part_ml[((base + s) * n_heads + h) * 2];
        const float c = ms == -INFINITY ? 0.0f : __expf(ms - mx);
        w[s] = c;
        ls += part_ml[((base + s) * n_heads + h) * 2 + 1] * c;
    }
    ls = wave_sum(ls);
    if (lane == 0) red[4 + wave] = ls;
    __syncthreads();
    const float l = (red[4] + red[5]) + (red[6] + red[7]);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;

    constexpr int PER = (DIM + 255) / 256;       // output elements per thread
    if (DIM < 256 && tid >= DIM) return;
    float acc[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) acc[j] = 0.0f;
    const float *pa = part_acc + (base * n_heads + h) * DIM + tid;
    const size_t stride = (size_t)n_heads * DIM;
#pragma unroll 8
    for (int s = 0; s < n_splits; s++) {
        const float c = w[s];
#pragma unroll
        for (int j = 0; j < PER; j++) acc[j] = __builtin_fmaf(pa[s * stride + j * 256], c, acc[j]);
    }
    float *o = out + ((size_t)y * n_heads + h) * DIM + tid;
#pragma unroll
    for (int j = 0; j < PER; j++) o[j * 256] = acc[j] * inv;
}

}  // namespace cwick
