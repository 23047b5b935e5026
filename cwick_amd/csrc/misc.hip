// misc.hip -- cache-append kernels (fp32 -> FP8 rows with block scales, fp32 ->
// bf16 rows) and the E4M3 decode self-check.  None of these is on the timed
// path; they exist so the engine can append rows to the device caches.
#include "common.hpp"

namespace cwick {

// One wave per (row, block): amax by wave reduction, then each lane encodes
// block/64 elements.  scale = amax/448, 1 for an all-zero block.
template <int DIM, int BLOCK>
__global__ void __launch_bounds__(256) quant_rows_kernel(const float *__restrict__ src, int64_t n,
                                                         uint8_t *__restrict__ dst,
                                                         float *__restrict__ scales) {
    constexpr int NBLK = (DIM + BLOCK - 1) / BLOCK;
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= n * NBLK) return;
    const int64_t row = item / NBLK;
    const int b = (int)(item % NBLK);
    const int c0 = b * BLOCK;
    const int len = (DIM - c0) < BLOCK ? (DIM - c0) : BLOCK;
    const float *x = src + row * DIM + c0;
    float amax = 0.0f;
    for (int i = lane; i < len; i += 64) amax = fmaxf(amax, fabsf(x[i]));
    amax = wave_max(amax);
    const float s = amax > 0.0f ? amax / 448.0f : 1.0f;
    if (lane == 0) scales[row * NBLK + b] = s;
    for (int i = lane; i < len; i += 64) {
        float v = x[i] / s;
        v = fminf(fmaxf(v, -448.0f), 448.0f);
        dst[row * DIM + c0 + i] = (uint8_t)f32_to_e4m3_rne(v);
    }
}

__global__ void __launch_bounds__(256) narrow_bf16_kernel(const float *__restrict__ src, int64_t n,
                                                          uint16_t *__restrict__ dst) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = (uint16_t)f32_to_bf16_rne(src[i]);
}

// bf16 rows back to fp32 (q35_widen_rows, src/q35_model.c:1543-1556): exact
__global__ void __launch_bounds__(256) widen_bf16_kernel(const uint16_t *__restrict__ src, int64_t n,
                                                         float *__restrict__ dst) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = bf16_to_f32(src[i]);
}

__global__ void __launch_bounds__(256) e4m3_table_kernel(float *out) {
    const uint32_t b = threadIdx.x;
    // the byte in the low and in the high half of the word must decode alike
    f32x2 lo = e4m3x2_to_f32<false>(b | (b << 8));
    f32x2 hi = e4m3x2_to_f32<true>((b << 16) | (b << 24));
    uint32_t bw = e4m3x2_to_bf16x2<false>(b | (b << 8));
    float vb = bf16lo_to_f32(bw);
    bool same = (__builtin_bit_cast(uint32_t, lo[0]) == __builtin_bit_cast(uint32_t, lo[1])) &&
                (__builtin_bit_cast(uint32_t, lo[0]) == __builtin_bit_cast(uint32_t, hi[0])) &&
                (__builtin_bit_cast(uint32_t, lo[0]) == __builtin_bit_cast(uint32_t, hi[1])) &&
                (__builtin_bit_cast(uint32_t, lo[0]) == __builtin_bit_cast(uint32_t, vb) ||
                 (lo[0] != lo[0] && vb != vb));
    // a disagreement between the conversion paths shows up as a value no E4M3
    // byte decodes to
    out[b] = same ? lo[0] : 12345.0f;
}

int launch_quant_latent(const float *rows, int64_t n, uint8_t *out_rows, float *out_scales,
                        hipStream_t s) {
    CWICK_REQUIRE(rows && out_rows && out_scales && n > 0, "quant_latent: bad argument");
    int64_t items = n * CWICK_HIP_LATENT_NBLK;
    dim3 grid((unsigned)((items + 3) / 4));
    quant_rows_kernel<CWICK_HIP_LATENT_KDIM, CWICK_HIP_LATENT_BLOCK>
        <<<grid, 256, 0, s>>>(rows, n, out_rows, out_scales);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_quant_ikeys(const float *rows, int64_t n, uint8_t *out_rows, float *out_scales,
                       hipStream_t s) {
    CWICK_REQUIRE(rows && out_rows && out_scales && n > 0, "quant_ikeys: bad argument");
    dim3 grid((unsigned)((n + 3) / 4));
    quant_rows_kernel<CWICK_HIP_INDEX_DIM, CWICK_HIP_INDEX_DIM>
        <<<grid, 256, 0, s>>>(rows, n, out_rows, out_scales);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_narrow_bf16(const float *src, int64_t n, uint16_t *dst, hipStream_t s) {
    CWICK_REQUIRE(src && dst && n > 0, "narrow_bf16: bad argument");
    int64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    narrow_bf16_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(src, n, dst);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_widen_bf16(const uint16_t *src, int64_t n, float *dst, hipStream_t s) {
    CWICK_REQUIRE(src && dst && n > 0, "widen_bf16: bad argument");
    int64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    widen_bf16_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(src, n, dst);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

// one wave: every lane-exchange primitive of common.hpp on the 64 words of `in`
__global__ void __launch_bounds__(64) lane_ops_kernel(const uint32_t *__restrict__ in, uint32_t *__restrict__ out) {
    const int l = threadIdx.x;
    const uint32_t v = in[l];
    const float f = __builtin_bit_cast(float, (v & 0x007FFFFFu) | 0x3F800000u);      // in [1, 2)
    out[l] = wave_sum_u32(v);
    out[64 + l] = wave_max_u32(v);
    out[128 + l] = wave_min_u32(v);
    out[192 + l] = wave_scan_u32(v);
    out[256 + l] = __builtin_bit_cast(uint32_t, wave_max(f));
    out[320 + l] = __builtin_bit_cast(uint32_t, xor16_max(f));
    out[384 + l] = __builtin_bit_cast(uint32_t, xor32_max(f));
    out[448 + l] = __builtin_bit_cast(uint32_t, xor16_sum(f));
    out[512 + l] = __builtin_bit_cast(uint32_t, xor32_sum(f));
    out[576 + l] = __builtin_bit_cast(uint32_t, group_step_sum<2>(f));
    out[640 + l] = __builtin_bit_cast(uint32_t, group_step_sum<4>(group_step_sum<2>(f)));
    out[704 + l] = __builtin_bit_cast(uint32_t, group_step_sum<8>(group_step_sum<4>(group_step_sum<2>(f))));
    out[768 + l] = __builtin_bit_cast(uint32_t, group_step_sum<16>(group_step_sum<8>(group_step_sum<4>(group_step_sum<2>(f)))));
}

int launch_lane_ops(const uint32_t *in64_dev, uint32_t *out832_dev, hipStream_t s) {
    lane_ops_kernel<<<1, 64, 0, s>>>(in64_dev, out832_dev);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_e4m3_table(float *out256_dev, hipStream_t s) {
    e4m3_table_kernel<<<1, 256, 0, s>>>(out256_dev);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
