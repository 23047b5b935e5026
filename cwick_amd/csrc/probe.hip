// probe.hip -- the two ceilings the attention kernels are judged against, measured on the device
// in hand rather than taken from the data sheet: a 128-bit grid-stride read over a buffer far
// larger than the caches (the `uint4` grid-stride sum of the reference's tools/gpubw.m, read
// rate of docs/PERF.md:997-1042) and a dense loop of matrix instructions with nothing else in it
// (bf16 32x32x16, and the FP8 16x16x128 form the MLA score kernel uses).  bench.py reports every
// kernel as a fraction of the published peak and of these.
#include "common.hpp"

namespace cwick {
namespace {

typedef __attribute__((ext_vector_type(8))) int i32x8;

__global__ void __launch_bounds__(256) probe_read_kernel(const u32x4 *__restrict__ src, size_t n16,
                                                         uint32_t *__restrict__ sink) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    u32x4 acc = {0u, 0u, 0u, 0u};
    // four loads in flight per lane
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const u32x4 a = __builtin_nontemporal_load(src + i);
        const u32x4 b = __builtin_nontemporal_load(src + i + stride);
        const u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride);
        const u32x4 d = __builtin_nontemporal_load(src + i + 3 * stride);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < n16; i += stride) acc ^= src[i];
    const uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (x == 0x9E3779B9u) sink[0] = x;                // never true for the fill pattern: keeps the loads alive
}

__global__ void __launch_bounds__(256) probe_fill_kernel(u32x4 *dst, size_t n16) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < n16; i += stride) dst[i] = (u32x4){(uint32_t)i, 1u, 2u, 3u};
}

// KIND 0: v_mfma_f32_32x32x16_bf16 (32768 flop), KIND 1: v_mfma_scale_f32_16x16x128_f8f6f4 on
// E4M3 operands (65536 flop).  Four independent accumulators per wave, four waves per SIMD.
template <int KIND>
__global__ void __launch_bounds__(256) probe_mfma_kernel(int iters, float *__restrict__ sink) {
    const int lane = threadIdx.x & 63;
    float total = 0.0f;
    if (KIND == 0) {
        bf16x8 a, b;
#pragma unroll
        for (int i = 0; i < 8; i++) { a[i] = (__bf16)(float)((lane + i) & 3); b[i] = (__bf16)(float)((lane >> 3) & 1); }
        f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
        for (int it = 0; it < iters; it++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
        }
        total = c0[0] + c1[1] + c2[2] + c3[3];
    } else {
        i32x8 a, b;
#pragma unroll
        for (int i = 0; i < 8; i++) { a[i] = 0x38383838 + lane; b[i] = 0x30303030 + i; }
        f32x4 c0 = {}, c1 = {}, c2 = {}, c3 = {};
        for (int it = 0; it < iters; it++) {
            c0 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c0, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            c1 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c1, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            c2 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c2, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            c3 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c3, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
        }
        total = c0[0] + c1[1] + c2[2] + c3[3];
    }
    if (total == 12345.678f) sink[0] = total;
}

}  // namespace

// best of `reps` timed launches, in GB/s (read) or TFLOP/s (mfma)
int run_probe_hbm_read(size_t bytes, int reps, double *gbps) {
    CWICK_REQUIRE(gbps && reps >= 1 && reps <= 1000, "probe_hbm_read: bad argument");
    CWICK_REQUIRE(bytes >= ((size_t)1 << 20) && bytes <= ((size_t)64 << 30) && bytes % 16 == 0,
                  "probe_hbm_read: bytes %zu (1 MiB .. 64 GiB, a multiple of 16)", bytes);
    void *buf = nullptr;
    uint32_t *sink = nullptr;
    CWICK_HIP_CALL(hipMalloc(&buf, bytes));
    if (!hip_ok(hipMalloc((void **)&sink, 256), "hipMalloc(sink)")) { (void)hipFree(buf); return 0; }
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const size_t n16 = bytes / 16;
    const unsigned grid = (unsigned)(num_cus() * 16);
    probe_fill_kernel<<<grid, 256>>>((u32x4 *)buf, n16);
    probe_read_kernel<<<grid, 256>>>((const u32x4 *)buf, n16, sink);      // warm-up
    float best = 1e30f;
    int ok = 1;
    for (int r = 0; r < reps && ok; r++) {
        (void)hipEventRecord(e0, nullptr);
        probe_read_kernel<<<grid, 256>>>((const u32x4 *)buf, n16, sink);
        (void)hipEventRecord(e1, nullptr);
        float ms = 0.0f;
        ok = hip_ok(hipEventSynchronize(e1), "probe_hbm_read") && hip_ok(hipEventElapsedTime(&ms, e0, e1), "probe_hbm_read");
        if (ms > 0.0f && ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(buf);
    (void)hipFree(sink);
    if (!ok) return 0;
    *gbps = (double)bytes / ((double)best * 1e-3) / 1e9;
    return 1;
}

int run_probe_mfma(int kind, int reps, double *tflops) {
    CWICK_REQUIRE(tflops && reps >= 1 && reps <= 1000, "probe_mfma: bad argument");
    CWICK_REQUIRE(kind == 0 || kind == 1, "probe_mfma: kind %d (0 bf16 32x32x16, 1 fp8 16x16x128)", kind);
    float *sink = nullptr;
    CWICK_HIP_CALL(hipMalloc((void **)&sink, 256));
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const int iters = 4096;
    const unsigned grid = (unsigned)(num_cus() * 4);                     // 16 waves per CU, 4 per SIMD
    const double flop = (double)grid * 4 /*waves*/ * iters * 4 /*mfma*/ * (kind == 0 ? 32768.0 : 65536.0);
    float best = 1e30f;
    int ok = 1;
    for (int r = 0; r < reps + 1 && ok; r++) {                           // the first launch is the warm-up
        (void)hipEventRecord(e0, nullptr);
        if (kind == 0) probe_mfma_kernel<0><<<grid, 256>>>(iters, sink);
        else probe_mfma_kernel<1><<<grid, 256>>>(iters, sink);
        (void)hipEventRecord(e1, nullptr);
        float ms = 0.0f;
        ok = hip_ok(hipEventSynchronize(e1), "probe_mfma") && hip_ok(hipEventElapsedTime(&ms, e0, e1), "probe_mfma");
        if (r > 0 && ms > 0.0f && ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (!ok) return 0;
    *tflops = flop / ((double)best * 1e-3) / 1e12;
    return 1;
}

}  // namespace cwick
