// common.hpp -- shared declarations of libcwick_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/cwick_hip.h"

namespace cwick {

// ---- error reporting -------------------------------------------------------
// Every extern "C" entry point returns 0 ("declined") after recording why.
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();
bool hip_ok(hipError_t e, const char *what);   // records the error text on failure

#define CWICK_REQUIRE(cond, ...)            \
    do {                                    \
        if (!(cond)) {                      \
            ::cwick::set_error(__VA_ARGS__); \
            return 0;                       \
        }                                   \
    } while (0)

#define CWICK_HIP_CALL(expr)                          \
    do {                                              \
        if (!::cwick::hip_ok((expr), #expr)) return 0; \
    } while (0)

// ---- runtime ---------------------------------------------------------------
bool backend_ready();                       // device 0 is up and selected
int num_cus();
// Grow-only scratch keyed by stream and slot.  A call's buffer stays valid for the kernels it
// enqueues (and for graphs captured from them) until the stream is released: growing allocates
// a new buffer and retires the old one, it neither frees nor waits.  Returns null (reason
// recorded) when it would have to allocate while the stream is being captured.
// Slot WS_NESTED belongs to launchers that other launchers call with operands in slot WS_MAIN
// (the top-k select inside the block selections).
constexpr int WS_MAIN = 0, WS_NESTED = 1, WS_SLOTS = 2;
void *workspace(hipStream_t s, size_t bytes, int slot = WS_MAIN);
uint32_t *ticket_counters(hipStream_t s);   // 64 dwords per stream, zero between kernels; null under capture if not there yet

// Phase timer: brackets the launches made while it is alive with two events on
// `s` when profiling is enabled; does nothing (and records nothing) otherwise.
struct ProfScope {
    ProfScope(int which, hipStream_t s);
    ~ProfScope();
    int which;
    hipStream_t stream;
    void *slot;
};

// Phase timer of exactly one kernel: when profiling is enabled the launch goes through
// hipExtLaunchKernelGGL with a start and a stop event that the runtime binds to the dispatch
// itself, so their difference is the kernel's own duration (what a kernel trace reports), not
// the dispatch latency that an event pair recorded around the launch includes.  Otherwise an
// ordinary launch, no events.
struct ProfKernel {
    ProfKernel(int which, hipStream_t s);
    ~ProfKernel();
    template <typename... KArgs, typename... Args>
    void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t smem, Args... args) {
        if (a) {
            hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)smem, stream, a, b, 0u, static_cast<KArgs>(args)...);
            bound = true;
        } else {
            kernel<<<grid, block, smem, stream>>>(static_cast<KArgs>(args)...);
        }
    }
    int which;
    hipStream_t stream;
    hipEvent_t a = nullptr, b = nullptr;
    bool bound = false;
};

// ---- kernel launchers (one per .hip file) ----------------------------------
int launch_gqa_decode(const uint16_t *k, const uint16_t *v, int64_t n_keys, int n_kv_heads,
                      int head_dim, const uint16_t *q, int n_heads, float scale, float *out,
                      hipStream_t s, const int32_t *sel = nullptr, int64_t n_rows = 0);
int launch_gqa_prefill(const uint16_t *k, const uint16_t *v, int64_t pos0, int64_t n,
                       int n_kv_heads, int head_dim, const uint16_t *q, int n_heads,
                       float scale, float *out, hipStream_t s);
int launch_mla_decode(const uint8_t *rows, const float *scales, int64_t row_bstride,
                      int64_t scale_bstride, int64_t n_rows, int batch, const int32_t *sel, int64_t n_list,
                      const uint16_t *q, int n_heads, float scale, const float *sink, float *out,
                      hipStream_t s, bool fixed_scratch = false);
int launch_mla_prefill(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                       const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s);
int launch_indexer_scores(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys,
                          const uint16_t *q_idx, const float *w, int n_idx_heads, int mode,
                          float *scores, hipStream_t s);
// ---- fused select: approximate scores with an error band, exact scores for the keys inside it
// (indexer_band.hip).  One of these per batch row, in the workspace:
struct IndexerBandRow {
    uint32_t n_cand;      // keys inside the band (may exceed the list's capacity)
    uint32_t fallback;    // the band could not be formed (bound not finite, NaN threshold)
    uint32_t pad[30];     // a row to a 128-byte line: the workgroups of different rows add to n_cand at the same time
};
constexpr int CWICK_INDEXER_BAND_CAP = 4096;   // candidate list entries per row
constexpr int CWICK_INDEXER_APPROX_KEYS = 2048;   // keys per workgroup (= per bound slot) of the approximate kernel
inline int indexer_approx_slots(int64_t n_keys) {
    return (int)((n_keys + CWICK_INDEXER_APPROX_KEYS - 1) / CWICK_INDEXER_APPROX_KEYS);
}
int launch_indexer_approx(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys, const uint16_t *q_idx,
                          const float *w, int n_idx_heads, float *scores, float *beta_slots,
                          IndexerBandRow *rows, uint32_t *digit0_slices, size_t digit0_row_dwords,
                          hipStream_t s);
__host__ __device__ inline bool indexer_band_failed(const IndexerBandRow &r, int cap) {
    return r.fallback != 0u || r.n_cand > (uint32_t)cap;
}
// shapes the banded path takes: rows that the many-workgroup top-k handles, k < n
inline bool indexer_band_applies(int64_t n_keys, int64_t k, int n_idx_heads) {
    return n_keys >= 16384 && n_keys <= 131072 && k < n_keys && n_idx_heads >= 1 && n_idx_heads <= 64;
}
// indexer and top-k in one: `scores` is scratch (its contents afterwards are not scores), the
// selected indices of every row go to out_idx[batch][k] in ascending order
int launch_indexer_banded(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys, const uint16_t *q_idx,
                          const float *w, int n_idx_heads, int64_t k, float *scores, int32_t *out_idx,
                          hipStream_t s);
// top-k machinery on approximate scores: finds T, then patches the scores (+inf / -inf / kept)
// and lists the keys within 2 beta of T.  `ws` holds topk_mw_workspace_bytes() at its start.
// With `digit0_done` the first-digit counts are already there: the approximate kernel left one
// 256-bin slice per workgroup (indexer_approx_slots(n) of them) at the start of each row's
// workspace, rows topk_mw_band_row_dwords(n) dwords apart.
size_t topk_mw_workspace_bytes(int batch, int64_t n);
size_t topk_mw_band_row_dwords(int64_t n);
int launch_topk_band_classify(float *scores, int batch, int64_t n, int64_t k, uint32_t *ws,
                              const float *beta_slots, int n_beta, int32_t *cand, int cap,
                              IndexerBandRow *rows, uint32_t *hi_count, bool digit0_done, hipStream_t s);
// The end of the banded select, after the candidates have their exact scores: ranks the
// candidates, writes the selected indices of every row that fitted the band, and runs the
// plain select for the rows that did not (their scores are the exact kernel's by then).
// `scores` is only read.
// hi_count: [batch][64] dwords, filled by launch_topk_band_classify.
// cand_score: [batch][cap], the exact score of every list entry (what the rescoring wrote).
int launch_topk_band_finish(float *scores, int batch, int64_t n, int64_t k, const int32_t *cand,
                            const float *cand_score, int cap, const IndexerBandRow *rows, uint32_t *hi_count,
                            int32_t *out_idx, hipStream_t s);
int launch_topk(const float *scores, int batch, int64_t n, int64_t k, int32_t *out_idx,
                hipStream_t s);
int launch_quant_latent(const float *rows, int64_t n, uint8_t *out_rows, float *out_scales,
                        hipStream_t s);
int launch_quant_ikeys(const float *rows, int64_t n, uint8_t *out_rows, float *out_scales,
                       hipStream_t s);
int launch_narrow_bf16(const float *src, int64_t n, uint16_t *dst, hipStream_t s);
int launch_mla_absorb(const uint16_t *kvb_w, const float *q, int64_t q_stride, int batch, int n_heads,
                      int q_dim, int nope, int rope, int kv_dim, int kv_lora, uint16_t *q_abs, hipStream_t s);
int launch_mla_expand(const uint16_t *kvb_w, const float *c_acc, int batch, int n_heads, int nope, int vdim,
                      int kv_dim, int kv_lora, float *out, hipStream_t s);
int launch_gqa_prepare(const float *q_proj, int64_t q_head_stride, const float *k_proj, const float *v_proj,
                       int64_t n, int64_t pos0, int n_heads, int n_kv_heads, int head_dim, const float *q_norm,
                       const float *k_norm, float eps, const float *rope_cos, const float *rope_sin, int rotary_dim,
                       uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache, hipStream_t s);
int launch_mla_prefill_wide(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n, const uint16_t *q,
                            int n_heads, float scale, float *out, hipStream_t s);
int launch_ikeys_pool(const float *tail_k, const float *tail_g, const uint16_t *ape, const float *knw, const float *knb,
                      float eps, int kpool, int64_t n_pools, uint8_t *out_rows, float *out_scales, float *out_f32,
                      hipStream_t s);
int launch_candidate_select(const float *scores, int batch, int64_t n, int block, int64_t topk_blocks, uint8_t *cand,
                            hipStream_t s);
int launch_mm_select(const uint16_t *idx_keys, const float *iq, int batch, int64_t limit0, int index_heads,
                     int index_dim, int block, int keep_blocks, float *scores, int64_t score_stride,
                     int32_t *blk_out, int32_t *sel, int64_t max_sel, int32_t *n_sel, hipStream_t s);
int launch_candidate_apply(float *scores, const uint8_t *cand, int batch, int64_t n, hipStream_t s);
int launch_glm_select(const float *scores, int batch, int64_t n_comp, int64_t npos, int kpool, int64_t topk,
                      int strict, int32_t *sel, int64_t max_sel, int32_t *n_sel, hipStream_t s);
int launch_dequant_latent(const uint8_t *rows, const float *scales, int64_t n, float *out, hipStream_t s);
int launch_dequant_ikeys(const uint8_t *rows, const float *scales, int64_t n, float *out, hipStream_t s);
int launch_widen_bf16(const uint16_t *src, int64_t n, float *dst, hipStream_t s);
int launch_e4m3_table(float *out256_dev, hipStream_t s);
int launch_lane_ops(const uint32_t *in64_dev, uint32_t *out832_dev, hipStream_t s);
int run_probe_hbm_read(size_t bytes, int reps, double *gbps);
int run_probe_mfma(int kind, int reps, double *tflops);

// ---- device helpers ---------------------------------------------------------
// order-preserving 32-bit key of a score for the radix select: larger score, larger key; NaN
// sorts below everything (key 0), -0.0 equals +0.0, and no number maps to 0
__device__ __forceinline__ uint32_t topk_key(float f) {
    if (f != f) return 0u;
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u << 1) == 0u) u = 0u;                       // -0.0 -> +0.0
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return u == 0u ? 1u : u;
}
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}
// low / high half of a dword holding two bf16
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) {
    return __builtin_bit_cast(float, w << 16);
}
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) {
    return __builtin_bit_cast(float, w & 0xFFFF0000u);
}
// round-to-nearest-even fp32 -> bf16 (finite inputs)
__device__ __forceinline__ uint32_t f32_to_bf16_rne(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}
// two fp32 -> one dword of two bf16 / two fp16, round to nearest even
// (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32)
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float v2f;
    typedef __attribute__((ext_vector_type(2))) __bf16 v2b;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f){lo, hi}, v2b));
}
__device__ __forceinline__ uint32_t pack_f16_rne(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float v2f;
    typedef __attribute__((ext_vector_type(2))) _Float16 v2h;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f){lo, hi}, v2h));
}
// acc + both halves of a dword of two bf16 / two fp16, in fp32 (one dot-product instruction)
__device__ __forceinline__ float pair_sum_bf16(uint32_t w, float acc) {
    typedef __attribute__((ext_vector_type(2))) __bf16 v2b;
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2b, w), __builtin_bit_cast(v2b, 0x3F803F80u), acc, false);
}
__device__ __forceinline__ float pair_sum_f16(uint32_t w, float acc) {
    typedef __attribute__((ext_vector_type(2))) _Float16 v2h;
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2h, w), __builtin_bit_cast(v2h, 0x3C003C00u), acc, false);
}
// Two E4M3 bytes -> one dword of two fp16 (exact: E4M3 fits fp16's normal range)
template <bool HI>
__device__ __forceinline__ uint32_t e4m3x2_to_f16x2(uint32_t w) {
    typedef __attribute__((ext_vector_type(2))) _Float16 v2h;
    v2h r = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w, 1.0f, HI);
    return __builtin_bit_cast(uint32_t, r);
}
// Two E4M3 bytes (low or high 16 bits of w) -> two fp32, hardware conversion
// (OCP E4M3fn on gfx950).
template <bool HI>
__device__ __forceinline__ f32x2 e4m3x2_to_f32(uint32_t w) {
    return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, HI);
}
// Two E4M3 bytes -> one dword of two bf16.  Every E4M3 value is exactly
// representable in bf16, so the conversion is exact.
template <bool HI>
__device__ __forceinline__ uint32_t e4m3x2_to_bf16x2(uint32_t w) {
    bf16x2 r = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, HI);
    return __builtin_bit_cast(uint32_t, r);
}

// what place N of this lane's row of sixteen lanes holds (DPP row broadcast)
template <int N>
__device__ __forceinline__ uint32_t row_place(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x150 + N, 0xF, 0xF, true);
}
// Lane l meets lane l ^ 16 (l ^ 32) without a trip through LDS: the rows of sixteen lanes (the
// halves of the wave) trade places between two copies of the value, and a commutative
// operation on the two copies is what a butterfly step would give, bit for bit.
__device__ __forceinline__ void lanes_swap16(uint32_t &a, uint32_t &b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void lanes_swap32(uint32_t &a, uint32_t &b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float xor16_max(float v) {
    uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
    lanes_swap16(a, b);
    return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ __forceinline__ float xor32_max(float v) {
    uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
    lanes_swap32(a, b);
    return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ __forceinline__ float xor16_sum(float v) {
    uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
    lanes_swap16(a, b);
    return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}
__device__ __forceinline__ float xor32_sum(float v) {
    uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
    lanes_swap32(a, b);
    return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}
// Reductions and scans over the wave without LDS.  Within a row of sixteen lanes through DPP:
// swap in pairs, swap pairs, mirror the half row, mirror the row (every step joins two groups
// of lanes that already agree, so all lanes end with the result); across rows the two swaps
// above.  A scan shifts within the row by 1, 2, 4, 8 and then hands the last lane of a row to
// the rows behind it.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xF, false);   // lanes without a source read 0
}
#define CWICK_WAVE_ALLREDUCE(v, OP)                                                         \
    do {                                                                                    \
        { const uint32_t o_ = dpp_u32<0xB1, 0xF>(v); v = OP(v, o_); }   /* quad_perm [1,0,3,2] */ \
        { const uint32_t o_ = dpp_u32<0x4E, 0xF>(v); v = OP(v, o_); }   /* quad_perm [2,3,0,1] */ \
        { const uint32_t o_ = dpp_u32<0x141, 0xF>(v); v = OP(v, o_); }  /* row_half_mirror */      \
        { const uint32_t o_ = dpp_u32<0x140, 0xF>(v); v = OP(v, o_); }  /* row_mirror */           \
        { uint32_t a_ = v, b_ = v; lanes_swap16(a_, b_); v = OP(a_, b_); }                  \
        { uint32_t a_ = v, b_ = v; lanes_swap32(a_, b_); v = OP(a_, b_); }                  \
    } while (0)
#define CWICK_OP_ADD(a, b) ((a) + (b))
#define CWICK_OP_MAX(a, b) ((a) > (b) ? (a) : (b))
#define CWICK_OP_MIN(a, b) ((a) < (b) ? (a) : (b))
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) { CWICK_WAVE_ALLREDUCE(v, CWICK_OP_ADD); return v; }
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) { CWICK_WAVE_ALLREDUCE(v, CWICK_OP_MAX); return v; }
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) { CWICK_WAVE_ALLREDUCE(v, CWICK_OP_MIN); return v; }
// inclusive prefix sum over the lanes of the wave
__device__ __forceinline__ uint32_t wave_scan_u32(uint32_t v) {
    v += dpp_u32<0x111, 0xF>(v);     // row_shr:1
    v += dpp_u32<0x112, 0xF>(v);     // row_shr:2
    v += dpp_u32<0x114, 0xF>(v);     // row_shr:4
    v += dpp_u32<0x118, 0xF>(v);     // row_shr:8
    v += dpp_u32<0x142, 0xA>(v);     // row_bcast:15 into rows 1 and 3
    v += dpp_u32<0x143, 0xC>(v);     // row_bcast:31 into rows 2 and 3
    return v;
}
// one step of a sum over aligned groups of lanes, every lane of the group ending with the total
// (a group of `width` lanes whose halves already hold their own totals): DPP inside a row of
// sixteen, the swaps across rows
template <int WIDTH>
__device__ __forceinline__ float group_step_sum(float v) {
    static_assert(WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 || WIDTH == 32 || WIDTH == 64, "group width");
    if (WIDTH == 32) return xor16_sum(v);
    if (WIDTH == 64) return xor32_sum(v);
    constexpr int CTRL = WIDTH == 2 ? 0xB1 : WIDTH == 4 ? 0x4E : WIDTH == 8 ? 0x141 : 0x140;
    return v + __builtin_bit_cast(float, dpp_u32<CTRL, 0xF>(__builtin_bit_cast(uint32_t, v)));
}
// the maximum over the wave in every lane
__device__ __forceinline__ float wave_max(float v) {
#define CWICK_DPP_MAX(ctrl)                                                                                   \
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, false)))
    CWICK_DPP_MAX(0xB1);     // quad_perm [1, 0, 3, 2]
    CWICK_DPP_MAX(0x4E);     // quad_perm [2, 3, 0, 1]
    CWICK_DPP_MAX(0x141);    // row_half_mirror
    CWICK_DPP_MAX(0x140);    // row_mirror
#undef CWICK_DPP_MAX
    return xor32_max(xor16_max(v));
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Round-to-nearest-even fp32 -> E4M3fn (the caller has clamped to +-448): the
// bit recipe of src/ds_quant.c:102-128, except that a round-up out of the last
// subnormal carries into the first normal (byte 0x08) instead of being masked
// away (`mm & 7u`, :127), so that the result is the nearest grid point as the
// reference's own round-trip check demands (tools/ds_verify.c:48-63).
__device__ __forceinline__ uint32_t f32_to_e4m3_rne(float v) {
    if (v == 0.0f) return 0u;
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    uint32_t sign = u >> 31;
    int32_t exp = (int32_t)((u >> 23) & 0xFFu) - 127;
    uint32_t m24 = (1u << 23) | (u & 0x7FFFFFu);
    if (exp >= -6) {
        uint32_t keep = m24 >> 20;
        uint32_t rem = m24 & 0xFFFFFu;
        if (rem > 0x80000u || (rem == 0x80000u && (keep & 1u))) keep++;
        int32_t e = exp;
        if (keep == 16u) { keep >>= 1; e++; }
        if (e > 8) { keep = 14u; e = 8; }
        return (sign << 7) | ((uint32_t)(e + 7) << 3) | (keep & 7u);
    }
    if (exp < -10) return sign << 7;
    int32_t sh = 14 - exp;
    uint32_t mm = m24 >> sh;
    uint32_t rem = m24 & ((1u << sh) - 1u);
    uint32_t half = 1u << (sh - 1);
    if (rem > half || (rem == half && (mm & 1u))) mm++;
    return (sign << 7) | mm;
}

}  // namespace cwick
