// prep.hip -- the steps on either side of the attention kernels, kept on the device so that the
// queries and the outputs never cross the host link:
//
//   mla_absorb   q_abs[h] = W_k[h]^T q_nope[h]  (+ the rope dims of q passed through), narrowed to
//                the bf16 the MLA kernels take   (src/attention.c:741-744, gemv_bf16_t :145-177)
//   mla_expand   attn_out[h] = W_v[h] c_acc[h]    (src/attention.c:812-815, gemv_bf16_n :184-224)
//   gqa_prepare  per-head RMS norm with (1 + w) weights, partial rotate-half RoPE, Q narrowed to
//                bf16, K and V rows narrowed and appended to the device cache
//                (src/q35_model.c:1627-1652; rms_norm_w :111-121, rope_apply :144-153)
//
// All three are bandwidth-bound passes over small operands (the kv_b_proj slice of a layer is
// 128 heads x 320 rows x 512 bf16 = 42 MB; a decode step of the norm touches 20 heads).  The
// sums are fp32 like the reference's; their order is the wave's tree, not the CPU's serial
// loop, so results agree to rounding, not bit for bit.
#include "common.hpp"

namespace cwick {
namespace {

// one workgroup per (head, query): 256 threads, thread c owns columns 2c and 2c+1 of a 512-wide
// latent; W_k rows are read as one dword per thread (coalesced), q_nope[h][r] is wave-uniform
__global__ void __launch_bounds__(256)
mla_absorb_kernel(const uint16_t *__restrict__ kvb_w, const float *__restrict__ q, int64_t q_stride,
                  int q_dim, int nope, int rope, int kv_dim, int kv_lora, uint16_t *__restrict__ out) {
    const int h = blockIdx.x, nh = gridDim.x, y = blockIdx.y, tid = threadIdx.x;
    __shared__ float qs[512];
    const float *qh = q + (size_t)y * q_stride + (size_t)h * q_dim;
    for (int i = tid; i < nope + rope; i += 256) qs[i] = qh[i];
    __syncthreads();
    const uint16_t *wk = kvb_w + (size_t)h * kv_dim * kv_lora;
    uint16_t *o = out + ((size_t)y * nh + h) * CWICK_HIP_LATENT_KDIM;
    for (int c0 = 2 * tid; c0 < kv_lora; c0 += 512) {
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll 8
        for (int r = 0; r < nope; r++) {
            const uint32_t w = *(const uint32_t *)(wk + (size_t)r * kv_lora + c0);
            const float a = qs[r];
            a0 = __builtin_fmaf(a, bf16lo_to_f32(w), a0);
            a1 = __builtin_fmaf(a, bf16hi_to_f32(w), a1);
        }
        *(uint32_t *)(o + c0) = pack_bf16_rne(a0, a1);
    }
    // the rope dims of the query pass through (zero when the model has none)
    for (int i = tid; i < CWICK_HIP_LATENT_KDIM - kv_lora; i += 256)
        o[kv_lora + i] = (uint16_t)f32_to_bf16_rne(i < rope ? qs[nope + i] : 0.0f);
}

// one workgroup per (head, query): four waves, wave w takes rows w, w + 4, ... of W_v; a lane
// reads eight bf16 of the row (16 bytes) and the matching eight floats of c_acc
__global__ void __launch_bounds__(256)
mla_expand_kernel(const uint16_t *__restrict__ kvb_w, const float *__restrict__ c_acc, int nope, int vdim,
                  int kv_dim, int kv_lora, float *__restrict__ out) {
    const int h = blockIdx.x, nh = gridDim.x, y = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *c = c_acc + ((size_t)y * nh + h) * kv_lora;
    const uint16_t *wv = kvb_w + ((size_t)h * kv_dim + nope) * kv_lora;
    float cv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) cv[i] = 8 * lane + i < kv_lora ? c[8 * lane + i] : 0.0f;
    for (int r = wave; r < vdim; r += 4) {
        float s = 0.0f;
        if (8 * lane < kv_lora) {
            const u32x4 w = *(const u32x4 *)(wv + (size_t)r * kv_lora + 8 * lane);
#pragma unroll
            for (int d = 0; d < 4; d++) {
                s = __builtin_fmaf(bf16lo_to_f32(w[d]), cv[2 * d], s);
                s = __builtin_fmaf(bf16hi_to_f32(w[d]), cv[2 * d + 1], s);
            }
        }
        s = wave_sum(s);
        if (lane == 0) out[((size_t)y * nh + h) * vdim + r] = s;
    }
}

// one wave per (token, head), q heads first, then k heads, then v heads (narrowed only)
__global__ void __launch_bounds__(256)
gqa_prepare_kernel(const float *__restrict__ q_proj, int64_t q_head_stride, const float *__restrict__ k_proj,
                   const float *__restrict__ v_proj, int64_t n, int64_t pos0, int H, int KV, int HD,
                   const float *__restrict__ q_norm, const float *__restrict__ k_norm, float eps,
                   const float *__restrict__ rope_cos, const float *__restrict__ rope_sin, int rotary,
                   uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_cache, uint16_t *__restrict__ v_cache) {
    __shared__ float buf[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_tok = H + 2 * KV;
    const int64_t item = (int64_t)blockIdx.x * 4 + wave;
    if (item >= n * per_tok) return;
    const int64_t t = item / per_tok;
    const int hh = (int)(item % per_tok);
    const int64_t p = pos0 + t;
    const float *src;
    const float *w = nullptr;
    uint16_t *dst;
    bool rot = true;
    if (hh < H) {
        src = q_proj + ((size_t)t * H + hh) * q_head_stride;
        w = q_norm;
        dst = q_out + ((size_t)t * H + hh) * HD;
    } else if (hh < H + KV) {
        src = k_proj + ((size_t)t * KV + (hh - H)) * HD;
        w = k_norm;
        dst = k_cache + ((size_t)p * KV + (hh - H)) * HD;
    } else {
        src = v_proj + ((size_t)t * KV + (hh - H - KV)) * HD;
        dst = v_cache + ((size_t)p * KV + (hh - H - KV)) * HD;
        rot = false;
    }
    float v[4];
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        v[i] = d < HD ? src[d] : 0.0f;
        acc = __builtin_fmaf(v[i], v[i], acc);
    }
    if (rot) {
        acc = wave_sum(acc);
        const float rstd = 1.0f / sqrtf(acc / (float)HD + eps);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < HD) {
                const float x = v[i] * rstd;
                buf[wave][d] = w ? x * (1.0f + w[d]) : x;
            }
        }
        // the partner element of the rotation was written by another lane of this wave: LDS
        // serves a wave's instructions in order, the barrier only pins the compiler's order
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const int pairs = rotary / 2;
        const float *cs = rope_cos + (size_t)p * pairs, *sn = rope_sin + (size_t)p * pairs;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d >= HD) continue;
            float x = buf[wave][d];
            if (d < pairs) {
                const float b = buf[wave][d + pairs];
                x = x * cs[d] - b * sn[d];
            } else if (d < 2 * pairs) {
                const float a = buf[wave][d - pairs];
                x = x * cs[d - pairs] + a * sn[d - pairs];
            }
            v[i] = x;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        if (d < HD) dst[d] = (uint16_t)f32_to_bf16_rne(v[i]);
    }
}

}  // namespace

int launch_mla_absorb(const uint16_t *kvb_w, const float *q, int64_t q_stride, int batch, int n_heads,
                      int q_dim, int nope, int rope, int kv_dim, int kv_lora, uint16_t *q_abs, hipStream_t s) {
    CWICK_REQUIRE(kvb_w && q && q_abs, "mla_absorb: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535 && n_heads >= 1 && n_heads <= 65535, "mla_absorb: batch %d, n_heads %d",
                  batch, n_heads);
    CWICK_REQUIRE(kv_lora == CWICK_HIP_LATENT_VDIM, "mla_absorb: kv_lora %d (the latent cache holds 512)", kv_lora);
    CWICK_REQUIRE(nope >= 1 && rope >= 0 && rope <= CWICK_HIP_LATENT_KDIM - CWICK_HIP_LATENT_VDIM && nope + rope <= q_dim &&
                      nope + rope <= 512 && nope <= kv_dim,
                  "mla_absorb: nope %d rope %d q_dim %d kv_dim %d", nope, rope, q_dim, kv_dim);
    CWICK_REQUIRE((uintptr_t)kvb_w % 4 == 0 && (uintptr_t)q_abs % 4 == 0, "mla_absorb: operands must be 4-byte aligned");
    mla_absorb_kernel<<<dim3(n_heads, batch), 256, 0, s>>>(kvb_w, q, q_stride, q_dim, nope, rope, kv_dim, kv_lora, q_abs);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_mla_expand(const uint16_t *kvb_w, const float *c_acc, int batch, int n_heads, int nope, int vdim,
                      int kv_dim, int kv_lora, float *out, hipStream_t s) {
    CWICK_REQUIRE(kvb_w && c_acc && out, "mla_expand: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535 && n_heads >= 1 && n_heads <= 65535, "mla_expand: batch %d, n_heads %d",
                  batch, n_heads);
    CWICK_REQUIRE(kv_lora == CWICK_HIP_LATENT_VDIM, "mla_expand: kv_lora %d (the latent cache holds 512)", kv_lora);
    CWICK_REQUIRE(vdim >= 1 && nope >= 0 && nope + vdim <= kv_dim, "mla_expand: nope %d vdim %d kv_dim %d", nope, vdim, kv_dim);
    CWICK_REQUIRE((uintptr_t)kvb_w % 16 == 0, "mla_expand: kv_b_proj must be 16-byte aligned");
    mla_expand_kernel<<<dim3(n_heads, batch), 256, 0, s>>>(kvb_w, c_acc, nope, vdim, kv_dim, kv_lora, out);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_gqa_prepare(const float *q_proj, int64_t q_head_stride, const float *k_proj, const float *v_proj,
                       int64_t n, int64_t pos0, int n_heads, int n_kv_heads, int head_dim, const float *q_norm,
                       const float *k_norm, float eps, const float *rope_cos, const float *rope_sin, int rotary_dim,
                       uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache, hipStream_t s) {
    CWICK_REQUIRE(q_proj && k_proj && v_proj && q_out && k_cache && v_cache, "gqa_prepare: null pointer");
    CWICK_REQUIRE(n >= 1 && pos0 >= 0 && n <= ((int64_t)1 << 24), "gqa_prepare: n %lld pos0 %lld", (long long)n, (long long)pos0);
    CWICK_REQUIRE(head_dim >= 2 && head_dim <= 256, "gqa_prepare: head_dim %d (at most 256)", head_dim);
    CWICK_REQUIRE(n_heads >= 1 && n_kv_heads >= 1 && q_head_stride >= head_dim, "gqa_prepare: heads %d/%d, stride %lld",
                  n_heads, n_kv_heads, (long long)q_head_stride);
    CWICK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0, "gqa_prepare: rotary_dim %d", rotary_dim);
    CWICK_REQUIRE(rotary_dim == 0 || (rope_cos && rope_sin), "gqa_prepare: rope tables missing");
    const int64_t items = n * (n_heads + 2 * n_kv_heads);
    gqa_prepare_kernel<<<dim3((unsigned)((items + 3) / 4)), 256, 0, s>>>(
        q_proj, q_head_stride, k_proj, v_proj, n, pos0, n_heads, n_kv_heads, head_dim, q_norm, k_norm, eps, rope_cos,
        rope_sin, rotary_dim, q_out, k_cache, v_cache);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
