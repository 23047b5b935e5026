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

// ---------------------------------------------------------------------------
// indexer key production, candidate blocks, dequantised read-back
// ---------------------------------------------------------------------------
namespace cwick {
namespace {

// One wave per closed pool (src/attention.c:486-525): layer-norm statistics of each of the kp
// raw key rows, a softmax over the pool slots of gate + position bias per dimension, the affine
// k_norm on the normalised rows, the weighted mean as the pool's key; then the row is quantised
// like every indexer key (one fp32 scale per row, amax / 448).  hd = 128: two dims per lane.
__global__ void __launch_bounds__(256)
ikeys_pool_kernel(const float *__restrict__ tail_k, const float *__restrict__ tail_g, const uint16_t *__restrict__ ape,
                  const float *__restrict__ knw, const float *__restrict__ knb, float eps, int kp, int64_t n_pools,
                  uint8_t *__restrict__ out_rows, float *__restrict__ out_scales, float *__restrict__ out_f32) {
    constexpr int HD = CWICK_HIP_INDEX_DIM;
    const int lane = threadIdx.x & 63;
    const int64_t pool = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pool >= n_pools) return;
    const float *k = tail_k + (size_t)pool * kp * HD, *gt = tail_g + (size_t)pool * kp * HD;
    // statistics in double like the reference's (sums of 128 floats are exact there in all but
    // contrived rows, so the order of the wave reduction does not show)
    float mean[8], inv[8], kv[8][2];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        mean[i] = inv[i] = kv[i][0] = kv[i][1] = 0.0f;
        if (i < kp) {
            kv[i][0] = k[i * HD + lane];
            kv[i][1] = k[i * HD + 64 + lane];
            mean[i] = (float)(wave_sum((double)kv[i][0] + (double)kv[i][1]) / (double)HD);
            const double t0 = (double)kv[i][0] - (double)mean[i], t1 = (double)kv[i][1] - (double)mean[i];
            inv[i] = 1.0f / sqrtf((float)(wave_sum(t0 * t0 + t1 * t1) / (double)HD) + eps);
        }
    }
    float res[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int d = lane + 64 * h;
        float lg[8], mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            lg[i] = -INFINITY;
            if (i < kp) {
                lg[i] = gt[i * HD + d] + bf16_to_f32(ape[i * HD + d]);
                mx = lg[i] > mx ? lg[i] : mx;
            }
        }
        float den = 0.0f, acc = 0.0f;
        const float w = knw[d], bb = knb[d];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i < kp) {
                const float p = expf(lg[i] - mx);
                den += p;
                const float nv = ((kv[i][h] - mean[i]) * inv[i]) * w + bb;
                acc += p * nv;
            }
        }
        res[h] = den > 0.0f ? acc / den : 0.0f;
    }
    if (out_f32) {
        out_f32[(size_t)pool * HD + lane] = res[0];
        out_f32[(size_t)pool * HD + 64 + lane] = res[1];
    }
    const float amax = wave_max(fmaxf(fabsf(res[0]), fabsf(res[1])));
    const float s = amax > 0.0f ? amax / 448.0f : 1.0f;
    if (lane == 0) out_scales[pool] = s;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        float v = res[h] / s;
        v = fminf(fmaxf(v, -448.0f), 448.0f);
        out_rows[(size_t)pool * HD + lane + 64 * h] = (uint8_t)f32_to_e4m3_rne(v);
    }
}

// block maxima of the scores, the partly filled last block forced in (src/ds_model.c:1127-1135)
__global__ void __launch_bounds__(256)
cand_blockmax_kernel(const float *__restrict__ scores, int64_t n, int bs, int64_t nblk, float *__restrict__ bsc) {
    const int lane = threadIdx.x & 63;
    const int64_t b = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row = blockIdx.y;
    if (b >= nblk) return;
    const float *s = scores + (size_t)row * n;
    const int64_t lo = b * bs, hi = lo + bs < n ? lo + bs : n;
    float mx = -INFINITY;
    for (int64_t t = lo + lane; t < hi; t += 64) mx = s[t] > mx ? s[t] : mx;
    mx = wave_max(mx);
    if (lane == 0) bsc[(size_t)row * nblk + b] = b == nblk - 1 ? INFINITY : mx;
}

__global__ void __launch_bounds__(256)
cand_mark_kernel(const int32_t *__restrict__ blk, int64_t k, int64_t n, int bs, uint8_t *__restrict__ cand) {
    const int row = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x;                 // one workgroup per chosen block
    if (i >= k) return;
    const int32_t b = blk[(size_t)row * k + i];
    if (b < 0) return;
    const int64_t lo = (int64_t)b * bs, hi = lo + bs < n ? lo + bs : n;
    for (int64_t t = lo + threadIdx.x; t < hi; t += 256) cand[(size_t)row * n + t] = 1;
}

__global__ void __launch_bounds__(256) cand_clear_kernel(uint8_t *__restrict__ cand, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < total; i += stride) cand[i] = 0;
}

// positions outside the candidate blocks cannot be selected (src/ds_model.c:1144-1147)
__global__ void __launch_bounds__(256)
cand_apply_kernel(float *__restrict__ scores, const uint8_t *__restrict__ cand, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < total; i += stride)
        if (!cand[i]) scores[i] = -INFINITY;
}

template <int DIM, int BLOCK>
__global__ void __launch_bounds__(256)
dequant_rows_kernel(const uint8_t *__restrict__ rows, const float *__restrict__ scales, int64_t n, float *__restrict__ out) {
    constexpr int NBLK = (DIM + BLOCK - 1) / BLOCK;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * 256, total = n * DIM;
    for (; i < total; i += stride) {
        const int64_t r = i / DIM;
        const int d = (int)(i % DIM);
        out[i] = e4m3x2_to_f32<false>((uint32_t)rows[i])[0] * scales[r * NBLK + d / BLOCK];
    }
}

}  // namespace

int launch_ikeys_pool(const float *tail_k, const float *tail_g, const uint16_t *ape, const float *knw, const float *knb,
                      float eps, int kpool, int64_t n_pools, uint8_t *out_rows, float *out_scales, float *out_f32,
                      hipStream_t s) {
    CWICK_REQUIRE(tail_k && tail_g && ape && knw && knb && out_rows && out_scales, "ikeys_pool: null pointer");
    CWICK_REQUIRE(kpool >= 1 && kpool <= 8, "ikeys_pool: kpool %d (1..8, src/attention.c:492)", kpool);
    CWICK_REQUIRE(n_pools >= 1 && n_pools <= ((int64_t)1 << 30), "ikeys_pool: n_pools %lld", (long long)n_pools);
    ikeys_pool_kernel<<<dim3((unsigned)((n_pools + 3) / 4)), 256, 0, s>>>(tail_k, tail_g, ape, knw, knb, eps, kpool,
                                                                        n_pools, out_rows, out_scales, out_f32);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_candidate_select(const float *scores, int batch, int64_t n, int block, int64_t topk_blocks, uint8_t *cand,
                            hipStream_t s) {
    CWICK_REQUIRE(scores && cand, "candidate_select: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535 && n >= 1 && n <= ((int64_t)1 << 30), "candidate_select: batch %d n %lld",
                  batch, (long long)n);
    CWICK_REQUIRE(block >= 1 && topk_blocks >= 1 && topk_blocks <= 65536, "candidate_select: block %d, blocks kept %lld",
                  block, (long long)topk_blocks);
    const int64_t nblk = (n + block - 1) / block;
    // (the top-k below keeps its own workspace slot, so the block scores can sit in this call's)
    CWICK_REQUIRE(nblk < 16384, "candidate_select: %lld blocks (at most 16383)", (long long)nblk);
    const size_t bsc_b = ((size_t)batch * nblk * 4 + 255) & ~(size_t)255;
    char *ws = (char *)workspace(s, bsc_b + (size_t)batch * topk_blocks * 4);
    if (!ws) return 0;                      // workspace() has recorded why
    float *bsc = (float *)ws;
    int32_t *blk = (int32_t *)(ws + bsc_b);
    cand_blockmax_kernel<<<dim3((unsigned)((nblk + 3) / 4), batch), 256, 0, s>>>(scores, n, block, nblk, bsc);
    CWICK_HIP_CALL(hipGetLastError());
    {
        const int64_t total = (int64_t)batch * n;
        int64_t blocks = (total + 255) / 256;
        if (blocks > 8192) blocks = 8192;
        cand_clear_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(cand, total);      // a kernel, not a memset: safe under graph capture
    }
    if (!launch_topk(bsc, batch, nblk, topk_blocks, blk, s)) return 0;
    cand_mark_kernel<<<dim3((unsigned)topk_blocks, batch), 256, 0, s>>>(blk, topk_blocks, n, block, cand);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

// The rest of indexer_select behind the pool scores (src/attention.c:585-620), one workgroup per
// query.  pools[want] are the chosen pools in ascending order (the top-k select's output);
// the list keeps the reference's order: the pools that score above the lowest chosen score in
// ascending order, then the pools that equal it, each as its kp positions c kp + r; the
// positions behind the last closed pool; then the query's own position unless `strict` or it is
// the last entry already (the reference tests sel[n-1] only, :618).  mode_whole: no more pools
// than wanted -- the list is the whole prefix 0 .. npos-1 and n_sel is -1 (:558-559).
// Entries behind the list are -1, which the attention kernels skip.
constexpr int GLM_THREADS = 256;
__global__ void __launch_bounds__(GLM_THREADS)
glm_expand_kernel(const float *__restrict__ scores, const int32_t *__restrict__ pools, int64_t want, int64_t n_comp,
                  int64_t npos, int kp, int strict, int mode_whole, int32_t *__restrict__ sel, int64_t max_sel,
                  int32_t *__restrict__ n_sel) {
    __shared__ uint32_t red[GLM_THREADS / 64];
    __shared__ uint32_t wave_gt[GLM_THREADS / 64], wave_eq[GLM_THREADS / 64];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int32_t *out = sel + (size_t)row * max_sel;
    if (mode_whole) {
        for (int64_t i = tid; i < max_sel; i += GLM_THREADS) out[i] = i < npos ? (int32_t)i : -1;
        if (tid == 0 && n_sel) n_sel[row] = -1;
        return;
    }
    const float *sc = scores + (size_t)row * n_comp;
    const int32_t *pl = pools + (size_t)row * want;
    // the lowest chosen score, as the select's own order key (so that -0.0 == +0.0)
    uint32_t kmin = 0xFFFFFFFFu;
    for (int64_t i = tid; i < want; i += GLM_THREADS) {
        const int32_t c = pl[i];
        if (c >= 0) {
            const uint32_t k = topk_key(sc[c]);
            kmin = k < kmin ? k : kmin;
        }
    }
    kmin = wave_min_u32(kmin);
    if (lane == 0) red[wave] = kmin;
    __syncthreads();
    kmin = red[0];
#pragma unroll
    for (int w = 1; w < GLM_THREADS / 64; w++) kmin = red[w] < kmin ? red[w] : kmin;
    // how many chosen pools score above it (they come first), and the last pool at it (the list's
    // last pool entry)
    uint32_t n_gt = 0, eq_last = 0;                 // eq_last: pool index + 1
    for (int64_t i = tid; i < want; i += GLM_THREADS) {
        const int32_t c = pl[i];
        if (c < 0) continue;
        if (topk_key(sc[c]) > kmin) n_gt++;
        else eq_last = (uint32_t)c + 1u > eq_last ? (uint32_t)c + 1u : eq_last;
    }
    n_gt = wave_sum_u32(n_gt);
    eq_last = wave_max_u32(eq_last);
    __syncthreads();
    if (lane == 0) red[wave] = n_gt, wave_eq[wave] = eq_last;
    __syncthreads();
    n_gt = 0, eq_last = 0;
#pragma unroll
    for (int w = 0; w < GLM_THREADS / 64; w++) {
        n_gt += red[w];
        eq_last = wave_eq[w] > eq_last ? wave_eq[w] : eq_last;
    }
    // places: a running count of both kinds over chunks of the pool list
    uint32_t base_gt = 0, base_eq = 0;
    for (int64_t i0 = 0; i0 < want; i0 += GLM_THREADS) {
        const int64_t i = i0 + tid;
        const int32_t c = i < want ? pl[i] : -1;
        const bool gt = c >= 0 && topk_key(sc[c]) > kmin, eq = c >= 0 && !gt;
        const uint32_t sg = wave_scan_u32(gt ? 1u : 0u), se = wave_scan_u32(eq ? 1u : 0u);
        __syncthreads();
        if (lane == 63) wave_gt[wave] = sg, wave_eq[wave] = se;
        __syncthreads();
        uint32_t og = base_gt, oe = base_eq, tg = 0, te = 0;
#pragma unroll
        for (int w = 0; w < GLM_THREADS / 64; w++) {
            if (w < wave) og += wave_gt[w], oe += wave_eq[w];
            tg += wave_gt[w], te += wave_eq[w];
        }
        if (c >= 0) {
            const uint32_t place = gt ? og + sg - 1u : n_gt + oe + se - 1u;
            for (int r = 0; r < kp; r++) out[(size_t)place * kp + r] = c * kp + r;
        }
        base_gt += tg, base_eq += te;
    }
    __syncthreads();
    // the tail, the query itself, the padding: one thread (a handful of entries) and then all
    const int64_t n_pool = (int64_t)(base_gt + base_eq) * kp;
    const int64_t tail = npos % kp;
    int64_t n = n_pool + tail;
    for (int64_t r = tid; r < tail; r += GLM_THREADS) out[n_pool + r] = (int32_t)(npos - tail + r);
    // the list's last entry before the self rule: the tail's, else the last pool at the lowest score
    const int64_t last = tail > 0 ? npos - 1 : (eq_last ? (int64_t)(eq_last - 1u) * kp + kp - 1 : -1);
    const bool add_self = !strict && last != npos - 1;
    if (tid == 0 && add_self) out[n] = (int32_t)(npos - 1);
    if (add_self) n++;
    for (int64_t i = n + tid; i < max_sel; i += GLM_THREADS) out[i] = -1;
    if (tid == 0 && n_sel) n_sel[row] = (int32_t)n;
}

int launch_glm_select(const float *scores, int batch, int64_t n_comp, int64_t npos, int kpool, int64_t topk,
                      int strict, int32_t *sel, int64_t max_sel, int32_t *n_sel, hipStream_t s) {
    CWICK_REQUIRE(scores && sel, "glm_select: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535 && n_comp >= 1 && n_comp <= ((int64_t)1 << 24),
                  "glm_select: batch %d, %lld pools", batch, (long long)n_comp);
    CWICK_REQUIRE(kpool >= 1 && kpool <= 8, "glm_select: kpool %d (1..8, src/attention.c:492)", kpool);
    CWICK_REQUIRE(topk >= 1 && topk <= 65536, "glm_select: topk %lld", (long long)topk);
    CWICK_REQUIRE(npos >= n_comp * kpool && npos < (n_comp + 1) * kpool,
                  "glm_select: %lld positions do not close exactly %lld pools of %d", (long long)npos,
                  (long long)n_comp, kpool);
    const int64_t want = (topk + kpool - 1) / kpool;
    CWICK_REQUIRE(max_sel >= (want + 1) * kpool && max_sel <= ((int64_t)1 << 24),
                  "glm_select: max_sel %lld (at least (ceil(topk / kpool) + 1) * kpool = %lld)", (long long)max_sel,
                  (long long)((want + 1) * kpool));
    if (n_comp <= want) {
        glm_expand_kernel<<<dim3(batch), GLM_THREADS, 0, s>>>(scores, nullptr, want, n_comp, npos, kpool, strict, 1, sel,
                                                            max_sel, n_sel);
        CWICK_HIP_CALL(hipGetLastError());
        return 1;
    }
    int32_t *pools = (int32_t *)workspace(s, (size_t)batch * want * sizeof(int32_t));
    if (!pools) return 0;                   // workspace() has recorded why
    if (!launch_topk(scores, batch, n_comp, want, pools, s)) return 0;
    glm_expand_kernel<<<dim3(batch), GLM_THREADS, 0, s>>>(scores, pools, want, n_comp, npos, kpool, strict, 0, sel,
                                                        max_sel, n_sel);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_candidate_apply(float *scores, const uint8_t *cand, int batch, int64_t n, hipStream_t s) {
    CWICK_REQUIRE(scores && cand && batch >= 1 && n >= 1, "candidate_apply: bad argument");
    const int64_t total = (int64_t)batch * n;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    cand_apply_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(scores, cand, total);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_dequant_latent(const uint8_t *rows, const float *scales, int64_t n, float *out, hipStream_t s) {
    CWICK_REQUIRE(rows && scales && out && n > 0, "dequant_latent: bad argument");
    int64_t blocks = (n * CWICK_HIP_LATENT_KDIM + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    dequant_rows_kernel<CWICK_HIP_LATENT_KDIM, CWICK_HIP_LATENT_BLOCK><<<dim3((unsigned)blocks), 256, 0, s>>>(rows, scales, n, out);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_dequant_ikeys(const uint8_t *rows, const float *scales, int64_t n, float *out, hipStream_t s) {
    CWICK_REQUIRE(rows && scales && out && n > 0, "dequant_ikeys: bad argument");
    int64_t blocks = (n * CWICK_HIP_INDEX_DIM + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    dequant_rows_kernel<CWICK_HIP_INDEX_DIM, CWICK_HIP_INDEX_DIM><<<dim3((unsigned)blocks), 256, 0, s>>>(rows, scales, n, out);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
