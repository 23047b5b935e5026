// mla_dsplit.hip -- absorbed-latent MLA with the contraction split over the waves
// (decode, sparse decode and chunked prefill of src/attention.c:749-811 /
// :1010-1019 over the FP8 latent).  This is the kernel the entry points use;
// mla_stream.hip and mla.hip are earlier schedules kept selectable
// (CWICK_HIP_MLA=stream|v1) as comparison arms.
//
//   workgroup = 4 waves, 32 query rows (heads of one query) x one key slice,
//   tiles of 32 keys.  Wave w owns latent dims 128w..128w+127 -- one scale
//   block -- for BOTH products:
//     scores   S^T[key][head] = sum over dims: the wave computes the partial dot
//              over its 128 dims (waves 0 and 1 also take 32 rope dims each),
//              multiplies by its block's fp32 scale, and the four partials are
//              summed through LDS (the only exchange, one barrier per tile);
//     values   O^T[dim][head]: the wave produces exactly its 128 output dims, with
//              weights p * scale[key][w].
//   So a wave touches only its own slice of every latent row: it fetches that
//   slice itself (global -> LDS by global_load_lds_dwordx4, no registers, one
//   tile ahead), converts it once for each product, keeps 40 registers of Q and
//   64 of output, and needs no merge at the end.  Two workgroups fit a CU, which
//   is what hides the LDS and barrier latency.
//
//   LDS tile layout [16-dim group][key position 0..31][16 B]: the K fragment
//   (A operand of S^T = K Q^T, v_mfma_f32_32x32x16_bf16) is a 16-byte read per
//   lane, 1 KiB contiguous per wave; the V^T fragment (A operand of
//   O^T = V^T P^T, v_mfma_f32_32x32x16_f16) comes from ds_read_b64_tr_b8, 128 B
//   contiguous per 16-lane group.  P^T is the score tile itself: one head per
//   lane column, contraction slots numbered to match the accumulator layout.
#include "common.hpp"
#include "merge.hpp"

#include <cstdlib>
#include <cstring>

namespace cwick {

int launch_mla_decode_v1(const uint8_t *rows, const float *scales, int64_t row_bstride,
                         int64_t scale_bstride, int64_t n_rows, int batch, const int32_t *sel,
                         int64_t n_list, const uint16_t *q, int n_heads, float scale, float *out,
                         hipStream_t s);
int launch_mla_prefill_v1(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                          const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s);
int launch_mla_decode_v2(const uint8_t *rows, const float *scales, int64_t row_bstride,
                         int64_t scale_bstride, int64_t n_rows, int batch, const int32_t *sel,
                         int64_t n_list, const uint16_t *q, int n_heads, float scale, float *out,
                         hipStream_t s);
int launch_mla_prefill_v2(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                          const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s);

namespace {

constexpr int KDIM = CWICK_HIP_LATENT_KDIM;   // 576
constexpr int VDIM = CWICK_HIP_LATENT_VDIM;   // 512
constexpr int NBLK = CWICK_HIP_LATENT_NBLK;   // 5
constexpr int THREADS = 256;
constexpr int TK = 32;                        // keys per tile
constexpr int ROWS = 32;                      // query rows per workgroup
constexpr float LAZY = 4.0f;                  // log2 slack of the running maximum
constexpr int WEXP = 10;                      // weights carry 2^(WEXP - e_run) <= 2^(LAZY + WEXP)
constexpr int E_NONE = -1000;

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

struct Params {
    const uint8_t *rows;
    const float *scales;
    int64_t row_bstride, scale_bstride, n_rows;
    const int32_t *sel;
    int64_t n_list, list_step;
    const uint16_t *q;
    int nh, nq;
    float scale;
    int n_splits;
    int64_t keys_per_split;   // multiple of TK
    float *out, *part_acc, *part_ml;
};

// what one wave keeps of one tile
struct WaveTile {
    uint8_t own[8][TK][16];       // its 8 sixteen-dim groups (128 dims)            4096 B
    uint8_t rope[2][TK][16];      // one rope pair (waves 0 and 1)                  1024 B
    float sc[2][TK];              // [0] scale of its block, [1] scale of the rope   256 B
};
struct Smem {
    WaveTile tile[2][4];          // [stage][wave]                                  43008 B
    float sx[2][4][4][64][4];     // [stage][wave][q4][lane][4]: partial scores     32768 B
};

__device__ __forceinline__ float pow2i(int e) {
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
    return __builtin_bit_cast(float, (uint32_t)(e + 127) << 23);
}

__global__ void __launch_bounds__(THREADS, 2) mla_dsplit_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    Smem &sm = *reinterpret_cast<Smem *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;    // = scale block = dim slice
    const int m = lane & 31;      // key position (scores) / head column / dim row
    const int g = lane >> 5;      // which half of the contraction slots
    const bool has_rope = wave < 2;

    // ---- work unit: consecutive units (the head blocks of one key slice) share an XCD ----
    const int n_hb = (p.nh + ROWS - 1) / ROWS;
    const int64_t total = (int64_t)gridDim.x;
    int64_t unit = blockIdx.x;
    if (total % 8 == 0) unit = (unit % 8) * (total / 8) + unit / 8;
    const int hb = (int)(unit % n_hb);
    const int split = (int)((unit / n_hb) % p.n_splits);
    const int y = (int)(unit / ((int64_t)n_hb * p.n_splits));

    const uint8_t *rows = p.rows + (size_t)y * p.row_bstride;
    const float *scales = p.scales + (size_t)y * p.scale_bstride;
    const int32_t *sel = p.sel ? p.sel + (size_t)y * p.n_list : nullptr;
    const int64_t limit = p.n_list + (int64_t)y * p.list_step;
    const int64_t k_begin = (int64_t)split * p.keys_per_split;
    int64_t k_end = k_begin + p.keys_per_split;
    if (k_end > limit) k_end = limit;
    const int n_tiles = k_end > k_begin ? (int)((k_end - k_begin + TK - 1) / TK) : 0;

    auto row_of = [&](int t) -> int {
        const int64_t i = k_begin + (int64_t)t * TK + m;
        int64_t r = -1;
        if (t < n_tiles && i < k_end) {
            r = sel ? (int64_t)sel[i] : i;
            if (r < 0 || r >= p.n_rows) r = -1;
        }
        return (int)r;
    };
    // 6 DMA instructions: lanes (m, g) fetch 16 B of row(m): own dim groups 2n+g
    // (n = 0..3), the wave's rope pair, and one fp32 scale (g = 0: own block,
    // g = 1: rope block).  Waves 2 and 3 have no rope share; their fifth
    // instruction re-reads an own group into the spare slot so that every wave
    // issues the same count.
    auto issue = [&](int r, WaveTile *b) {
        const int64_t rc = r >= 0 ? r : 0;            // masked positions fetch row 0, weight 0
        const uint8_t *gsrc = rows + rc * KDIM + 128 * wave + 16 * g;
#pragma unroll
        for (int n = 0; n < 4; n++)
            __builtin_amdgcn_global_load_lds((glb_void *)(gsrc + 32 * n), (lds_void *)&b->own[2 * n][0][0], 16, 0, 0);
        const uint8_t *rsrc = has_rope ? rows + rc * KDIM + 512 + 32 * wave + 16 * g : gsrc;
        __builtin_amdgcn_global_load_lds((glb_void *)rsrc, (lds_void *)&b->rope[0][0][0], 16, 0, 0);
        const float *ssrc = scales + rc * NBLK + (g ? 4 : wave);
        __builtin_amdgcn_global_load_lds((glb_void *)ssrc, (lds_void *)&b->sc[0][0], 4, 0, 0);
    };

    int row_cur = row_of(0);
    int row_nxt = row_of(1);
    if (n_tiles > 0) issue(row_cur, &sm.tile[0][wave]);

    // ---- this wave's Q fragments (B operand): pair j of its block = dims
    // 128w + 32j + 16g + [0,8) and + [8,16); rope pair = dims 512 + 32w + ...
    bf16x8 qf[10];
    {
        int head = hb * ROWS + m;
        if (head >= p.nh) head = p.nh - 1;
        const uint16_t *qrow = p.q + ((size_t)y * p.nh + head) * KDIM + 16 * g;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            qf[2 * j] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + 128 * wave + 32 * j));
            qf[2 * j + 1] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + 128 * wave + 32 * j + 8));
        }
        const int ro = has_rope ? 512 + 32 * wave : 0;
        qf[8] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + ro));
        qf[9] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + ro + 8));
    }

    f32x16 oacc[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = 0.0f;
    float m_ref = -INFINITY, l_part = 0.0f;
    int e_run = E_NONE;
    const float c0 = p.scale * 1.44269504088896340736f;   // scores live in log2 units

    // transpose-read addressing (constant per lane): 16-lane group G, lane gi in it
    const int G = lane >> 4, gi = lane & 15;
    const int tr_k = gi >> 1;
    const int tr_pos = 4 * (G >> 1) + (tr_k & 3) + 8 * (tr_k >> 2);   // + 16 s
    const int tr_dgo = G & 1;                                         // + 2 db
    const int tr_byte = 8 * (gi & 1);

    for (int t = 0; t < n_tiles; t++) {
        const int stage = t & 1;
        const uint32_t valid = (uint32_t)__ballot(row_cur >= 0);      // lanes 0..31 <-> positions
        const bool my_valid = row_cur >= 0;
        WaveTile &B = sm.tile[stage][wave];
        // tile t has landed once nothing of ours is in flight; then start tile t+1
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        row_cur = row_nxt;
        if (t + 1 < n_tiles) {
            issue(row_cur, &sm.tile[stage ^ 1][wave]);
            row_nxt = row_of(t + 2);
        }

        // ---- partial scores over this wave's dims ----
        f32x16 acc_a, acc_b, acc_r;
#pragma unroll
        for (int i = 0; i < 16; i++) { acc_a[i] = 0.0f; acc_b[i] = 0.0f; acc_r[i] = 0.0f; }
#pragma unroll
        for (int j = 0; j < 5; j++) {
            if (j == 4 && !has_rope) break;
            const u32x4 raw = j < 4 ? *(const u32x4 *)&B.own[2 * j + g][m][0] : *(const u32x4 *)&B.rope[g][m][0];
            u32x4 ka, kb;
            ka[0] = e4m3x2_to_bf16x2<false>(raw[0]);
            ka[1] = e4m3x2_to_bf16x2<true>(raw[0]);
            ka[2] = e4m3x2_to_bf16x2<false>(raw[1]);
            ka[3] = e4m3x2_to_bf16x2<true>(raw[1]);
            kb[0] = e4m3x2_to_bf16x2<false>(raw[2]);
            kb[1] = e4m3x2_to_bf16x2<true>(raw[2]);
            kb[2] = e4m3x2_to_bf16x2<false>(raw[3]);
            kb[3] = e4m3x2_to_bf16x2<true>(raw[3]);
            if (j < 4) {
                acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka), qf[2 * j], acc_a, 0, 0, 0);
                acc_b = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb), qf[2 * j + 1], acc_b, 0, 0, 0);
            } else {
                acc_r = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka), qf[8], acc_r, 0, 0, 0);
                acc_r = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb), qf[9], acc_r, 0, 0, 0);
            }
        }
        // accumulator register i <-> position (i/4)*8 + 4g + i%4; apply the block scales
        // and publish the partial
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 s_own = *(const f32x4 *)&B.sc[0][8 * q4 + 4 * g];
            const f32x4 s_rope = *(const f32x4 *)&B.sc[1][8 * q4 + 4 * g];
            f32x4 part;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                part[r] = (acc_a[4 * q4 + r] + acc_b[4 * q4 + r]) * s_own[r];
                if (has_rope) part[r] = __builtin_fmaf(acc_r[4 * q4 + r], s_rope[r], part[r]);
            }
            *(f32x4 *)&sm.sx[stage][wave][q4][lane][0] = part;
        }

        // ---- normaliser of this wave's fp16 value weights ----
        float o_shift = 1.0f;
        {
            float sv = (my_valid && g == 0) ? B.sc[0][m] : 0.0f;
            sv = wave_max(sv);
            const uint32_t mb = __builtin_bit_cast(uint32_t, sv);
            const int e_tile = sv > 0.0f ? (int)((mb >> 23) & 0xFFu) - 126 : E_NONE;
            if (e_tile > e_run) {
                if (e_run != E_NONE) o_shift = pow2i(e_run - e_tile);
                e_run = e_tile;
            }
        }
        const float wfac = e_run == E_NONE ? 0.0f : pow2i(WEXP - e_run);

        __syncthreads();          // all four partials of this tile are in sx[stage]

        // ---- full scores: every wave sums the four partials in the same order ----
        f32x16 S;
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            f32x4 a = *(const f32x4 *)&sm.sx[stage][0][q4][lane][0];
            const f32x4 b = *(const f32x4 *)&sm.sx[stage][1][q4][lane][0];
            const f32x4 c = *(const f32x4 *)&sm.sx[stage][2][q4][lane][0];
            const f32x4 d = *(const f32x4 *)&sm.sx[stage][3][q4][lane][0];
#pragma unroll
            for (int r = 0; r < 4; r++) S[4 * q4 + r] = ((a[r] + b[r]) + (c[r] + d[r])) * c0;
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int pos = (i >> 2) * 8 + 4 * g + (i & 3);
            if (!((valid >> pos) & 1u)) S[i] = -INFINITY;
            tmax = fmaxf(tmax, S[i]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const bool bump = tmax > m_ref + LAZY;
        if (__any(bump) || o_shift != 1.0f) {
            const float m_new = bump ? tmax : m_ref;
            const float corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_ref - m_new);
            m_ref = m_new;
            l_part *= corr;
            const float oc = corr * o_shift;
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[db][i] *= oc;
        }
        const float m_use = m_ref == -INFINITY ? 0.0f : m_ref;
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            S[i] = __builtin_amdgcn_exp2f(S[i] - m_use);      // masked: exp2(-inf) = 0
            psum += S[i];
        }
        l_part += psum;

        // ---- values for this wave's 128 dims: weights p * scale[key][w] ----
        u32x4 pw[2];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 s4 = *(const f32x4 *)&B.sc[0][8 * q4 + 4 * g];
            pw[q4 >> 1][2 * (q4 & 1)] = pack_f16_rne(S[4 * q4 + 0] * (s4[0] * wfac), S[4 * q4 + 1] * (s4[1] * wfac));
            pw[q4 >> 1][2 * (q4 & 1) + 1] = pack_f16_rne(S[4 * q4 + 2] * (s4[2] * wfac), S[4 * q4 + 3] * (s4[3] * wfac));
        }
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const i32x2 raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (lds_i32x2 *)&B.own[2 * db + tr_dgo][16 * s + tr_pos][tr_byte]);
                u32x4 vh;
                vh[0] = e4m3x2_to_f16x2<false>((uint32_t)raw[0]);
                vh[1] = e4m3x2_to_f16x2<true>((uint32_t)raw[0]);
                vh[2] = e4m3x2_to_f16x2<false>((uint32_t)raw[1]);
                vh[3] = e4m3x2_to_f16x2<true>((uint32_t)raw[1]);
                oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    __builtin_bit_cast(f16x8, vh), __builtin_bit_cast(f16x8, pw[s]), oacc[db], 0, 0, 0);
            }
    }

    // ---- epilogue: every wave writes its own 128 dims ----
    const int head = hb * ROWS + m;
    if (head >= p.nh) return;
    const float L = l_part + __shfl_xor(l_part, 32, 64);     // same in all four waves
    const float unit_f = e_run == E_NONE ? 0.0f : pow2i(e_run - WEXP);
    if (p.n_splits == 1) {
        const float inv = L > 0.0f ? unit_f / L : 0.0f;
        float *o = p.out + ((size_t)y * p.nh + head) * VDIM + 128 * wave + 4 * g;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r] * inv;
                *(f32x4 *)(o + 32 * db + 8 * q4) = v;
            }
    } else {
        const size_t pr = ((size_t)y * p.n_splits + split) * p.nh + head;
        float *o = p.part_acc + pr * VDIM + 128 * wave + 4 * g;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r] * unit_f;
                *(f32x4 *)(o + 32 * db + 8 * q4) = v;
            }
        if (wave == 0 && g == 0) {
            p.part_ml[pr * 2 + 0] = m_ref * 0.69314718055994530942f;   // the merge pass works in e-units
            p.part_ml[pr * 2 + 1] = L;
        }
    }
}

int run(Params &p, hipStream_t s) {
    static bool attr_set = false;
    const size_t smem = sizeof(Smem);
    if (!attr_set) {
        CWICK_HIP_CALL(hipFuncSetAttribute((const void *)mla_dsplit_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const int n_hb = (p.nh + ROWS - 1) / ROWS;
    const int64_t total = (int64_t)n_hb * p.n_splits * p.nq;
    CWICK_REQUIRE(total <= 0x7FFFFFFF, "mla: grid of %lld workgroups is too large", (long long)total);
    if (p.n_splits > 1) {
        const size_t acc_b = (size_t)p.nq * p.n_splits * p.nh * VDIM * sizeof(float);
        const size_t ml_b = (size_t)p.nq * p.n_splits * p.nh * 2 * sizeof(float);
        char *ws = (char *)workspace(s, acc_b + ml_b);
        CWICK_REQUIRE(ws, "mla: workspace allocation failed");
        p.part_acc = (float *)ws;
        p.part_ml = (float *)(ws + acc_b);
    }
    {
        ProfScope ps(CWICK_HIP_PROF_MLA, s);
        mla_dsplit_kernel<<<dim3((unsigned)total), THREADS, smem, s>>>(p);
    }
    CWICK_HIP_CALL(hipGetLastError());
    if (p.n_splits > 1) {
        ProfScope ps(CWICK_HIP_PROF_MLA_MERGE, s);
        splitk_merge_kernel<VDIM><<<dim3(p.nh, p.nq), 256, 0, s>>>(p.part_acc, p.part_ml, p.n_splits, p.nh, p.out);
        CWICK_HIP_CALL(hipGetLastError());
    }
    return 1;
}

// CWICK_HIP_MLA = v1 | stream selects an earlier schedule (comparison arms)
int variant() {
    static int v = -1;
    if (v < 0) {
        const char *e = getenv("CWICK_HIP_MLA");
        v = !e ? 0 : (!strcmp(e, "v1") ? 1 : (!strcmp(e, "stream") ? 2 : 0));
    }
    return v;
}

int splits_per_cu() {
    static int v = -1;
    if (v < 0) {
        const char *e = getenv("CWICK_HIP_MLA_WG_PER_CU");
        v = e ? atoi(e) : 2;
        if (v < 1 || v > 8) v = 2;
    }
    return v;
}

}  // namespace

int launch_mla_decode(const uint8_t *rows, const float *scales, int64_t row_bstride,
                      int64_t scale_bstride, int64_t n_rows, int batch, const int32_t *sel,
                      int64_t n_list, const uint16_t *q, int n_heads, float scale, float *out,
                      hipStream_t s) {
    if (variant() == 1)
        return launch_mla_decode_v1(rows, scales, row_bstride, scale_bstride, n_rows, batch, sel, n_list,
                                    q, n_heads, scale, out, s);
    if (variant() == 2)
        return launch_mla_decode_v2(rows, scales, row_bstride, scale_bstride, n_rows, batch, sel, n_list,
                                    q, n_heads, scale, out, s);
    CWICK_REQUIRE(rows && scales && q && out, "mla_decode: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 4096, "mla_decode: batch %d", batch);
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "mla_decode: n_heads %d (1..128)", n_heads);
    CWICK_REQUIRE(n_rows >= 1 && n_rows <= ((int64_t)1 << 31) - 1, "mla_decode: n_rows %lld",
                  (long long)n_rows);
    CWICK_REQUIRE(n_list >= 1 && n_list <= ((int64_t)1 << 31) - 1, "mla_decode: n_list %lld",
                  (long long)n_list);
    CWICK_REQUIRE(sel || n_list <= n_rows, "mla_decode: n_list %lld exceeds n_rows %lld",
                  (long long)n_list, (long long)n_rows);
    CWICK_REQUIRE(scale > 0.0f && scale < INFINITY, "mla_decode: scale must be positive");
    CWICK_REQUIRE((uintptr_t)rows % 16 == 0 && row_bstride % 16 == 0 && (uintptr_t)q % 16 == 0 &&
                      (uintptr_t)out % 16 == 0 && (uintptr_t)scales % 4 == 0,
                  "mla_decode: rows, q and out must be 16-byte aligned");
    Params p{};
    p.rows = rows; p.scales = scales; p.row_bstride = row_bstride; p.scale_bstride = scale_bstride;
    p.n_rows = n_rows; p.sel = sel; p.n_list = n_list; p.list_step = 0;
    p.q = q; p.nh = n_heads; p.nq = batch; p.scale = scale; p.out = out;
    // two workgroups are resident per CU: one round of workgroups
    const int n_hb = (n_heads + ROWS - 1) / ROWS;
    int64_t want = (int64_t)splits_per_cu() * num_cus() / ((int64_t)n_hb * batch);
    if (want < 1) want = 1;
    if (want > MERGE_MAX_SPLITS) want = MERGE_MAX_SPLITS;
    int64_t per = (n_list + want - 1) / want;
    per = ((per + TK - 1) / TK) * TK;
    p.keys_per_split = per;
    p.n_splits = (int)((n_list + per - 1) / per);
    return run(p, s);
}

int launch_mla_prefill(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                       const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s) {
    if (variant() == 1) return launch_mla_prefill_v1(rows, scales, pos0, n, q, n_heads, scale, out, s);
    if (variant() == 2) return launch_mla_prefill_v2(rows, scales, pos0, n, q, n_heads, scale, out, s);
    CWICK_REQUIRE(rows && scales && q && out, "mla_prefill: null pointer");
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "mla_prefill: n_heads %d (1..128)", n_heads);
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= ((int64_t)1 << 31) - 1 && n <= (1 << 22),
                  "mla_prefill: pos0 %lld n %lld", (long long)pos0, (long long)n);
    CWICK_REQUIRE(scale > 0.0f && scale < INFINITY, "mla_prefill: scale must be positive");
    CWICK_REQUIRE((uintptr_t)rows % 16 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)out % 16 == 0,
                  "mla_prefill: rows, q and out must be 16-byte aligned");
    Params p{};
    p.rows = rows; p.scales = scales; p.row_bstride = 0; p.scale_bstride = 0;
    p.n_rows = pos0 + n; p.sel = nullptr; p.n_list = pos0 + 1; p.list_step = 1;
    p.q = q; p.nh = n_heads; p.nq = (int)n; p.scale = scale; p.out = out;
    p.n_splits = 1;
    p.keys_per_split = ((pos0 + n + TK - 1) / TK) * TK;
    return run(p, s);
}

}  // namespace cwick
