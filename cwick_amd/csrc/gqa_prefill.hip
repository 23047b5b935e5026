// gqa_prefill.hip -- causal GQA prefill on the bf16 matrix cores (the prefill
// branch of the reference's mixer_attn, src/q35_model.c:1713-1746: per head and
// per 128-query tile S = scale*Q*K^T over the rectangle, -1e30 tail, softmax,
// O = S*V).  Here: one pass, online softmax, the triangle only.
//
// MFMA-bound.  Work decomposition
//   workgroup = 4 waves = 128 query rows that share one kv head: the GROUP
//   query heads of the kv head times P = 128/GROUP consecutive positions
//   (heads-as-M: K and V tiles are read once for all heads of the group).
//   wave = 32 rows.  Key tiles of TK = 32, K and V copied global -> LDS as they
//   are ([key][dim] bf16, double buffered, next tile prefetched in registers).
//   scores:  S^T[key][row] = K[key][dim] . Q^T[dim][row], v_mfma_f32_32x32x16_bf16,
//            K fragments from LDS, Q fragments resident in registers.
//            One query row per lane column: softmax statistics are per-lane.
//   values:  O^T[dim][row] += V^T[dim][key] . P^T[key][row].  P^T is the score
//            accumulator itself (rounded to bf16) -- its register layout is the
//            B-operand layout once the contraction slots are numbered to match;
//            V^T fragments come out of the row-major V tile through the LDS
//            transpose read (ds_read_b64_tr_b16), so nothing is transposed by hand.
//   The running maximum is only advanced when a tile beats it by more than 8
//   (in log2 units), so the 128 output registers are rescaled a few times per
//   row block instead of once per tile.
#include "common.hpp"

namespace cwick {

constexpr int PF_THREADS = 256;
constexpr int PF_TK = 32;
constexpr int PF_HD = 256;
constexpr int PF_LD = PF_HD + 8;            // LDS row stride in bf16 (16 B pad)
constexpr int PF_ROWS = 128;                // query rows per workgroup
// Resident workgroups per CU the register budget is sized for: 1 leaves each
// wave the whole 512-register file (Q fragments 64 + output 128 + staging),
// 2 would need the kernel to fit 256 and spills today.
constexpr int PF_WG_PER_CU = 1;

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

struct PfSmem {
    uint16_t k[2][PF_TK][PF_LD];
    uint16_t v[2][PF_TK][PF_LD];
};

template <int GROUP>
__global__ void __launch_bounds__(PF_THREADS, PF_WG_PER_CU)
gqa_prefill_kernel(const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
                   const uint16_t *__restrict__ Q, int64_t pos0, int64_t n, int n_kv_heads,
                   float scale_log2e, float *__restrict__ out) {
    constexpr int P = PF_ROWS / GROUP;      // positions per workgroup
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    PfSmem &sm = *reinterpret_cast<PfSmem *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int g = lane >> 5;                // 0/1

    const int kvh = blockIdx.y;
    // heavy (late) position blocks first: better tail balance under the causal triangle
    const int64_t pblk = (int64_t)gridDim.x - 1 - blockIdx.x;
    const int64_t t0 = pblk * P;
    const int n_heads = n_kv_heads * GROUP;
    const int64_t kv_stride = (int64_t)n_kv_heads * PF_HD;
    const int64_t q_stride = (int64_t)n_heads * PF_HD;
    const int64_t n_keys_all = pos0 + n;

    // this lane's query row
    const int r = wave * 32 + l32;
    const int j = r / P;                    // head within the group
    const int64_t t = t0 + (r % P);         // position within the chunk
    const bool row_live = t < n;
    const int64_t tq = row_live ? t : n - 1;
    const int64_t my_limit = pos0 + tq;     // last visible key

    // Q fragments: B operand, lane (row, g) holds dims 16ks+8g .. +8
    bf16x8 qf[16];
    {
        const uint16_t *qrow = Q + tq * q_stride + (size_t)(kvh * GROUP + j) * PF_HD + 8 * g;
#pragma unroll
        for (int ks = 0; ks < 16; ks++)
            qf[ks] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + 16 * ks));
    }

    f32x16 oacc[8];
#pragma unroll
    for (int db = 0; db < 8; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = 0.0f;
    float m_ref = -INFINITY, l_part = 0.0f;

    // keys 0 .. last position of the block (clipped to the chunk)
    int64_t last_t = t0 + P - 1;
    if (last_t > n - 1) last_t = n - 1;
    const int64_t wg_keys = pos0 + last_t + 1;
    const int n_tiles = (int)((wg_keys + PF_TK - 1) / PF_TK);
    const int64_t first_masked_key = pos0 + t0;   // tiles ending at or below this need no mask
    const bool precise = wg_keys <= 2048;         // workgroup-uniform

    const uint16_t *Kg = K + (size_t)kvh * PF_HD;
    const uint16_t *Vg = V + (size_t)kvh * PF_HD;

    // global -> register staging of one tile: 32 rows x 512 B, 4 x 16 B per thread
    // One set of staging registers serves K (in flight during the score MFMAs)
    // and then V (in flight during softmax and the value MFMAs).
    u32x4 st[4];
    auto load_rows = [&](const uint16_t *base, int tile) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = tid + PF_THREADS * i;
            int64_t row = (int64_t)tile * PF_TK + (c >> 5);
            if (row > n_keys_all - 1) row = n_keys_all - 1;     // masked anyway
            st[i] = *(const u32x4 *)(base + row * kv_stride + (c & 31) * 8);
        }
    };
    auto store_rows = [&](uint16_t (*dst)[PF_LD]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = tid + PF_THREADS * i;
            *(u32x4 *)&dst[c >> 5][(c & 31) * 8] = st[i];
        }
    };

    load_rows(Kg, 0);
    store_rows(sm.k[0]);
    load_rows(Vg, 0);
    store_rows(sm.v[0]);
    __syncthreads();

    for (int tile = 0; tile < n_tiles; tile++) {
        const int buf = tile & 1;
        const bool more = tile + 1 < n_tiles;
        if (more) load_rows(Kg, tile + 1);

        // ---- scores: S^T[32 keys][32 rows] ----
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            const bf16x8 ka = __builtin_bit_cast(bf16x8, *(const u32x4 *)&sm.k[buf][l32][16 * ks + 8 * g]);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[ks], s, 0, 0, 0);
        }
        if (more) {
            store_rows(sm.k[buf ^ 1]);
            load_rows(Vg, tile + 1);
        }
        // register i holds key (i/4)*8 + 4g + i%4 of the tile for this lane's row
        const int64_t key0 = (int64_t)tile * PF_TK;
        const bool need_mask = key0 + PF_TK - 1 > first_masked_key;
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float x = s[i] * scale_log2e;
            if (need_mask) {
                const int64_t key = key0 + (i >> 2) * 8 + 4 * g + (i & 3);
                if (key > my_limit) x = -INFINITY;
            }
            s[i] = x;
            tmax = fmaxf(tmax, x);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        if (__any(tmax > m_ref + 8.0f)) {
            const float m_new = fmaxf(m_ref, tmax);
            const float corr = __builtin_amdgcn_exp2f(m_ref - m_new);       // first tile: exp2(-inf) = 0
            m_ref = m_new;
            l_part *= corr;
#pragma unroll
            for (int db = 0; db < 8; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[db][i] *= corr;
        }
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            s[i] = __builtin_amdgcn_exp2f(s[i] - m_ref);                    // masked: 0
            psum += s[i];
        }
        l_part += psum;

        // ---- values: two k-steps of 16 keys ----
        // contraction slot (g, jj) of step ks2 <-> tile key 16*ks2 + (jj/4)*8 + 4g + jj%4,
        // i.e. score register 8*ks2 + jj: P^T needs no data movement.
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ks2++) {
            u32x4 pw;
#pragma unroll
            for (int h = 0; h < 4; h++)
                pw[h] = pack_bf16_rne(s[8 * ks2 + 2 * h], s[8 * ks2 + 2 * h + 1]);
            const bf16x8 pb = __builtin_bit_cast(bf16x8, pw);
            // Short prefixes: few keys carry the whole weight, so the 2^-9 rounding of
            // each bf16 weight shows in an O(1) output.  There the rounding residual
            // goes through the matrix core as well (weights good to 2^-17).
            bf16x8 pb_lo = pb;
            if (precise) {
                u32x4 pl;
#pragma unroll
                for (int h = 0; h < 4; h++)
                    pl[h] = pack_bf16_rne(s[8 * ks2 + 2 * h] - bf16lo_to_f32(pw[h]),
                                          s[8 * ks2 + 2 * h + 1] - bf16hi_to_f32(pw[h]));
                pb_lo = __builtin_bit_cast(bf16x8, pl);
            }
            // transpose read: within a 16-lane group, lane i addresses key (i/4), dims
            // 4*(i%4)..+4 of a 4 x 16 tile and receives dim (i) for the 4 keys.
            const int grp = lane >> 4;                    // 16-lane group 0..3
            const int gi = lane & 15;
            const int dim_in = 16 * (grp & 1) + 4 * (gi & 3);
            const int key_a = 16 * ks2 + 4 * (grp >> 1) + (gi >> 2);   // slots jj = 0..3
            const int key_b = key_a + 8;                                // slots jj = 4..7
#pragma unroll
            for (int db = 0; db < 8; db++) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4 *)&sm.v[buf][key_a][32 * db + dim_in]);
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4 *)&sm.v[buf][key_b][32 * db + dim_in]);
                typedef __attribute__((ext_vector_type(8))) short s16x8;
                const s16x8 va8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, va8), pb,
                                                                   oacc[db], 0, 0, 0);
                if (precise)
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, va8), pb_lo, oacc[db], 0, 0, 0);
            }
        }

        if (more) store_rows(sm.v[buf ^ 1]);
        __syncthreads();
    }

    // ---- epilogue ----
    const float l = l_part + __shfl_xor(l_part, 32, 64);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    if (row_live) {
        float *o = out + t * q_stride + (size_t)(kvh * GROUP + j) * PF_HD + 4 * g;
#pragma unroll
        for (int db = 0; db < 8; db++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                f32x4 w;
#pragma unroll
                for (int i = 0; i < 4; i++) w[i] = oacc[db][4 * b4 + i] * inv;
                *(f32x4 *)(o + 32 * db + 8 * b4) = w;
            }
    }
}

template <int GROUP>
static int run_gqa_prefill(const uint16_t *k, const uint16_t *v, int64_t pos0, int64_t n,
                           int n_kv_heads, const uint16_t *q, float scale, float *out,
                           hipStream_t s) {
    static bool attr_set = false;
    const size_t smem = sizeof(PfSmem);
    if (!attr_set) {
        CWICK_HIP_CALL(hipFuncSetAttribute((const void *)gqa_prefill_kernel<GROUP>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    constexpr int P = PF_ROWS / GROUP;
    const int64_t pblocks = (n + P - 1) / P;
    CWICK_REQUIRE(pblocks <= 0x7FFFFFFF && n_kv_heads <= 65535, "gqa_prefill: grid too large");
    {
        ProfScope ps(CWICK_HIP_PROF_GQA_PREFILL, s);
        gqa_prefill_kernel<GROUP><<<dim3((unsigned)pblocks, n_kv_heads), PF_THREADS, smem, s>>>(
            k, v, q, pos0, n, n_kv_heads, scale * 1.44269504088896340736f, out);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_gqa_prefill(const uint16_t *k, const uint16_t *v, int64_t pos0, int64_t n,
                       int n_kv_heads, int head_dim, const uint16_t *q, int n_heads, float scale,
                       float *out, hipStream_t s) {
    CWICK_REQUIRE(k && v && q && out, "gqa_prefill: null pointer");
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= ((int64_t)1 << 30),
                  "gqa_prefill: pos0 %lld n %lld", (long long)pos0, (long long)n);
    CWICK_REQUIRE(head_dim == PF_HD, "gqa_prefill: head_dim %d is not supported (256 only)", head_dim);
    CWICK_REQUIRE(n_kv_heads >= 1 && n_heads >= n_kv_heads && n_heads % n_kv_heads == 0,
                  "gqa_prefill: n_heads %d is not a multiple of n_kv_heads %d", n_heads, n_kv_heads);
    CWICK_REQUIRE(scale > 0.0f && scale < INFINITY, "gqa_prefill: scale must be positive");
    CWICK_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)q | (uintptr_t)out) % 16 == 0,
                  "gqa_prefill: K, V, q and out must be 16-byte aligned");
    switch (n_heads / n_kv_heads) {
        case 1: return run_gqa_prefill<1>(k, v, pos0, n, n_kv_heads, q, scale, out, s);
        case 2: return run_gqa_prefill<2>(k, v, pos0, n, n_kv_heads, q, scale, out, s);
        case 4: return run_gqa_prefill<4>(k, v, pos0, n, n_kv_heads, q, scale, out, s);
        case 8: return run_gqa_prefill<8>(k, v, pos0, n, n_kv_heads, q, scale, out, s);
        default: break;
    }
    set_error("gqa_prefill: group %d is not supported (1, 2, 4, 8)", n_heads / n_kv_heads);
    return 0;
}

}  // namespace cwick
