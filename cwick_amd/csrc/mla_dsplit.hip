// mla_dsplit.hip -- absorbed-latent MLA with the contraction split over the waves
// (decode, sparse decode and chunked prefill of src/attention.c:749-811 /
// :1010-1019 over the FP8 latent).  An earlier schedule than the one the entry
// points use (mla_roles.hip), kept selectable as a comparison arm
// (CWICK_HIP_MLA=dsplit).
//
//   workgroup = 8 waves = 2 teams of 4, 32 query rows (heads of one query) x one
//   key slice; the teams take alternate 32-key tiles of the slice and meet once,
//   at the end, through LDS -- so one workgroup per CU leaves one partial per CU
//   (the partial volume written for the merge pass is what the whole step pays
//   most for).  In a team, wave w owns latent dims 128w..128w+127 -- one scale
//   block -- for BOTH products:
//     scores   S^T[key][head]: the wave computes the partial dot over its 128 dims
//              (waves 0 and 1 also take 32 rope dims each), times its block's
//              fp32 scale; the four partials meet in LDS, where wave w sums
//              quarter w of the tile (8 keys), takes exp2 against the running
//              reference and publishes weights, scores and the quarter maximum;
//     values   O^T[dim][head]: every wave reads the 32 weights back and produces
//              exactly its 128 output dims, with weights p * scale[key][w].
//   The running reference moves only when a tile exceeds it by 2^LAZY (always on
//   the first tile); all four waves see the same maxima and take the same branch,
//   then recompute the weights from the published scores.
//   A wave touches only its own slice of every latent row: it fetches that slice
//   itself (global -> LDS by global_load_lds_dwordx4, no registers, one tile
//   ahead).  The copies are issued from inline assembly and the barriers wait
//   for LDS traffic only, so the tile in flight stays in flight across them.
//
//   LDS tile layout [16-dim group][key position 0..31][16 B]: the K fragment
//   (A operand of S^T = K Q^T, v_mfma_f32_32x32x16_bf16) is a 16-byte read per
//   lane, 1 KiB contiguous per wave; the V^T fragment (A operand of
//   O^T = V^T P^T, v_mfma_f32_32x32x16_f16) comes from ds_read_b64_tr_b8, 128 B
//   contiguous per 16-lane group.  P^T is the score tile itself: one head per
//   lane column, contraction slots numbered to match the accumulator layout.
//
//   Split-K partials are stored in accumulator-fragment order
//   [split][head block][wave][db][q4][lane][4] (every store 1 KiB contiguous);
//   mla_merge_frag_kernel reads them in the same order with all loads in flight.
#include "common.hpp"
#include "merge.hpp"

#include <cstdlib>
#include <cstring>

namespace cwick {
namespace {

constexpr int KDIM = CWICK_HIP_LATENT_KDIM;   // 576
constexpr int VDIM = CWICK_HIP_LATENT_VDIM;   // 512
constexpr int NBLK = CWICK_HIP_LATENT_NBLK;   // 5
constexpr int THREADS = 512;
constexpr int TEAMS = 2;
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
    int64_t keys_per_split;   // multiple of TEAMS * TK
    float *out, *part_acc, *part_ml;
};

// what one wave keeps of one tile
struct WaveTile {
    uint8_t own[8][TK][16];       // its 8 sixteen-dim groups (128 dims)            4096 B
    uint8_t rope[2][TK][16];      // one rope pair (waves 0 and 1)                  1024 B
    float sc[2][TK];              // [0] scale of its block, [1] scale of the rope   256 B
};
// what the four waves of a team exchange per tile
struct TeamX {
    float sx[4][4][64][4];        // [wave][quarter][lane][4]: partial scores       16 KiB
    float ps[4][64][4];           // [quarter][lane][4]: weights exp2(s - m_ref)     4 KiB
    float ss[4][64][4];           // [quarter][lane][4]: scaled, masked scores       4 KiB
    float qm[4][64];              // [quarter][lane]: maximum of the quarter         1 KiB
};
struct Smem {
    WaveTile tile[2][TEAMS][4];   // [stage][team][wave]                            84 KiB
    TeamX x[TEAMS];               //                                                50 KiB
    float lq[TEAMS][4][64];       // per-wave row sums at the end
    float mt[TEAMS][64];          // per-team running reference at the end
    int et[TEAMS][4];             // per-wave weight exponent at the end
};

// workgroup barrier that orders LDS traffic only: a __syncthreads() would also wait for the
// global->LDS copies of the next tile, which are meant to stay in flight across it
#define LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

__device__ __forceinline__ float pow2i(int e) {
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
    return __builtin_bit_cast(float, (uint32_t)(e + 127) << 23);
}

__global__ void __launch_bounds__(THREADS, 2) mla_dsplit_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    Smem &sm = *reinterpret_cast<Smem *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);   // = scale block = dim slice = score quarter
    const int team = __builtin_amdgcn_readfirstlane(tid >> 8);         // teams take alternate tiles of the slice
    const int m = lane & 31;           // key position (scores) / head column / dim row
    const int g = lane >> 5;           // which half of the contraction slots
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
    const int n_iter = (n_tiles + TEAMS - 1) / TEAMS;   // both teams run this many rounds

    // row of this lane's key position in round j (tile TEAMS*j + team), -1 = masked
    auto row_of = [&](int j) -> int {
        const int t = TEAMS * j + team;
        const int64_t i = k_begin + (int64_t)t * TK + m;
        int64_t r = -1;
        if (t < n_tiles && i < k_end) {
            r = sel ? (int64_t)sel[i] : i;
            if (r < 0 || r >= p.n_rows) r = -1;
        }
        return (int)r;
    };
    // global -> LDS copies, written as assembly so that the compiler keeps no account of them:
    // it would otherwise wait for the tile in flight before unrelated LDS reads and barriers.
    // The loop waits for them itself (s_waitcnt vmcnt(0) at its top).
    auto dma16 = [&](const void *gp, const void *lp) {
        const uint32_t off = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void *)lp);
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gp), "s"(off) : "memory");
    };
    auto dma4 = [&](const void *gp, const void *lp) {
        const uint32_t off = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void *)lp);
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gp), "s"(off) : "memory");
    };
    auto issue = [&](int r, WaveTile *b) {
        const int64_t rc = r >= 0 ? r : 0;            // masked positions fetch row 0, weight 0
        const uint8_t *gsrc = rows + rc * KDIM + 128 * wave + 16 * g;
#pragma unroll
        for (int n = 0; n < 4; n++) dma16(gsrc + 32 * n, &b->own[2 * n][0][0]);
        const uint8_t *rsrc = has_rope ? rows + rc * KDIM + 512 + 32 * wave + 16 * g : gsrc;
        dma16(rsrc, &b->rope[0][0][0]);
        const float *ssrc = scales + rc * NBLK + (g ? 4 : wave);
        dma4(ssrc, &b->sc[0][0]);
    };

    int row_cur = row_of(0);
    int row_nxt = row_of(1);
    if (n_iter > 0) issue(row_cur, &sm.tile[0][team][wave]);

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

    // the Q fragments are complete before the loop: nothing in it has to wait for them
#pragma unroll
    for (int i = 0; i < 10; i++) asm volatile("" : "+v"(qf[i]));
    f32x16 oacc[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = 0.0f;
    float m_ref = -INFINITY, l_q = 0.0f;
    int e_run = E_NONE;
    const float c0 = p.scale * 1.44269504088896340736f;   // scores live in log2 units

    const int G = lane >> 4, gi = lane & 15;
    const int tr_k = gi >> 1;
    const int tr_pos = 4 * (G >> 1) + (tr_k & 3) + 8 * (tr_k >> 2);   // + 16 s
    const int tr_dgo = G & 1;                                         // + 2 db
    const int tr_byte = 8 * (gi & 1);
    TeamX &X = sm.x[team];

    for (int j = 0; j < n_iter; j++) {
        const int stage = j & 1;
        const uint32_t valid = (uint32_t)__ballot(row_cur >= 0);      // lanes 0..31 <-> positions
        WaveTile &B = sm.tile[stage][team][wave];
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        row_cur = row_nxt;
        if (j + 1 < n_iter) {
            row_nxt = row_of(j + 2);      // (a list entry, when there is a list, arrives before the copies start)
            issue(row_cur, &sm.tile[stage ^ 1][team][wave]);
        }

        // ---- phase 1: partial scores over this wave's dims ----
        f32x16 acc_a, acc_b, acc_r;
#pragma unroll
        for (int i = 0; i < 16; i++) { acc_a[i] = 0.0f; acc_b[i] = 0.0f; acc_r[i] = 0.0f; }
#pragma unroll
        for (int jj = 0; jj < 5; jj++) {
            if (jj == 4 && !has_rope) break;
            const u32x4 raw = jj < 4 ? *(const u32x4 *)&B.own[2 * jj + g][m][0] : *(const u32x4 *)&B.rope[g][m][0];
            u32x4 ka, kb;
            ka[0] = e4m3x2_to_bf16x2<false>(raw[0]);
            ka[1] = e4m3x2_to_bf16x2<true>(raw[0]);
            ka[2] = e4m3x2_to_bf16x2<false>(raw[1]);
            ka[3] = e4m3x2_to_bf16x2<true>(raw[1]);
            kb[0] = e4m3x2_to_bf16x2<false>(raw[2]);
            kb[1] = e4m3x2_to_bf16x2<true>(raw[2]);
            kb[2] = e4m3x2_to_bf16x2<false>(raw[3]);
            kb[3] = e4m3x2_to_bf16x2<true>(raw[3]);
            if (jj < 4) {
                acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka), qf[2 * jj], acc_a, 0, 0, 0);
                acc_b = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb), qf[2 * jj + 1], acc_b, 0, 0, 0);
            } else {
                acc_r = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka), qf[8], acc_r, 0, 0, 0);
                acc_r = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb), qf[9], acc_r, 0, 0, 0);
            }
        }
        // accumulator register i <-> position (i/4)*8 + 4g + i%4
        f32x4 sown[4];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 s_own = *(const f32x4 *)&B.sc[0][8 * q4 + 4 * g];
            const f32x4 s_rope = *(const f32x4 *)&B.sc[1][8 * q4 + 4 * g];
            sown[q4] = s_own;
            f32x4 part;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                part[r] = (acc_a[4 * q4 + r] + acc_b[4 * q4 + r]) * s_own[r];
                if (has_rope) part[r] = __builtin_fmaf(acc_r[4 * q4 + r], s_rope[r], part[r]);
            }
            *(f32x4 *)&X.sx[wave][q4][lane][0] = part;
        }
        // normaliser of this wave's fp16 value weights: largest scale among the valid keys
        float o_shift = 1.0f;
        {
            float sv = 0.0f;
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float v = sown[q4][r];
                    if (valid != 0xFFFFFFFFu && !((valid >> (8 * q4 + 4 * g + r)) & 1u)) v = 0.0f;
                    sv = fmaxf(sv, v);
                }
            sv = fmaxf(sv, __shfl_xor(sv, 32, 64));
            sv = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, sv)));
            const uint32_t mb = __builtin_bit_cast(uint32_t, sv);
            const int e_tile = sv > 0.0f ? (int)((mb >> 23) & 0xFFu) - 126 : E_NONE;
            if (e_tile > e_run) {
                if (e_run != E_NONE) o_shift = pow2i(e_run - e_tile);
                e_run = e_tile;
            }
        }
        const float wfac = e_run == E_NONE ? 0.0f : pow2i(WEXP - e_run);

        LDS_BARRIER();          // the four partials of each team's tile are in sx

        // ---- phase 2: this wave finishes quarter `wave` of the scores (positions 8 wave + 4 g + r) ----
        float p4sum;
        {
            const f32x4 a = *(const f32x4 *)&X.sx[0][wave][lane][0];
            const f32x4 b = *(const f32x4 *)&X.sx[1][wave][lane][0];
            const f32x4 c = *(const f32x4 *)&X.sx[2][wave][lane][0];
            const f32x4 d = *(const f32x4 *)&X.sx[3][wave][lane][0];
            f32x4 s4, p4;
            float qmax = -INFINITY;
            const float m_use = m_ref == -INFINITY ? 0.0f : m_ref;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                s4[r] = ((a[r] + b[r]) + (c[r] + d[r])) * c0;
                if (!((valid >> (8 * wave + 4 * g + r)) & 1u)) s4[r] = -INFINITY;
                qmax = fmaxf(qmax, s4[r]);
                p4[r] = __builtin_amdgcn_exp2f(s4[r] - m_use);
            }
            qmax = fmaxf(qmax, __shfl_xor(qmax, 32, 64));
            p4sum = (p4[0] + p4[1]) + (p4[2] + p4[3]);
            *(f32x4 *)&X.ps[wave][lane][0] = p4;
            *(f32x4 *)&X.ss[wave][lane][0] = s4;
            X.qm[wave][lane] = qmax;
        }

        LDS_BARRIER();          // weights, scores and quarter maxima of the tile are published

        // ---- phase 3: weights of the whole tile, values for this wave's 128 dims ----
        f32x16 P;
        const float tmax = fmaxf(fmaxf(X.qm[0][lane], X.qm[1][lane]), fmaxf(X.qm[2][lane], X.qm[3][lane]));
        const bool bump = tmax > m_ref + LAZY;
        float corr = 1.0f;
        if (__any(bump)) {
            // the running reference moves (always on the first tile): redo the weights from the scores
            const float m_new = bump ? tmax : m_ref;
            corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_ref - m_new);
            m_ref = m_new;
            const float m_use = m_ref == -INFINITY ? 0.0f : m_ref;
            float qs[4];
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const f32x4 s4 = *(const f32x4 *)&X.ss[q4][lane][0];
#pragma unroll
                for (int r = 0; r < 4; r++) P[4 * q4 + r] = __builtin_amdgcn_exp2f(s4[r] - m_use);
                qs[q4] = (P[4 * q4] + P[4 * q4 + 1]) + (P[4 * q4 + 2] + P[4 * q4 + 3]);
            }
            p4sum = wave == 0 ? qs[0] : (wave == 1 ? qs[1] : (wave == 2 ? qs[2] : qs[3]));
            l_q *= corr;
        } else {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const f32x4 p4 = *(const f32x4 *)&X.ps[q4][lane][0];
#pragma unroll
                for (int r = 0; r < 4; r++) P[4 * q4 + r] = p4[r];
            }
        }
        l_q += p4sum;
        const float oc = corr * o_shift;
        if (__any(oc != 1.0f)) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[db][i] *= oc;
        }

        u32x4 pw[2];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 s4 = sown[q4];
            pw[q4 >> 1][2 * (q4 & 1)] = pack_f16_rne(P[4 * q4 + 0] * (s4[0] * wfac), P[4 * q4 + 1] * (s4[1] * wfac));
            pw[q4 >> 1][2 * (q4 & 1) + 1] = pack_f16_rne(P[4 * q4 + 2] * (s4[2] * wfac), P[4 * q4 + 3] * (s4[3] * wfac));
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

    // ---- the two teams meet: team 1 parks its state in LDS (over the tile buffers) ----
    float (*park)[16][64][4] = reinterpret_cast<float (*)[16][64][4]>(&sm.tile[0][0][0]);   // [wave][i][lane][4]
    sm.lq[team][wave][lane] = l_q + __shfl_xor(l_q, 32, 64);
    if (wave == 0) sm.mt[team][lane] = m_ref;
    if (lane == 0) sm.et[team][wave] = e_run;
    LDS_BARRIER();              // nobody reads tiles any more
    if (team == 1) {
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r];
                *(f32x4 *)&park[wave][db * 4 + q4][lane][0] = v;
            }
    }
    LDS_BARRIER();
    if (team == 1) return;

    const float m0 = sm.mt[0][lane], m1 = sm.mt[1][lane];
    const float M = fmaxf(m0, m1);
    const float a0 = m0 == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m0 - M);
    const float a1 = m1 == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m1 - M);
    const int e0 = sm.et[0][wave], e1 = sm.et[1][wave];
    const int E = e0 > e1 ? e0 : e1;
    const float f0 = e0 == E_NONE ? 0.0f : a0 * pow2i(e0 - E);
    const float f1 = e1 == E_NONE ? 0.0f : a1 * pow2i(e1 - E);
    const float L = a0 * ((sm.lq[0][0][lane] + sm.lq[0][1][lane]) + (sm.lq[0][2][lane] + sm.lq[0][3][lane])) +
                    a1 * ((sm.lq[1][0][lane] + sm.lq[1][1][lane]) + (sm.lq[1][2][lane] + sm.lq[1][3][lane]));
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 v = *(const f32x4 *)&park[wave][db * 4 + q4][lane][0];
#pragma unroll
            for (int r = 0; r < 4; r++) oacc[db][4 * q4 + r] = oacc[db][4 * q4 + r] * f0 + v[r] * f1;
        }

    const int head = hb * ROWS + m;
    if (head >= p.nh) return;
    const float unit_f = E == E_NONE ? 0.0f : pow2i(E - WEXP);
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
        // fragment-native layout [y][split][hb][wave][db][q4][lane][4]: every store is 1 KiB contiguous
        const size_t pb = ((size_t)y * p.n_splits + split) * n_hb + hb;
        float *o = p.part_acc + pb * (ROWS * VDIM) + (size_t)wave * 4096 + lane * 4;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r] * unit_f;
                *(f32x4 *)(o + (db * 4 + q4) * 256) = v;
            }
        if (wave == 0 && g == 0) {
            p.part_ml[(pb * ROWS + m) * 2 + 0] = M * 0.69314718055994530942f;
            p.part_ml[(pb * ROWS + m) * 2 + 1] = L;
        }
    }
}

// merge of fragment-layout partials: workgroup = one group of 64 float4 (fixed wave, db, q4
// of one head block); its waves (up to sixteen, one per split when there are fewer) take
// splits w, w + n_waves, ... and meet in LDS.  Every wave has all its loads in flight at once
// (eight splits per batch); which splits exist is uniform per wave, so absent ones cost nothing.
constexpr int MW = 16;
__global__ void __launch_bounds__(64 * MW)
mla_merge_frag_kernel(const float *__restrict__ part_acc, const float *__restrict__ part_ml,
                      int n_splits, int n_hb, int nh, float *__restrict__ out) {
    __shared__ float red_m[MW][64];
    __shared__ float red_l[MW][64];
    __shared__ f32x4 red_a[MW][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6), mw = (int)blockDim.x >> 6;
    const int grp = blockIdx.x & 63, hb = blockIdx.x >> 6, y = blockIdx.y;
    const int m = lane & 31, g = lane >> 5;
    const size_t sb = (size_t)y * n_splits;
    const float *ml = part_ml + ((sb * n_hb + hb) * ROWS + m) * 2;
    const size_t ml_stride = (size_t)n_hb * ROWS * 2;
    const float *pa = part_acc + (sb * n_hb + hb) * (ROWS * VDIM) + (size_t)grp * 256 + lane * 4;
    const size_t pa_stride = (size_t)n_hb * ROWS * VDIM;

    // first batch: everything in flight before anything is waited for
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
    red_m[wv][lane] = mx;
    __syncthreads();
    for (int w = 0; w < mw; w++) mx = fmaxf(mx, red_m[w][lane]);

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
    red_l[wv][lane] = ls;
    red_a[wv][lane] = acc;
    __syncthreads();
    if (wv != 0) return;
    float l = 0.f;
    f32x4 r4 = {0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < mw; w++) {
        l += red_l[w][lane];
        const f32x4 t = red_a[w][lane];
#pragma unroll
        for (int r = 0; r < 4; r++) r4[r] += t[r];
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const int head = hb * ROWS + m;
    if (head >= nh) return;
    // grp = (wave*4 + db)*4 + q4 -> dims 128 wave + 32 db + 8 q4 + 4 g
    const int dim = 128 * (grp >> 4) + 32 * ((grp >> 2) & 3) + 8 * (grp & 3) + 4 * g;
#pragma unroll
    for (int r = 0; r < 4; r++) r4[r] *= inv;
    *(f32x4 *)(out + ((size_t)y * nh + head) * VDIM + dim) = r4;
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
        const size_t acc_b = (size_t)p.nq * p.n_splits * n_hb * ROWS * VDIM * sizeof(float);
        const size_t ml_b = (size_t)p.nq * p.n_splits * n_hb * ROWS * 2 * sizeof(float);
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
        mla_merge_frag_kernel<<<dim3(n_hb * 64, p.nq), 64 * (p.n_splits < MW ? p.n_splits : MW), 0, s>>>(p.part_acc, p.part_ml, p.n_splits, n_hb, p.nh, p.out);
        CWICK_HIP_CALL(hipGetLastError());
    }
    return 1;
}

int splits_per_cu() {
    static int v = -1;
    if (v < 0) {
        const char *e = getenv("CWICK_HIP_MLA_WG_PER_CU");
        v = e ? atoi(e) : 1;
        if (v < 1 || v > 8) v = 1;
    }
    return v;
}

}  // namespace

int launch_mla_decode_v3(const uint8_t *rows, const float *scales, int64_t row_bstride,
                      int64_t scale_bstride, int64_t n_rows, int batch, const int32_t *sel,
                      int64_t n_list, const uint16_t *q, int n_heads, float scale, float *out,
                      hipStream_t s) {
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
    per = ((per + TEAMS * TK - 1) / (TEAMS * TK)) * (TEAMS * TK);
    p.keys_per_split = per;
    p.n_splits = (int)((n_list + per - 1) / per);
    return run(p, s);
}

int launch_mla_prefill_v3(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                       const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s) {
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
    p.keys_per_split = ((pos0 + n + TEAMS * TK - 1) / (TEAMS * TK)) * (TEAMS * TK);
    return run(p, s);
}

}  // namespace cwick
