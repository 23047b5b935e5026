// gqa_prefill.hip -- causal GQA prefill on the bf16 matrix cores (the prefill
// branch of the reference's mixer_attn, src/q35_model.c:1713-1746: per head and
// per 128-query tile S = scale*Q*K^T over the rectangle, -1e30 tail, softmax,
// O = S*V).  Here: one pass, online softmax, the triangle only.
//
// MFMA-bound, and on this machine that means LDS-aware: a 32x32x16 MFMA takes
// 32 cycles and its A operand is 1 KiB, so four SIMDs that each fetch their own
// A fragments need the whole 128 B/clk of LDS.  Every wave therefore owns 64
// query rows (two 32-row column blocks) and uses each K / V^T fragment twice.
//
//   workgroup = 4 waves = 256 query rows that share one kv head: the GROUP
//   query heads of the kv head times P = 256/GROUP consecutive positions
//   (heads-as-M: K and V tiles are read once for all heads of the group).
//   Key tiles of TK = 32.  K and V go global -> LDS by global_load_lds_dwordx4
//   (no staging registers), one workgroup barrier per tile.
//   scores:  S^T[key][row] = K[key][dim] . Q^T[dim][row], v_mfma_f32_32x32x16_bf16,
//            K fragments from LDS, Q fragments of the first column block resident in
//            registers, those of the second re-read from a per-lane LDS park.
//            One query row per lane column: softmax statistics are per-lane.
//            The score accumulators are pinned to VGPRs (inline assembly): through the
//            builtin every MFMA result is placed in AGPRs, which the outputs fill.
//   values:  O^T[dim][row] += V^T[dim][key] . P^T[key][row].  P^T is the score
//            accumulator itself (rounded to bf16) -- its register layout is the
//            B-operand layout once the contraction slots are numbered to match;
//            V^T fragments come out of the V tile through the LDS transpose read
//            (ds_read_b64_tr_b16).  The 256 output registers live in AGPRs.
//   schedule: one wave per SIMD, so the loop is software-pipelined by hand, three
//            tiles deep: step t interleaves, MFMA by MFMA, the scores of tile t+2, the
//            softmax of tile t+1 (VALU, in the shadow of the matrix instructions) and
//            the value products of tile t.  The barrier that opens step t+1 sits near
//            the end of step t and the first fragments of step t+1 are fetched behind
//            it, so the matrix pipe does not drain between steps.  K is copied three
//            tiles ahead into two buffers, V two tiles ahead into three: a tile costs
//            about 1400 cycles of the CU's copy path, so the copies are spread over the
//            whole step and only K has to land within it.
//   The softmax reference of a row is the maximum of its first tile and stays
//   there while later scores exceed it by less than 64 (log2 units): weights up
//   to 2^64 lose nothing in bf16 or fp32.  A wave that meets a larger score
//   leaves the fast loop for a slow one that moves the reference and rescales
//   the accumulators (in place, in AGPRs) every tile.
//   Position blocks that see at most 1024 keys run the PRECISE variant (the
//   rounding residual of the weights goes through the matrix core too) in the
//   simpler two-stage schedule: scores of tile t+1, then its softmax next to
//   the value products of tile t.
//
//   LDS tile layout: 16 blocks of 1 KiB (+64 B pad), block b = 16-byte columns
//   2b and 2b+1 of all 32 keys, slot (c&1)*32 + (key ^ 8(c&1)).  A K fragment
//   read (ds_read_b128) covers one whole block; a transpose read touches four
//   64-byte segments that fall into different banks.
#include "common.hpp"

#include <mutex>

namespace cwick {

constexpr int PF_THREADS = 256;
constexpr int PF_TK = 32;
constexpr int PF_HD = 256;
constexpr int PF_ROWS = 256;                // query rows per workgroup
constexpr int PF_BLK = 1024 + 64;           // bytes between LDS blocks
constexpr int PF_TILE = 16 * PF_BLK;        // one K or V tile in LDS
constexpr int PF_PRE = 4;                   // k-steps of fragment prefetch in the score loop
constexpr int PF_QX0 = 0;                   // first k-step of column block B whose Q fragment is parked in LDS

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void pf_lds_void;

struct PfSmem {
    unsigned char k[2][PF_TILE];
    unsigned char v[3][PF_TILE];                // the pipelined body keeps three V tiles, the other two
    // Q fragments of column block B, k-steps PF_QX0..15, parked per lane: the register file
    // holds 256 accumulators + 64 Q registers + the working set, not 128 Q registers
    u32x4 qx[PF_THREADS / 64][16 - PF_QX0][64];
};

// workgroup barrier that orders LDS traffic only (the copies of later tiles stay in flight)
#define PF_LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

// PRECISE: the bf16 rounding residual of the weights goes through the matrix core as well
// (position blocks that see at most 1024 keys; see the launcher).  The body of one workgroup:
template <int GROUP, bool PRECISE>
__device__ __forceinline__ void
gqa_prefill_body(unsigned char *smem_raw, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
                 const uint16_t *__restrict__ Q, int64_t pos0, int64_t n, int n_kv_heads,
                 float scale_log2e, float *__restrict__ out, int64_t pblk, int kvh) {
    constexpr int P = PF_ROWS / GROUP;      // positions per workgroup
    PfSmem &sm = *reinterpret_cast<PfSmem *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int g = lane >> 5;                // 0/1

    const int64_t t0 = pblk * P;
    const int n_heads = n_kv_heads * GROUP;
    const int64_t kv_stride = (int64_t)n_kv_heads * PF_HD;
    const int64_t q_stride = (int64_t)n_heads * PF_HD;
    const int64_t n_keys_all = pos0 + n;

    // keys 0 .. last position of the block (clipped to the chunk)
    int64_t last_t = t0 + P - 1;
    if (last_t > n - 1) last_t = n - 1;
    const int64_t wg_keys = pos0 + last_t + 1;
    const int n_tiles = (int)((wg_keys + PF_TK - 1) / PF_TK);
    const int64_t first_masked_key = pos0 + t0;   // tiles ending at or below this need no mask
    constexpr bool precise = PRECISE;

    // ---- global -> LDS copies.  Wave w copies blocks 4w..4w+3 of a tile; lane l of a copy
    // lands in slot l of the block: column 2b + (l>>5), key (l&31) ^ 8(l>>5).
    const int cp_key = l32 ^ (g << 3);
    const uint16_t *Kg = K + (size_t)kvh * PF_HD + 8 * g;
    const uint16_t *Vg = V + (size_t)kvh * PF_HD + 8 * g;
    const uint32_t lds_k = (uint32_t)(uintptr_t)(pf_lds_void *)&sm.k[0][0];
    const uint32_t lds_v = (uint32_t)(uintptr_t)(pf_lds_void *)&sm.v[0][0];
    // (32-bit row arithmetic: at most 2^30 keys, and a row of at most 64 kv heads)
    const uint32_t last_key = (uint32_t)(n_keys_all - 1), kv_stride32 = (uint32_t)kv_stride;
    auto copy_src = [&](const uint16_t *base, int tile) -> const uint16_t * {
        uint32_t row = (uint32_t)tile * PF_TK + (uint32_t)cp_key;
        row = row < last_key ? row : last_key;                  // masked anyway
        return base + (uint64_t)row * kv_stride32 + 64 * wave;
    };
    // The 32 i bytes to the lane's source are the instruction's immediate offset (no address
    // arithmetic per copy); the hardware adds that offset to the LDS address as well, so M0 is
    // set 32 i bytes below the block.
    auto copy_one = [&](const uint16_t *src, uint32_t lds_tile, int i) {      // block 4 wave + i
        const uint32_t off = __builtin_amdgcn_readfirstlane(lds_tile + (uint32_t)((4 * wave + i) * PF_BLK - 32 * i));
        switch (i) {
            case 0: asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(off) : "memory"); break;
            case 1: asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:32" ::"v"(src), "s"(off) : "memory"); break;
            case 2: asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:64" ::"v"(src), "s"(off) : "memory"); break;
            default: asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:96" ::"v"(src), "s"(off) : "memory"); break;
        }
    };
    auto issue = [&](const uint16_t *base, uint32_t lds_tile, int tile) {
        const uint16_t *src = copy_src(base, tile);
#pragma unroll
        for (int i = 0; i < 4; i++) copy_one(src, lds_tile, i);
    };

    // The first tiles are requested before the query rows: one trip to memory for all of them
    // instead of one for Q, one for tile 0 and one for tile 1 (K has two buffers, V at least two).
    issue(Kg, lds_k, 0);
    issue(Vg, lds_v, 0);
    if (n_tiles > 1) {
        issue(Kg, lds_k + PF_TILE, 1);
        if (!precise) issue(Vg, lds_v + PF_TILE, 1);
    }

    // this lane's two query rows (column blocks A and B of the wave)
    int64_t t_row[2], my_limit[2];
    int j_row[2];
    bool row_live[2];
    bf16x8 qf[2][16];                       // B operand: lane (row, g) holds dims 16ks+8g .. +8
                                            // (qf[1][PF_QX0..15] only pass through, see PfSmem::qx)
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int r = wave * 64 + 32 * c + l32;
        j_row[c] = r / P;
        t_row[c] = t0 + (r % P);
        row_live[c] = t_row[c] < n;
        const int64_t tq = row_live[c] ? t_row[c] : n - 1;
        my_limit[c] = pos0 + tq;
        const uint16_t *qrow = Q + tq * q_stride + (size_t)(kvh * GROUP + j_row[c]) * PF_HD + 8 * g;
#pragma unroll
        for (int ks = 0; ks < 16; ks++)
            qf[c][ks] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + 16 * ks));
    }
#pragma unroll
    for (int ks = PF_QX0; ks < 16; ks++) sm.qx[wave][ks - PF_QX0][lane] = __builtin_bit_cast(u32x4, qf[1][ks]);

    // K fragment of k-step ks: block ks, slot 32g + (l32 ^ 8g)
    const uint32_t kfrag_off = (uint32_t)((32 * g + (l32 ^ (g << 3))) * 16);
    // transpose read (ds_read_b64_tr_b16): within a 16-lane group, lane i addresses key (i/4),
    // dims 4*(i%4)..+4 of a 4-key x 16-dim patch and receives dim i for the 4 keys.
    // For output block db: dims 32db + 16(grp&1) + 4(gi&3): column c = 4db + 2(grp&1) + ((gi&3)>>1)
    const int grp = lane >> 4, gi = lane & 15;
    const int v_col = (gi & 3) >> 1;                              // parity of the 16-byte column
    const int v_key0 = 4 * (grp >> 1) + (gi >> 2);                // + 16 ks2 (+8 for the second half)
    auto vfrag_off = [&](int key) -> uint32_t {
        return (uint32_t)((grp & 1) * PF_BLK + (v_col * 32 + (key ^ (v_col << 3))) * 16 + (gi & 1) * 8);
    };
    uint32_t v_off[2][2];
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ks2++) {
        v_off[ks2][0] = vfrag_off(16 * ks2 + v_key0);
        v_off[ks2][1] = vfrag_off(16 * ks2 + v_key0 + 8);
    }

    f32x16 oacc[2][8];
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
        for (int db = 0; db < 8; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) oacc[c][db][i] = 0.0f;
    float m_ref[2] = {-INFINITY, -INFINITY}, l_part[2] = {0.0f, 0.0f};

    // scores of one tile for both column blocks
    // One wave per SIMD: nothing hides an LDS round trip, so the fragments are fetched PF_PRE
    // k-steps ahead of the MFMAs that use them.
    // Score MFMA with its accumulator pinned to VGPRs: through the builtin the allocator places
    // every MFMA result in AGPRs, which the 256 output accumulators fill, and moves registers
    // back and forth every tile.  Opaque to the compiler's hazard tracking: score_done() goes
    // between the last MFMA and the first VALU read of the result.
    auto score_mfma = [&](f32x16 &acc, bf16x8 a, bf16x8 b, bool first) {
        if (first) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
    };
    auto score_done = [&]() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); };
    // ck / cv >= 0: the copies of K(ck) and V(cv) are issued between the MFMAs (an LDS-DMA
    // instruction occupies the issue slot for about as long as two MFMAs run).  Tile u of K or V
    // lives in buffer u & 1.
    auto scores = [&](int tile, f32x16 (&s)[2], int ck, int cv) {
        const unsigned char *kb = &sm.k[tile & 1][0] + kfrag_off;
        const u32x4 *qb = &sm.qx[wave][0][lane];
        u32x4 ka[PF_PRE], qa[PF_PRE];
#pragma unroll
        for (int ks = 0; ks < PF_PRE; ks++) {
            ka[ks] = *(const u32x4 *)(kb + ks * PF_BLK);
            if (ks >= PF_QX0) qa[ks] = qb[(ks - PF_QX0) * 64];
        }
        const bool do_k = ck >= 0 && ck < n_tiles, do_v = cv >= 0 && cv < n_tiles;
        const uint16_t *src_k = copy_src(Kg, do_k ? ck : 0);
        const uint16_t *src_v = copy_src(Vg, do_v ? cv : 0);
        const uint32_t dst_k = lds_k + (uint32_t)((ck & 1) * PF_TILE);
        const uint32_t dst_v = lds_v + (uint32_t)((cv & 1) * PF_TILE);
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            const bf16x8 kf = __builtin_bit_cast(bf16x8, ka[ks % PF_PRE]);
            const bf16x8 q1 = ks < PF_QX0 ? qf[1][ks] : __builtin_bit_cast(bf16x8, qa[ks % PF_PRE]);
            if (ks + PF_PRE < 16) {
                ka[ks % PF_PRE] = *(const u32x4 *)(kb + (ks + PF_PRE) * PF_BLK);
                if (ks + PF_PRE >= PF_QX0) qa[ks % PF_PRE] = qb[(ks + PF_PRE - PF_QX0) * 64];
            }
            score_mfma(s[0], kf, qf[0][ks], ks == 0);
            score_mfma(s[1], kf, q1, ks == 0);
            if ((ks & 1) == 0) {
                if (ks < 8) { if (do_k) copy_one(src_k, dst_k, ks >> 1); }
                else if (do_v) copy_one(src_v, dst_v, (ks - 8) >> 1);
            }
        }
        score_done();
    };
    // the same from global memory (the slow loop of the pipelined body: its K tile has already
    // been overwritten in LDS)
    auto scores_global = [&](int tile, f32x16 (&s)[2]) {
        int64_t row = (int64_t)tile * PF_TK + l32;
        if (row > n_keys_all - 1) row = n_keys_all - 1;             // masked anyway
        const uint16_t *kr = K + row * kv_stride + (size_t)kvh * PF_HD + 8 * g;
        const u32x4 *qb = &sm.qx[wave][0][lane];
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            const bf16x8 kf = __builtin_bit_cast(bf16x8, *(const u32x4 *)(kr + 16 * ks));
            const bf16x8 q1 = ks < PF_QX0 ? qf[1][ks] : __builtin_bit_cast(bf16x8, qb[(ks - PF_QX0) * 64]);
            score_mfma(s[0], kf, qf[0][ks], ks == 0);
            score_mfma(s[1], kf, q1, ks == 0);
        }
        score_done();
    };
    // softmax bookkeeping of one tile and column block, in two parts.
    // register i holds key (i/4)*8 + 4g + i%4 of the tile for this lane's row.
    // sm_prep: mask the raw scores, return this lane's maximum in log2 units.
    auto sm_prep = [&](int tile, int c, f32x16 &s) -> float {
        const int64_t key0 = (int64_t)tile * PF_TK;
        float tmax = -INFINITY;
        if (key0 + PF_TK - 1 > first_masked_key) {          // workgroup-uniform: a tile on the diagonal
            // position (i/4)*8 + i%4 + 4g of the tile is visible up to lim
            int64_t lim64 = my_limit[c] - key0 - 4 * g;
            const int lim = lim64 > 64 ? 64 : (lim64 < -1 ? -1 : (int)lim64);
#pragma unroll
            for (int i = 0; i < 16; i++)
                if ((i >> 2) * 8 + (i & 3) > lim) s[i] = -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[i]);
        return tmax * scale_log2e;                           // the scale is positive: max commutes
    };
    // sm_finish: raw scores -> bf16 weights (and their rounding residual) against m_ref.
    auto sm_finish = [&](int c, f32x16 &s, u32x4 (&pw)[2], u32x4 (&pl)[2]) {
        const float m_use = m_ref[c] == -INFINITY ? 0.0f : m_ref[c];
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            s[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], scale_log2e, -m_use));   // masked: 0
            if (precise) psum += s[i];
        }
        // contraction slot (g, jj) of step ks2 <-> tile key 16*ks2 + (jj/4)*8 + 4g + jj%4,
        // i.e. score register 8*ks2 + jj: P^T needs no data movement.
        // With single-term weights the row sum is the sum of the ROUNDED weights: the output is
        // then a convex combination of value rows whatever the rounding did (a row dominated by
        // one key is exact), and the error is 2^-9 of the spread of the values, not of their size.
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ks2++)
#pragma unroll
            for (int h = 0; h < 4; h++) {
                pw[ks2][h] = pack_bf16_rne(s[8 * ks2 + 2 * h], s[8 * ks2 + 2 * h + 1]);
                if (precise)
                    pl[ks2][h] = pack_bf16_rne(s[8 * ks2 + 2 * h] - bf16lo_to_f32(pw[ks2][h]),
                                               s[8 * ks2 + 2 * h + 1] - bf16hi_to_f32(pw[ks2][h]));
                else
                    psum = pair_sum_bf16(pw[ks2][h], psum);
            }
        l_part[c] += psum;
    };
    // The running reference m_ref is the row maximum of tile 0 and stays there while later tiles
    // exceed it by less than 2^SLACK: weights up to 2^SLACK are as exact in bf16 and fp32 as
    // weights up to 1.  The slow loop moves it (and rescales) when a tile beats it by 2^8.
    constexpr float SLACK = 64.0f;
    auto sm_move_ref = [&](int c, float tmax) -> float {
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        float corr = 1.0f;
        if (tmax > m_ref[c] + 8.0f) {
            corr = __builtin_amdgcn_exp2f(m_ref[c] - tmax);              // first tile: exp2(-inf) = 0
            m_ref[c] = tmax;
            l_part[c] *= corr;
        }
        return corr;
    };
    // value MFMAs of one tile for both column blocks
    auto values = [&](int tile, const u32x4 (&pw)[2][2], const u32x4 (&pl)[2][2]) {
        const unsigned char *vb = &sm.v[PRECISE ? (tile & 1) : (tile % 3)][0];
        // step st = 8 ks2 + db; its two transpose reads are issued PF_PRE steps ahead
        s16x4 lo[PF_PRE], hi[PF_PRE];
        auto fetch = [&](int st, int slot) {
            const int ks2 = st >> 3, db = st & 7;
            lo[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(vb + v_off[ks2][0] + db * (2 * PF_BLK)));
            hi[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(vb + v_off[ks2][1] + db * (2 * PF_BLK)));
        };
#pragma unroll
        for (int st = 0; st < PF_PRE; st++) fetch(st, st);
#pragma unroll
        for (int st = 0; st < 16; st++) {
            const int ks2 = st >> 3, db = st & 7;
            typedef __attribute__((ext_vector_type(8))) short s16x8;
            const bf16x8 va = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo[st % PF_PRE], hi[st % PF_PRE], 0, 1, 2, 3, 4, 5, 6, 7));
            if (st + PF_PRE < 16) fetch(st + PF_PRE, st % PF_PRE);
#pragma unroll
            for (int c = 0; c < 2; c++) {
                oacc[c][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, __builtin_bit_cast(bf16x8, pw[c][ks2]), oacc[c][db], 0, 0, 0);
                if (precise)
                    oacc[c][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, __builtin_bit_cast(bf16x8, pl[c][ks2]), oacc[c][db], 0, 0, 0);
            }
        }
    };
    // The accumulators live in AGPRs.  Written as ordinary arithmetic a rescale makes the
    // compiler move them to VGPRs for the whole loop (and spill), and so does a rescale under a
    // condition; so the fast loop has none, and the slow loop scales every tile, in place.
    auto rescale = [&](const float (&corr)[2]) {
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int db = 0; db < 8; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    float tmp;
                    asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\t"
                                 "v_accvgpr_write_b32 %0, %1"
                                 : "+a"(oacc[c][db][i]), "=&v"(tmp)
                                 : "v"(corr[c]));
                }
    };
    // top of step t: the tiles step t reads have landed (this wave's part, then everyone's), and
    // all reads of step t-1 are over, so the copies of step t may overwrite its buffers
    auto step_top = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PF_LDS_BARRIER();
    };

    if constexpr (PRECISE) {
        // ---- prologue: K(0), V(0), K(1) are on their way; scores and softmax of tile 0 (sets the reference) ----
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PF_LDS_BARRIER();

        u32x4 pw[2][2], pl[2][2];
        {
            f32x16 s[2];
            scores(0, s, -1, -1);
#pragma unroll
            for (int c = 0; c < 2; c++) {
                (void)sm_move_ref(c, sm_prep(0, c, s[c]));                  // nothing accumulated yet
                sm_finish(c, s[c], pw[c], pl[c]);
            }
        }

        // ---- fast loop: scores(t+1); then softmax(t+1) beside values(t); no rescale.  The softmax
        // is speculative: whether a row outgrew the reference is looked at after the MFMAs.
        int t = 0;
        bool slow = false;
        for (; t + 1 < n_tiles; t++) {
            step_top();
            f32x16 s[2];
            scores(t + 1, s, t + 2, t + 1);
            u32x4 pwn[2][2], pln[2][2];
            const float l_save[2] = {l_part[0], l_part[1]};
            const float x0 = sm_prep(t + 1, 0, s[0]), x1 = sm_prep(t + 1, 1, s[1]);
            sm_finish(0, s[0], pwn[0], pln[0]);
            sm_finish(1, s[1], pwn[1], pln[1]);
            values(t, pw, pl);
            if (__any(x0 > m_ref[0] + SLACK || x1 > m_ref[1] + SLACK)) {   // a row outgrew the reference
                l_part[0] = l_save[0];
                l_part[1] = l_save[1];
                slow = true;
                break;
            }
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int k2 = 0; k2 < 2; k2++) {
                    pw[c][k2] = pwn[c][k2];
                    pl[c][k2] = pln[c][k2];
                }
        }
        // ---- slow loop (rare): the reference follows the maximum, accumulators rescaled every tile.
        // It resumes step t after its top, copies and values(t); the scores are recomputed.
        if (slow) {
            bool resumed = true;
            for (; t + 1 < n_tiles; t++) {
                if (!resumed) step_top();
                f32x16 s[2];
                scores(t + 1, s, resumed ? -1 : t + 2, resumed ? -1 : t + 1);
                u32x4 pwn[2][2], pln[2][2];
                float corr[2];
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    corr[c] = sm_move_ref(c, sm_prep(t + 1, c, s[c]));
                    sm_finish(c, s[c], pwn[c], pln[c]);
                }
                if (!resumed) values(t, pw, pl);
                resumed = false;
                rescale(corr);
#pragma unroll
                for (int c = 0; c < 2; c++)
#pragma unroll
                    for (int k2 = 0; k2 < 2; k2++) {
                        pw[c][k2] = pwn[c][k2];
                        pl[c][k2] = pln[c][k2];
                    }
            }
        }
        // ---- last tile's values ----
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PF_LDS_BARRIER();
        values(n_tiles - 1, pw, pl);

    } else {
        // ---- pipelined body: step t computes the scores of tile t+2, the softmax of tile t+1 and the
        // value products of tile t, interleaved MFMA by MFMA so that the softmax (VALU), the fragment
        // reads (LDS) and the copies issue in the shadow of the matrix instructions.  The loop is
        // rotated: the barrier that opens step t+1 sits in slot 14 of step t (by then every
        // fragment read of step t has returned and the copies issued in slots 0..7 have landed), and
        // slots 14 and 15 already fetch the first fragments of step t+1, so the matrix pipe does not
        // drain between steps.  Only tiles below the diagonal take this form; the (at most three)
        // tiles on it and the tail run in sequence.
        constexpr float BIG = 18446744073709551616.0f;                  // 2^SLACK
        u32x4 ka[2], qa[2];                                             // fragments of the next two slots
        s16x4 lo[2], hi[2];
        // V(t) lives in buffer t mod 3, carried along as t3 (no division in the loop)
        auto next3 = [](int x) -> int { return x == 2 ? 0 : x + 1; };
        int t3 = 0;
        auto fetch = [&](int t, int t3, int i, int slot) {              // fragments of slot i of step t
            const unsigned char *kb = &sm.k[t & 1][0] + kfrag_off;      // K(t+2)
            const unsigned char *vb = &sm.v[t3][0];                     // V(t)
            ka[slot] = *(const u32x4 *)(kb + i * PF_BLK);
            if (i >= PF_QX0) qa[slot] = sm.qx[wave][i - PF_QX0][lane];
            const int ks2 = i >> 3, db = i & 7;
            lo[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(vb + v_off[ks2][0] + db * (2 * PF_BLK)));
            hi[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(vb + v_off[ks2][1] + db * (2 * PF_BLK)));
        };
        // the running sums as opaque instructions: left to the compiler, the thirty-two additions
        // of a step sink to its end, a dependent chain behind the last MFMA
        // (one dot-product instruction per packed pair: acc += lo * 1 + hi * 1)
        const uint32_t ones_bf16 = 0x3F803F80u;
        auto psum_pair = [&](float &acc, uint32_t w) { asm volatile("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(acc) : "s"(ones_bf16), "v"(w)); };
        auto pstep = [&](int t, int t3, f32x16 (&sc)[2], f32x16 (&sn)[2], const u32x4 (&pc)[2][2],
                         u32x4 (&pn)[2][2], float (&ps)[2]) {
            const int t3n = next3(t3);
            const uint16_t *src_k = nullptr, *src_v = nullptr;
            uint32_t dst_k = 0, dst_v = 0;
            const float mu0 = m_ref[0], mu1 = m_ref[1];
            float p0 = 0.0f, p1 = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                typedef __attribute__((ext_vector_type(8))) short s16x8;
                const int ks2 = i >> 3, db = i & 7;
                const bf16x8 kf = __builtin_bit_cast(bf16x8, ka[i & 1]);
                const bf16x8 q1 = i < PF_QX0 ? qf[1][i] : __builtin_bit_cast(bf16x8, qa[i & 1]);
                const bf16x8 va = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo[i & 1], hi[i & 1], 0, 1, 2, 3, 4, 5, 6, 7));
                score_mfma(sn[0], kf, qf[0][i], i == 0);
                sc[0][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[0][i], scale_log2e, -mu0));
                if (i == 0) {
                    // where this step's copies come from and go to, worked out behind the
                    // first MFMA (past the last tile: clipped rows into a dead buffer)
                    src_k = copy_src(Kg, t + 3);
                    src_v = copy_src(Vg, t + 2);
                    dst_k = lds_k + (uint32_t)(((t + 1) & 1) * PF_TILE);
                    dst_v = lds_v + (uint32_t)(next3(t3n) * PF_TILE);
                }
                __builtin_amdgcn_sched_barrier(0);
                oacc[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, __builtin_bit_cast(bf16x8, pc[0][ks2]), oacc[0][db], 0, 0, 0);
                sc[1][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[1][i], scale_log2e, -mu1));
                __builtin_amdgcn_sched_barrier(0);
                score_mfma(sn[1], kf, q1, i == 0);
                if (i == 14) {                                       // the top of step t+1
                    // all but this step's three V copies: K(t+3) and V(t+1) have landed
                    asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
                    PF_LDS_BARRIER();
                }
                if (i < 14) fetch(t, t3, i + 2, i & 1);
                else fetch(t + 1, t3n, i - 14, i & 1);
                __builtin_amdgcn_sched_barrier(0);
                oacc[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, __builtin_bit_cast(bf16x8, pc[1][ks2]), oacc[1][db], 0, 0, 0);
                if (i & 1) {                                         // weights, and the sum of the rounded weights
                    const uint32_t w0 = pack_bf16_rne(sc[0][i - 1], sc[0][i]);
                    const uint32_t w1 = pack_bf16_rne(sc[1][i - 1], sc[1][i]);
                    pn[0][ks2][(i & 7) >> 1] = w0;
                    pn[1][ks2][(i & 7) >> 1] = w1;
                    psum_pair(p0, w0);
                    psum_pair(p1, w1);
                }
                if (!(i & 1)) {
                    if (i < 8) copy_one(src_k, dst_k, i >> 1);
                    else copy_one(src_v, dst_v, (i - 8) >> 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            ps[0] = p0;
            ps[1] = p1;
        };
        auto issue_copies = [&](int t) {                                 // what step t fetches
            if (t + 3 < n_tiles) issue(Kg, lds_k + (uint32_t)(((t + 3) & 1) * PF_TILE), t + 3);
            if (t + 2 < n_tiles) issue(Vg, lds_v + (uint32_t)(((t + 2) % 3) * PF_TILE), t + 2);
        };

        // prologue (K(0), V(0), K(1), V(1) are on their way), K(2); scores and softmax of tile 0 (sets the reference),
        // scores of tile 1.  From then on step t fetches K(t+3) and V(t+2).
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // K(0), V(0), K(1), V(1)
        PF_LDS_BARRIER();
        u32x4 pa[2][2], pb[2][2], pl[2][2];
        f32x16 sa[2], sb[2];
        scores(0, sa, -1, -1);
#pragma unroll
        for (int c = 0; c < 2; c++) {
            (void)sm_move_ref(c, sm_prep(0, c, sa[c]));                     // nothing accumulated yet
            sm_finish(c, sa[c], pa[c], pl[c]);
        }
        if (n_tiles > 1) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            PF_LDS_BARRIER();
            if (n_tiles > 2) issue(Kg, lds_k, 2);
            scores(1, sa, -1, -1);
        }
        // now: sa = raw scores of tile t+1, pa = weights of tile t, for t = 0
        const int d0 = (int)((first_masked_key + 1) / PF_TK);            // tiles 0 .. d0-1 need no mask
        int t = 0;
        bool slow = false;
        bool top_done = false;                                           // the top of step t has been passed already
        auto more = [&]() -> bool { return t + 1 < d0 && t + 2 < n_tiles; };
        if (more()) {
            step_top();
            fetch(0, 0, 0, 0);
            fetch(0, 0, 1, 1);
            top_done = true;
            for (;;) {
                float ps[2];
                pstep(t, t3, sa, sb, pa, pb, ps);
                if (__any(ps[0] > BIG || ps[1] > BIG)) { slow = true; break; }
                l_part[0] += ps[0];
                l_part[1] += ps[1];
                t++;
                t3 = next3(t3);
                if (!more()) {
#pragma unroll
                    for (int c = 0; c < 2; c++) {
                        sa[c] = sb[c];
                        pa[c][0] = pb[c][0];
                        pa[c][1] = pb[c][1];
                    }
                    break;
                }
                pstep(t, t3, sb, sa, pb, pa, ps);
                if (__any(ps[0] > BIG || ps[1] > BIG)) { slow = true; break; }
                l_part[0] += ps[0];
                l_part[1] += ps[1];
                t++;
                t3 = next3(t3);
                if (!more()) break;
            }
            score_done();
        }
        // the tiles on the diagonal and the tail, in sequence
        if (!slow)
            for (; t < n_tiles; t++) {
                if (!top_done) step_top();
                top_done = false;
                issue_copies(t);
                bool bad = false;
                const float l_save[2] = {l_part[0], l_part[1]};
                if (t + 1 < n_tiles) {
                    const float x0 = sm_prep(t + 1, 0, sa[0]), x1 = sm_prep(t + 1, 1, sa[1]);
                    sm_finish(0, sa[0], pb[0], pl[0]);
                    sm_finish(1, sa[1], pb[1], pl[1]);
                    bad = __any(x0 > m_ref[0] + SLACK || x1 > m_ref[1] + SLACK);
                }
                values(t, pa, pl);
                if (bad) {
                    l_part[0] = l_save[0];
                    l_part[1] = l_save[1];
                    slow = true;
                    break;
                }
                if (t + 2 < n_tiles) scores(t + 2, sa, -1, -1);
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    pa[c][0] = pb[c][0];
                    pa[c][1] = pb[c][1];
                }
            }
        // slow loop (rare): entered after the top, the copies and the value products of step t; the
        // reference follows the maximum and the accumulators are rescaled every tile
        if (slow) {
            bool resumed = true;
            for (; t + 1 < n_tiles; t++) {
                if (!resumed) {
                    if (!top_done) step_top();
                    top_done = false;
                    issue_copies(t);
                }
                f32x16 s[2];
                scores_global(t + 1, s);
                float corr[2];
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    corr[c] = sm_move_ref(c, sm_prep(t + 1, c, s[c]));
                    sm_finish(c, s[c], pb[c], pl[c]);
                }
                if (!resumed) values(t, pa, pl);
                resumed = false;
                rescale(corr);
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    pa[c][0] = pb[c][0];
                    pa[c][1] = pb[c][1];
                }
            }
            if (!top_done) step_top();
            values(n_tiles - 1, pa, pl);
        }
    }

    // ---- epilogue ----
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const float l = l_part[c] + __shfl_xor(l_part[c], 32, 64);
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        if (row_live[c]) {
            float *o = out + t_row[c] * q_stride + (size_t)(kvh * GROUP + j_row[c]) * PF_HD + 4 * g;
#pragma unroll
            for (int db = 0; db < 8; db++)
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++) {
                    f32x4 w;
#pragma unroll
                    for (int i = 0; i < 4; i++) w[i] = oacc[c][db][4 * b4 + i] * inv;
                    *(f32x4 *)(o + 32 * db + 8 * b4) = w;
                }
        }
    }
}

// One launch: position blocks below n_prec take the PRECISE body.
template <int GROUP>
__global__ void __launch_bounds__(PF_THREADS, 1)
gqa_prefill_kernel(const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
                   const uint16_t *__restrict__ Q, int64_t pos0, int64_t n, int n_kv_heads,
                   float scale_log2e, float *__restrict__ out, int64_t n_prec, int64_t pblocks,
                   uint32_t *__restrict__ tickets) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    __shared__ uint32_t sh_item;
    // One workgroup per compute unit stays for the whole launch and draws its (position block,
    // kv head) items from a counter: a compute unit that the dispatcher would leave empty for
    // 4 to 30 us between two workgroups goes on at once, and XCDs that run slower than the others
    // (two of the eight took 6 % longer for the same share) simply draw fewer items.  Items are
    // handed out from the most expensive position block to the cheapest (the last ones to start
    // must be the short ones).  A block costs its number of key tiles, and 1.6 times that in the
    // PRECISE variant: rank r = item / n_kv_heads in the merge of the two descending sequences
    // 10 (p+1), p >= n_prec, and 16 (p+1), p < n_prec.
    // The first item of a workgroup is its own index, without a ticket: read-modify-writes of one
    // address from all XCDs are served one after the other (about 0.15 us each), so a first
    // draw by every workgroup at once would start the last of them tens of microseconds late.
    // Later draws come one by one as the items end.
    const uint32_t total = (uint32_t)(pblocks * n_kv_heads);
    uint32_t item = blockIdx.x;
    for (;;) {
        if (item >= total) break;
        const int64_t rank = (int64_t)item / n_kv_heads;
        const int kvh = (int)(item % (uint32_t)n_kv_heads);
        int64_t pblk = -1, before = 0;                  // precise blocks ranked before this one
        for (int64_t pp = n_prec - 1; pp >= 0; pp--) {
            int64_t qmin = 16 * (pp + 1) / 10;          // plain blocks q >= qmin cost more than precise block pp
            if (qmin < n_prec) qmin = n_prec;
            const int64_t rk = (qmin < pblocks ? pblocks - qmin : 0) + (n_prec - 1 - pp);
            if (rk == rank) pblk = pp;
            if (rk < rank) before++;
        }
        if (pblk < 0) pblk = pblocks - 1 - (rank - before);
        if (pblk < n_prec) gqa_prefill_body<GROUP, true>(smem_raw, K, V, Q, pos0, n, n_kv_heads, scale_log2e, out, pblk, kvh);
        else gqa_prefill_body<GROUP, false>(smem_raw, K, V, Q, pos0, n, n_kv_heads, scale_log2e, out, pblk, kvh);
        // nothing of the last item may still be on its way into LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (threadIdx.x == 0) sh_item = gridDim.x + atomicAdd(&tickets[0], 1u);
        __syncthreads();
        item = sh_item;
        __syncthreads();                                 // everybody has the item, and is done with the last one's LDS
    }
    // the last workgroup to leave puts the counters back to zero for the next launch (every
    // workgroup has drawn its last ticket before it counts itself out)
    if (threadIdx.x == 0) {
        const uint32_t gone = atomicAdd(&tickets[1], 1u);
        if (gone == gridDim.x - 1) {
            __hip_atomic_store(&tickets[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&tickets[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// rows that see at most this many keys take the two-term-weight variant
static int64_t gqa_precise_keys() {
    static const int64_t v = [] {
        const char *e = getenv("CWICK_HIP_GQA_PRECISE_KEYS");
        const int64_t x = e ? atoll(e) : 1024;
        return x < 0 ? (int64_t)0 : x;
    }();
    return v;
}

template <int GROUP>
static int run_gqa_prefill(const uint16_t *k, const uint16_t *v, int64_t pos0, int64_t n,
                           int n_kv_heads, const uint16_t *q, float scale, float *out,
                           hipStream_t s) {
    static std::once_flag attr_once;
    static hipError_t attr_err = hipSuccess;
    const size_t smem = sizeof(PfSmem);
    std::call_once(attr_once, [&] {
        attr_err = hipFuncSetAttribute((const void *)gqa_prefill_kernel<GROUP>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    });
    CWICK_HIP_CALL(attr_err);
    constexpr int P = PF_ROWS / GROUP;
    const int64_t pblocks = (n + P - 1) / P;
    CWICK_REQUIRE(pblocks * n_kv_heads <= 0x7FFFFFFF, "gqa_prefill: grid too large");
    // Short prefixes: few keys carry the whole weight, so the 2^-9 rounding of each bf16 weight
    // shows in an O(1) output.  Position blocks that see at most 1024 keys run the variant that
    // also feeds the rounding residual through the matrix core (weights good to 2^-17).
    int64_t n_prec = 0;
    while (n_prec < pblocks) {
        int64_t last_t = (n_prec + 1) * P - 1;
        if (last_t > n - 1) last_t = n - 1;
        if (pos0 + last_t + 1 > gqa_precise_keys()) break;
        n_prec++;
    }
    uint32_t *tickets = ticket_counters(s);
    if (!tickets) return 0;                 // ticket_counters() has recorded why
    const int64_t items = pblocks * n_kv_heads;
    const int64_t wgs = items < num_cus() ? items : num_cus();      // the LDS of a compute unit holds one workgroup
    {
        ProfKernel pk(CWICK_HIP_PROF_GQA_PREFILL, s);
        pk.launch(gqa_prefill_kernel<GROUP>, dim3((unsigned)wgs), dim3(PF_THREADS), smem,
                  k, v, q, pos0, n, n_kv_heads, scale * 1.44269504088896340736f, out, n_prec, pblocks, tickets);
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
