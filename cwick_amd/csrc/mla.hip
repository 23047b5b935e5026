// mla.hip -- absorbed-latent MLA over the FP8 latent cache: the two reductions
// of the reference's mla_latent_decode (src/attention.c:749-811) as one
// flash-attention pass on the bf16 matrix cores.
//
//     scores[h][i] = (q_abs[h] . c[sel[i]]) * scale          K = all 576 dims
//     p            = softmax_i(scores[h])
//     c_acc[h]     = sum_i p[h][i] * c[sel[i]][0..512)        V = first 512 dims
//
// c[t][d] = e4m3(rows[t][d]) * scales[t][d/128].  Every E4M3 value is exact in
// bf16 and in fp16, so the bytes are widened without the scale.  Scores: bf16
// MFMA (the query is bf16), the fp32 block scale multiplies the fp32 partial
// dot of its 128-dim block.  Values: fp16 MFMA, the block scale is folded into
// the softmax weight before that is rounded to fp16 (11-bit significand).
//
// Work decomposition
//   workgroup = 256 threads = 4 waves, 32 query rows (heads of one query) x
//   one slice of keys; tiles of TK = 64 keys.
//   scores:  S^T[key][head] = K[key][dim] . Q^T[dim][head] with
//            v_mfma_f32_16x16x32_bf16.  Wave w owns keys 16w..16w+15 of the
//            tile and takes its K fragments straight from global memory (each
//            key row is needed by exactly one wave), Q fragments live in
//            registers for the whole kernel.  The result lands with one head
//            per lane column, so softmax statistics are per-lane scalars.
//   values:  O^T[dim][head] += V^T[dim][key] . P^T[key][head].  Wave w owns
//            dims 128w..128w+127 -- exactly one scale block, so the weights it
//            reads are p * scales[key][w].  V^T comes from LDS, where the tile
//            was written transposed ([dim][key], bf16) by all 256 threads; P
//            goes through LDS in four pre-scaled copies.
//   decode:  the key range is split over workgroups (flash-decoding); each
//            writes un-normalised (m, l, acc) partials and a merge kernel
//            combines them.  prefill: one workgroup walks the whole causal
//            prefix of its query and writes the normalised output.
#include "common.hpp"
#include "merge.hpp"

namespace cwick {

constexpr int KDIM = CWICK_HIP_LATENT_KDIM;   // 576
constexpr int VDIM = CWICK_HIP_LATENT_VDIM;   // 512
constexpr int NBLK = CWICK_HIP_LATENT_NBLK;   // 5
constexpr int MLA_THREADS = 256;
constexpr int TK = 64;                        // keys per tile
constexpr int ROWS = 32;                      // query rows (heads) per workgroup
constexpr int VT_STRIDE = TK + 8;             // bf16 elements per V^T row (16 B pad)
constexpr int PS_STRIDE = TK + 8;

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

struct MlaParams {
    const uint8_t *rows;      // [.][n_rows][576]
    const float *scales;      // [.][n_rows][5]
    int64_t row_bstride;      // bytes between queries' caches (0: shared)
    int64_t scale_bstride;    // floats
    int64_t n_rows;           // valid rows per cache
    const int32_t *sel;       // [nq][n_list] or null
    int64_t n_list;           // keys of query 0
    int64_t list_step;        // keys of query y = n_list + y*list_step (prefill: 1)
    const uint16_t *q;        // [nq][nh][576] bf16
    int nh;
    int nq;
    float scale;
    int n_splits;
    int64_t keys_per_split;   // multiple of TK
    float *out;               // [nq][nh][512]          (n_splits == 1)
    float *part_acc;          // [nq][n_splits][nh][512] (n_splits > 1)
    float *part_ml;           // [nq][n_splits][nh][2]
};

struct MlaSmem {
    uint16_t vt[VDIM][VT_STRIDE];          // V^T tile, bf16
    uint16_t ps[4][ROWS][PS_STRIDE];       // p * scales[key][blk], bf16, blk = 0..3
    float sc[TK][NBLK + 1];                // scales[key][blk] (0 for masked keys); [5] pads
    int32_t rowid[TK];                     // cache row of each tile key, -1 = masked
    float wmax[4][ROWS];                   // per-wave tile maxima
    float wsum[4][ROWS];                   // per-wave row sums (epilogue)
    uint32_t scmax_bits;                   // largest value scale of the tile, as bits
};

__global__ void __launch_bounds__(MLA_THREADS, 1) mla_fwd_kernel(const MlaParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    MlaSmem &sm = *reinterpret_cast<MlaSmem *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l16 = lane & 15;
    const int g = lane >> 4;               // 0..3

    // ---- which (head block, query, split) is this workgroup? ----
    // Linear ids go round-robin over the 8 XCDs; renumber so that consecutive
    // work units (the head blocks of one key slice) share an XCD and its L2.
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

    // ---- Q fragments: 2 head blocks x 18 k-steps, kept for the whole kernel ----
    // k-step pair j covers dims 64j..64j+63; lane group g holds dims
    // 64j+16g..+16: the first 8 feed step 2j, the next 8 step 2j+1.  The K
    // fragments below use the same assignment (the contraction index may be
    // permuted freely as long as both operands agree).
    bf16x8 qf[2][18];
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) {
        int head = hb * ROWS + h2 * 16 + l16;
        if (head >= p.nh) head = p.nh - 1;
        const uint16_t *qrow = p.q + ((size_t)y * p.nh + head) * KDIM;
#pragma unroll
        for (int j = 0; j < 9; j++) {
            const u32x4 a = *(const u32x4 *)(qrow + 64 * j + 16 * g);
            const u32x4 b = *(const u32x4 *)(qrow + 64 * j + 16 * g + 8);
            qf[h2][2 * j] = __builtin_bit_cast(bf16x8, a);
            qf[h2][2 * j + 1] = __builtin_bit_cast(bf16x8, b);
        }
    }

    f32x4 oacc[8][2];
#pragma unroll
    for (int db = 0; db < 8; db++)
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) oacc[db][h2] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run[2] = {-INFINITY, -INFINITY};
    float l_part[2] = {0.f, 0.f};
    // The value weights p*scale go through the matrix core as fp16 (11-bit
    // significand; bf16's 8 bits would cost 2^-9 of the output whenever one key
    // dominates).  They are kept inside fp16's normal range by a power-of-two
    // normaliser: e_run is the largest binary exponent of any value scale seen so
    // far (scale * 2^-e_run < 1), weights are multiplied by 2^(14 - e_run), the
    // accumulator is in those units and is shifted (exactly) when e_run grows.
    constexpr int E_NONE = -1000;
    int e_run = E_NONE;

    for (int64_t t0 = k_begin; t0 < k_end; t0 += TK) {
        // ---- tile bookkeeping: cache row and scales of each key ----
        if (tid < TK) {
            const int64_t i = t0 + tid;
            int64_t r = -1;
            if (i < k_end) {
                r = sel ? (int64_t)sel[i] : i;
                if (r < 0 || r >= p.n_rows) r = -1;
            }
            sm.rowid[tid] = (int32_t)r;
            if (tid == 0) sm.scmax_bits = 0u;
        }
        __syncthreads();   // also: everyone is done with the previous tile's LDS
        for (int idx = tid; idx < TK * NBLK; idx += MLA_THREADS) {
            const int key = idx / NBLK, blk = idx % NBLK;
            const int r = sm.rowid[key];
            const float sv = r >= 0 ? scales[(size_t)r * NBLK + blk] : 0.0f;
            sm.sc[key][blk] = sv;
            // positive floats order like their bit patterns
            if (blk < 4 && sv > 0.0f) atomicMax(&sm.scmax_bits, __builtin_bit_cast(uint32_t, sv));
        }

        // ---- this wave's K fragments: issue the loads first ----
        const int my_row_s = sm.rowid[wave * 16 + l16];
        const int my_row_c = my_row_s >= 0 ? my_row_s : 0;   // masked keys read row 0
        u32x4 kraw[9];
        {
            const uint8_t *kr = rows + (size_t)my_row_c * KDIM + 16 * g;
#pragma unroll
            for (int j = 0; j < 9; j++) kraw[j] = *(const u32x4 *)(kr + 64 * j);
        }

        // ---- V^T tile: 4 keys x 16 dims per thread-step, transposed into LDS ----
        {
            const int kq = lane & 15;                  // key quad: keys 4kq..4kq+3
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int chunk = it * 16 + wave * 4 + (lane >> 4);   // 16-dim chunk, 0..31
                u32x4 raw[4];
#pragma unroll
                for (int a = 0; a < 4; a++) {
                    const int r = sm.rowid[4 * kq + a];
                    raw[a] = *(const u32x4 *)(rows + (size_t)(r >= 0 ? r : 0) * KDIM + 16 * chunk);
                }
#pragma unroll
                for (int dw = 0; dw < 4; dw++) {
                    // dims 4dw..4dw+3 of the chunk, for the 4 keys
                    uint32_t lo[4], hi[4];   // fp16 pairs (dim 4dw,4dw+1) and (4dw+2,4dw+3)
#pragma unroll
                    for (int a = 0; a < 4; a++) {
                        lo[a] = e4m3x2_to_f16x2<false>(raw[a][dw]);
                        hi[a] = e4m3x2_to_f16x2<true>(raw[a][dw]);
                    }
                    // gather one dim over the 4 keys: low halves, then high halves
                    const int d = chunk * 16 + dw * 4;
                    u32x2 w0, w1, w2, w3;
                    w0[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x05040100u);
                    w0[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x05040100u);
                    w1[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u);
                    w1[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302u);
                    w2[0] = __builtin_amdgcn_perm(hi[1], hi[0], 0x05040100u);
                    w2[1] = __builtin_amdgcn_perm(hi[3], hi[2], 0x05040100u);
                    w3[0] = __builtin_amdgcn_perm(hi[1], hi[0], 0x07060302u);
                    w3[1] = __builtin_amdgcn_perm(hi[3], hi[2], 0x07060302u);
                    *(u32x2 *)&sm.vt[d + 0][4 * kq] = w0;
                    *(u32x2 *)&sm.vt[d + 1][4 * kq] = w1;
                    *(u32x2 *)&sm.vt[d + 2][4 * kq] = w2;
                    *(u32x2 *)&sm.vt[d + 3][4 * kq] = w3;
                }
            }
        }
        __syncthreads();   // sc[] and vt[] are complete

        // ---- normaliser of the fp16 value weights ----
        float o_shift = 1.0f;            // exact power of two applied to the accumulator
        {
            const uint32_t mb = sm.scmax_bits;
            const int e_tile = mb ? (int)((mb >> 23) & 0xFFu) - 126 : E_NONE;
            if (e_tile > e_run) {
                if (e_run != E_NONE) {
                    const int d = e_run - e_tile;
                    o_shift = __builtin_ldexpf(1.0f, d < -120 ? -120 : d);
                }
                e_run = e_tile;
            }
        }
        int wexp = 14 - e_run;
        wexp = wexp > 120 ? 120 : (wexp < -120 ? -120 : wexp);
        const float wfac = e_run == E_NONE ? 0.0f : __builtin_ldexpf(1.0f, wexp);

        // ---- scores for this wave's 16 keys ----
        float s[2][4];
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
            for (int i = 0; i < 4; i++) s[h2][i] = 0.0f;
#pragma unroll
        for (int blk = 0; blk < NBLK; blk++) {
            f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
            const int j0 = blk * 2, j1 = blk == 4 ? 9 : blk * 2 + 2;
#pragma unroll
            for (int j = j0; j < j1; j++) {
                u32x4 ka, kb;
                ka[0] = e4m3x2_to_bf16x2<false>(kraw[j][0]);
                ka[1] = e4m3x2_to_bf16x2<true>(kraw[j][0]);
                ka[2] = e4m3x2_to_bf16x2<false>(kraw[j][1]);
                ka[3] = e4m3x2_to_bf16x2<true>(kraw[j][1]);
                kb[0] = e4m3x2_to_bf16x2<false>(kraw[j][2]);
                kb[1] = e4m3x2_to_bf16x2<true>(kraw[j][2]);
                kb[2] = e4m3x2_to_bf16x2<false>(kraw[j][3]);
                kb[3] = e4m3x2_to_bf16x2<true>(kraw[j][3]);
                const bf16x8 a0 = __builtin_bit_cast(bf16x8, ka);
                const bf16x8 a1 = __builtin_bit_cast(bf16x8, kb);
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++) {
                    acc[h2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[h2][2 * j], acc[h2], 0, 0, 0);
                    acc[h2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qf[h2][2 * j + 1], acc[h2], 0, 0, 0);
                }
            }
            // rows of the result are keys 16*wave + 4g + i
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float ks = sm.sc[wave * 16 + 4 * g + i][blk] * p.scale;
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++) s[h2][i] = __builtin_fmaf(acc[h2][i], ks, s[h2][i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (sm.rowid[wave * 16 + 4 * g + i] < 0)
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++) s[h2][i] = -INFINITY;

        // ---- tile maximum per head: lane, lane groups, waves ----
        float tmax[2];
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
            float v = fmaxf(fmaxf(s[h2][0], s[h2][1]), fmaxf(s[h2][2], s[h2][3]));
            v = fmaxf(v, __shfl_xor(v, 16, 64));
            v = fmaxf(v, __shfl_xor(v, 32, 64));
            tmax[h2] = v;
        }
        if (g == 0) {
            sm.wmax[wave][l16] = tmax[0];
            sm.wmax[wave][16 + l16] = tmax[1];
        }
        __syncthreads();
        float corr[2];
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
            float mt = fmaxf(fmaxf(sm.wmax[0][h2 * 16 + l16], sm.wmax[1][h2 * 16 + l16]),
                             fmaxf(sm.wmax[2][h2 * 16 + l16], sm.wmax[3][h2 * 16 + l16]));
            const float m_new = fmaxf(m_run[h2], mt);
            const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
            corr[h2] = __expf(m_run[h2] - m_safe);      // exp(-inf) = 0 on the first live tile
            m_run[h2] = m_new;
            float psum = 0.0f;
            float pv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                pv[i] = __expf(s[h2][i] - m_safe);      // masked: exp(-inf) = 0
                psum += pv[i];
            }
            l_part[h2] = l_part[h2] * corr[h2] + psum;
            // four copies of p, each folded with the value scale of one dim block
#pragma unroll
            for (int blk = 0; blk < 4; blk++) {
                float w[4];
#pragma unroll
                for (int i = 0; i < 4; i++)
                    w[i] = pv[i] * (sm.sc[wave * 16 + 4 * g + i][blk] * wfac);   // <= 2^14
                u32x2 pk;
                pk[0] = pack_f16_rne(w[0], w[1]);
                pk[1] = pack_f16_rne(w[2], w[3]);
                *(u32x2 *)&sm.ps[blk][h2 * 16 + l16][wave * 16 + 4 * g] = pk;
            }
        }
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
            const float oc = corr[h2] * o_shift;
#pragma unroll
            for (int db = 0; db < 8; db++) oacc[db][h2] *= oc;
        }
        __syncthreads();   // ps[] complete

        // ---- values: dims 128*wave .. 128*wave+127, all TK keys ----
#pragma unroll
        for (int ks = 0; ks < TK / 32; ks++) {
            f16x8 pb[2];
#pragma unroll
            for (int h2 = 0; h2 < 2; h2++)
                pb[h2] = __builtin_bit_cast(
                    f16x8, *(const u32x4 *)&sm.ps[wave][h2 * 16 + l16][32 * ks + 8 * g]);
#pragma unroll
            for (int db = 0; db < 8; db++) {
                const f16x8 va = __builtin_bit_cast(
                    f16x8, *(const u32x4 *)&sm.vt[128 * wave + 16 * db + l16][32 * ks + 8 * g]);
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++)
                    oacc[db][h2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb[h2], oacc[db][h2], 0, 0, 0);
            }
        }
    }
    // accumulator units -> true units
    float o_unit = 0.0f;
    if (e_run != E_NONE) {
        int ue = e_run - 14;
        ue = ue > 120 ? 120 : (ue < -120 ? -120 : ue);
        o_unit = __builtin_ldexpf(1.0f, ue);
    }

    // ---- epilogue: row sums over lane groups and waves ----
    __syncthreads();
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) {
        float v = l_part[h2];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (g == 0) sm.wsum[wave][h2 * 16 + l16] = v;
    }
    __syncthreads();
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) {
        const int head = hb * ROWS + h2 * 16 + l16;
        if (head >= p.nh) continue;
        const float l = sm.wsum[0][h2 * 16 + l16] + sm.wsum[1][h2 * 16 + l16] +
                        sm.wsum[2][h2 * 16 + l16] + sm.wsum[3][h2 * 16 + l16];
        if (p.n_splits == 1) {
            const float inv = l > 0.0f ? o_unit / l : 0.0f;
            float *o = p.out + ((size_t)y * p.nh + head) * VDIM + 128 * wave + 4 * g;
#pragma unroll
            for (int db = 0; db < 8; db++) *(f32x4 *)(o + 16 * db) = oacc[db][h2] * inv;
        } else {
            const size_t pr = ((size_t)y * p.n_splits + split) * p.nh + head;
            float *o = p.part_acc + pr * VDIM + 128 * wave + 4 * g;
#pragma unroll
            for (int db = 0; db < 8; db++) *(f32x4 *)(o + 16 * db) = oacc[db][h2] * o_unit;
            if (wave == 0 && g == 0) {
                p.part_ml[pr * 2 + 0] = m_run[h2];
                p.part_ml[pr * 2 + 1] = l;
            }
        }
    }
}

static int run_mla(MlaParams &p, hipStream_t s) {
    static bool attr_set = false;
    const size_t smem = sizeof(MlaSmem);
    if (!attr_set) {
        CWICK_HIP_CALL(hipFuncSetAttribute((const void *)mla_fwd_kernel,
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
        mla_fwd_kernel<<<dim3((unsigned)total), MLA_THREADS, smem, s>>>(p);
    }
    CWICK_HIP_CALL(hipGetLastError());
    if (p.n_splits > 1) {
        ProfScope ps(CWICK_HIP_PROF_MLA_MERGE, s);
        splitk_merge_kernel<VDIM><<<dim3(p.nh, p.nq), 256, 0, s>>>(p.part_acc, p.part_ml, p.n_splits, p.nh, p.out);
        CWICK_HIP_CALL(hipGetLastError());
    }
    return 1;
}

int launch_mla_decode_v1(const uint8_t *rows, const float *scales, int64_t row_bstride,
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
                      (uintptr_t)out % 16 == 0,
                  "mla_decode: rows, q and out must be 16-byte aligned");
    MlaParams p{};
    p.rows = rows; p.scales = scales; p.row_bstride = row_bstride; p.scale_bstride = scale_bstride;
    p.n_rows = n_rows; p.sel = sel; p.n_list = n_list; p.list_step = 0;
    p.q = q; p.nh = n_heads; p.nq = batch; p.scale = scale; p.out = out;
    // one workgroup per CU is resident (LDS); aim for one round of workgroups
    const int n_hb = (n_heads + ROWS - 1) / ROWS;
    int64_t want = num_cus() / ((int64_t)n_hb * batch);
    if (want < 1) want = 1;
    int64_t per = (n_list + want - 1) / want;
    per = ((per + TK - 1) / TK) * TK;
    p.keys_per_split = per;
    p.n_splits = (int)((n_list + per - 1) / per);
    return run_mla(p, s);
}

int launch_mla_prefill_v1(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                       const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s) {
    CWICK_REQUIRE(rows && scales && q && out, "mla_prefill: null pointer");
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "mla_prefill: n_heads %d (1..128)", n_heads);
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= ((int64_t)1 << 31) - 1 && n <= (1 << 22),
                  "mla_prefill: pos0 %lld n %lld", (long long)pos0, (long long)n);
    CWICK_REQUIRE(scale > 0.0f && scale < INFINITY, "mla_prefill: scale must be positive");
    CWICK_REQUIRE((uintptr_t)rows % 16 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)out % 16 == 0,
                  "mla_prefill: rows, q and out must be 16-byte aligned");
    MlaParams p{};
    p.rows = rows; p.scales = scales; p.row_bstride = 0; p.scale_bstride = 0;
    p.n_rows = pos0 + n; p.sel = nullptr; p.n_list = pos0 + 1; p.list_step = 1;
    p.q = q; p.nh = n_heads; p.nq = (int)n; p.scale = scale; p.out = out;
    p.n_splits = 1;
    p.keys_per_split = ((pos0 + n + TK - 1) / TK) * TK;
    return run_mla(p, s);
}

}  // namespace cwick
