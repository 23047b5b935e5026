// mla_stream.hip -- absorbed-latent MLA, streaming form (decode, sparse decode and
// chunked prefill of src/attention.c:749-811 / :1010-1019 over the FP8 latent).
//
// Same mathematics as mla.hip; a different schedule, built to keep the matrix
// core fed at batch 1 where a workgroup lives for only a few thousand cycles:
//
//   * workgroup = 4 waves on the SAME 32 query rows (heads of one query); each
//     wave streams its own 32-key tiles of the workgroup's key slice (tiles
//     w, w+4, ...).  There is no workgroup barrier in the loop: a wave owns its
//     LDS buffers, its running (m, l) and a full 512 x 32 output accumulator;
//     the four waves are merged once, at the end, through LDS.
//   * tiles travel global -> LDS without touching registers
//     (global_load_lds_dwordx4: lane l's 16 bytes land at base + 16 l), one tile
//     ahead of the compute, into the layout
//         tile[16-dim group dg = 0..35][key position 0..31][16 bytes]
//     from which both operands read conflict-free:
//       K fragment  (scores, A operand of S^T = K Q^T): lane (position m, half g)
//                   reads 16 B at [2jj+g][m] -- 64 lanes cover 1 KiB contiguous;
//       V^T fragment (values, A operand of O^T = V^T P^T): the LDS transpose read
//                   ds_read_b64_tr_b8 hands lane (dim, g) the 8 key bytes of its
//                   dim; the 16 lanes of a group address 8 positions x 16 B =
//                   128 B contiguous.
//     The E4M3 bytes are widened in registers (exactly) to bf16 for the scores
//     and to fp16 for the values; the per-128-dim fp32 block scales arrive by
//     the same route ([blk][position]) and multiply the fp32 partial dots
//     (scores) or the softmax weights (values).
//   * v_mfma_f32_32x32x16_{bf16,f16}: one head per lane column, so the softmax
//     statistics are lane scalars and P^T is the score accumulator itself (the
//     contraction slots of the value MFMA are numbered to match its layout).
//   * lazy running maximum (advance only when a tile beats it by 2^4) so the 256
//     accumulator registers are rarely rescaled; weights are kept in fp16 range
//     by a power-of-two normaliser of the value scales.
#include "common.hpp"
#include "merge.hpp"

namespace cwick {

namespace {

constexpr int KDIM = CWICK_HIP_LATENT_KDIM;   // 576
constexpr int VDIM = CWICK_HIP_LATENT_VDIM;   // 512
constexpr int NBLK = CWICK_HIP_LATENT_NBLK;   // 5
constexpr int THREADS = 256;
constexpr int TKW = 32;                       // keys per wave tile
constexpr int NDG = KDIM / 16;                // 36 sixteen-dim groups per row
constexpr int ROWS = 32;                      // query rows per workgroup
constexpr int DMA_PER_TILE = NDG / 2 + 3;     // LDS-DMA instructions per tile (rows + scales)
constexpr float LAZY = 4.0f;                  // log2 slack of the running maximum
constexpr int WEXP = 10;                      // weights carry 2^(WEXP - e_run): <= 2^(LAZY + WEXP)
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
    int64_t keys_per_split;   // multiple of 4*TKW
    float *out, *part_acc, *part_ml;
};

struct WaveBuf {
    uint8_t tile[NDG][TKW][16];   // 18432 B
    float sc[6][TKW];             // [blk][position]; row 5 is padding for the paired DMA
};
struct Smem {
    WaveBuf buf[4][2];            // [wave][stage]: 153600 B, reused as merge scratch
    float mrg_m[4][ROWS];
    float mrg_l[4][ROWS];
    int mrg_e[4];
};

__device__ __forceinline__ float pow2i(int e) {
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
    return __builtin_bit_cast(float, (uint32_t)(e + 127) << 23);
}

__global__ void __launch_bounds__(THREADS, 1) mla_stream_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    Smem &sm = *reinterpret_cast<Smem *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int m = lane & 31;      // key position (scores) / head column / dim row
    const int g = lane >> 5;      // which half of the contraction slots

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
    const int n_tiles = k_end > k_begin ? (int)((k_end - k_begin + TKW - 1) / TKW) : 0;

    // ---- tile fetch: one tile = 18 row DMAs (2 dim groups x 32 positions each) + 3 scale DMAs
    auto row_of = [&](int t) -> int {
        const int64_t i = k_begin + (int64_t)t * TKW + m;
        int64_t r = -1;
        if (t < n_tiles && i < k_end) {
            r = sel ? (int64_t)sel[i] : i;
            if (r < 0 || r >= p.n_rows) r = -1;
        }
        return (int)r;
    };
    auto issue = [&](int r, WaveBuf *b) {
        const int64_t rc = r >= 0 ? r : 0;            // masked positions fetch row 0, weight 0
        const uint8_t *gsrc = rows + rc * KDIM + 16 * g;
#pragma unroll
        for (int n = 0; n < NDG / 2; n++)
            __builtin_amdgcn_global_load_lds((glb_void *)(gsrc + 32 * n), (lds_void *)&b->tile[2 * n][0][0],
                                             16, 0, 0);
        const float *ssrc = scales + rc * NBLK;
#pragma unroll
        for (int n = 0; n < 3; n++) {
            int blk = 2 * n + g;
            blk = blk > 4 ? 4 : blk;
            __builtin_amdgcn_global_load_lds((glb_void *)(ssrc + blk), (lds_void *)&b->sc[2 * n][0], 4, 0, 0);
        }
    };

    int t = wave;
    int row_cur = row_of(t);          // row of the tile about to be fetched
    int row_nxt = row_of(t + 4);
    if (t < n_tiles) issue(row_cur, &sm.buf[wave][0]);

    // ---- Q fragments (B operand): lane (head m, half g) holds, for pair jj,
    // dims 32jj+16g+[0,8) (step 2jj) and 32jj+16g+[8,16) (step 2jj+1)
    bf16x8 qf[36];
    {
        int head = hb * ROWS + m;
        if (head >= p.nh) head = p.nh - 1;
        const uint16_t *qrow = p.q + ((size_t)y * p.nh + head) * KDIM + 16 * g;
#pragma unroll
        for (int jj = 0; jj < 18; jj++) {
            qf[2 * jj] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + 32 * jj));
            qf[2 * jj + 1] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qrow + 32 * jj + 8));
        }
    }

    f32x16 oacc[16];
#pragma unroll
    for (int db = 0; db < 16; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = 0.0f;
    float m_ref = -INFINITY, l_part = 0.0f;
    int e_run = E_NONE;
    const float c0 = p.scale * 1.44269504088896340736f;   // scores live in log2 units

    // transpose-read addressing (constant per lane): 16-lane group G, lane i in it
    const int G = lane >> 4, gi = lane & 15;
    const int tr_k = gi >> 1;                                 // contraction slot 0..7
    const int tr_pos = 4 * (G >> 1) + (tr_k & 3) + 8 * (tr_k >> 2);   // + 16 s
    const int tr_dgo = G & 1;                                 // + 2 db
    const int tr_byte = 8 * (gi & 1);

    int stage = 0;
    while (t < n_tiles) {
        const int row_this = row_cur;
        const uint64_t valid64 = __ballot(row_this >= 0);
        const uint32_t valid = (uint32_t)valid64;             // lanes 0..31 <-> positions
        WaveBuf &B = sm.buf[wave][stage];
        // fetch the next tile of this wave into the other stage, then wait for this one
        const int tn = t + 4;
        row_cur = row_nxt;
        asm volatile("" ::: "memory");
        if (tn < n_tiles) {
            issue(row_cur, &sm.buf[wave][stage ^ 1]);
            row_nxt = row_of(tn + 4);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DMA_PER_TILE) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }

        // ---- normaliser of the fp16 value weights (wave-uniform) ----
        float o_shift = 1.0f;
        {
            float sv = 0.0f;
            if (row_this >= 0 && g == 0)
                sv = fmaxf(fmaxf(B.sc[0][m], B.sc[1][m]), fmaxf(B.sc[2][m], B.sc[3][m]));
            sv = wave_max(sv);
            const uint32_t mb = __builtin_bit_cast(uint32_t, sv);
            const int e_tile = sv > 0.0f ? (int)((mb >> 23) & 0xFFu) - 126 : E_NONE;
            if (e_tile > e_run) {
                if (e_run != E_NONE) o_shift = pow2i(e_run - e_tile);
                e_run = e_tile;
            }
        }
        const float wfac = e_run == E_NONE ? 0.0f : pow2i(WEXP - e_run);

        // ---- scores: S^T[32 positions][32 heads] ----
        f32x16 S;
#pragma unroll
        for (int i = 0; i < 16; i++) S[i] = 0.0f;
        // The LDS read of pair jj+1 is issued before the MFMAs of pair jj and the
        // scheduler is fenced per pair: left alone it hoists every fragment load to
        // the top, runs out of registers and spills the Q fragments.
        u32x4 raw = *(const u32x4 *)&B.tile[g][m][0];
#pragma unroll
        for (int blk = 0; blk < NBLK; blk++) {
            f32x16 acc;
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] = 0.0f;
            const int j0 = 4 * blk, j1 = blk == 4 ? 18 : 4 * blk + 4;
#pragma unroll
            for (int jj = j0; jj < j1; jj++) {
                u32x4 nxt = raw;
                if (jj + 1 < 18) nxt = *(const u32x4 *)&B.tile[2 * (jj + 1) + g][m][0];
                u32x4 ka, kb;
                ka[0] = e4m3x2_to_bf16x2<false>(raw[0]);
                ka[1] = e4m3x2_to_bf16x2<true>(raw[0]);
                ka[2] = e4m3x2_to_bf16x2<false>(raw[1]);
                ka[3] = e4m3x2_to_bf16x2<true>(raw[1]);
                kb[0] = e4m3x2_to_bf16x2<false>(raw[2]);
                kb[1] = e4m3x2_to_bf16x2<true>(raw[2]);
                kb[2] = e4m3x2_to_bf16x2<false>(raw[3]);
                kb[3] = e4m3x2_to_bf16x2<true>(raw[3]);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka), qf[2 * jj], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb), qf[2 * jj + 1], acc, 0, 0, 0);
                raw = nxt;
                __builtin_amdgcn_sched_barrier(0);
            }
            // accumulator register i <-> position (i/4)*8 + 4g + i%4
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const f32x4 s4 = *(const f32x4 *)&B.sc[blk][8 * q4 + 4 * g];
#pragma unroll
                for (int r = 0; r < 4; r++) S[4 * q4 + r] = __builtin_fmaf(acc[4 * q4 + r], s4[r], S[4 * q4 + r]);
            }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int pos = (i >> 2) * 8 + 4 * g + (i & 3);
            float x = S[i] * c0;
            if (!((valid >> pos) & 1u)) x = -INFINITY;
            S[i] = x;
            tmax = fmaxf(tmax, x);
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
            // The accumulator lives in the AGPR half of the register file.  A plain
            // `oacc *= oc` makes the compiler move all 256 values to the VGPR half
            // for the whole loop and spill the Q fragments; so the rare rescale is
            // spelled out: read one AGPR, multiply, write it back.  (The MFMAs that
            // produced / will consume these registers are hundreds of instructions
            // away on either side, far beyond any MFMA<->VALU wait-state rule.)
            for (int db = 0; db < 16; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    float tmp;
                    asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\t"
                                 "v_accvgpr_write_b32 %0, %1"
                                 : "+a"(oacc[db][i]), "=&v"(tmp)
                                 : "v"(oc));
                }
        }
        const float m_use = m_ref == -INFINITY ? 0.0f : m_ref;
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            S[i] = __builtin_amdgcn_exp2f(S[i] - m_use);      // masked: exp2(-inf) = 0
            psum += S[i];
        }
        l_part += psum;

        // ---- values: O^T[512 dims][32 heads] += V^T[dims][32 positions] . P^T ----
        i32x2 vraw = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (lds_i32x2 *)&B.tile[tr_dgo][tr_pos][tr_byte]);
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {
            u32x4 pw[2];
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const f32x4 s4 = *(const f32x4 *)&B.sc[blk][8 * q4 + 4 * g];
                const float w0 = S[4 * q4 + 0] * (s4[0] * wfac), w1 = S[4 * q4 + 1] * (s4[1] * wfac);
                const float w2 = S[4 * q4 + 2] * (s4[2] * wfac), w3 = S[4 * q4 + 3] * (s4[3] * wfac);
                // register 8s+j <-> slot j of step s
                pw[q4 >> 1][2 * (q4 & 1)] = pack_f16_rne(w0, w1);
                pw[q4 >> 1][2 * (q4 & 1) + 1] = pack_f16_rne(w2, w3);
            }
#pragma unroll
            for (int dbl = 0; dbl < 4; dbl++) {
                const int db = 4 * blk + dbl;
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    // next fragment in flight before this one is consumed
                    const int nstep = 2 * db + s + 1;
                    i32x2 vnxt = vraw;
                    if (nstep < 32)
                        vnxt = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                            (lds_i32x2 *)&B.tile[2 * (nstep >> 1) + tr_dgo][16 * (nstep & 1) + tr_pos][tr_byte]);
                    u32x4 vh;
                    vh[0] = e4m3x2_to_f16x2<false>((uint32_t)vraw[0]);
                    vh[1] = e4m3x2_to_f16x2<true>((uint32_t)vraw[0]);
                    vh[2] = e4m3x2_to_f16x2<false>((uint32_t)vraw[1]);
                    vh[3] = e4m3x2_to_f16x2<true>((uint32_t)vraw[1]);
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        __builtin_bit_cast(f16x8, vh), __builtin_bit_cast(f16x8, pw[s]), oacc[db], 0, 0, 0);
                    vraw = vnxt;
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        t = tn;
        stage ^= 1;
    }

    // ---- merge the four waves ----
    const float l_wave = l_part + __shfl_xor(l_part, 32, 64);
    if (g == 0) sm.mrg_m[wave][m] = m_ref;
    if (lane == 0) sm.mrg_e[wave] = e_run;
    __syncthreads();                       // every wave is done with its tile buffers
    const float M = fmaxf(fmaxf(sm.mrg_m[0][m], sm.mrg_m[1][m]), fmaxf(sm.mrg_m[2][m], sm.mrg_m[3][m]));
    const int E = max(max(sm.mrg_e[0], sm.mrg_e[1]), max(sm.mrg_e[2], sm.mrg_e[3]));
    const float f_soft = (m_ref == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_ref - M);
    const float f_all = (e_run == E_NONE) ? 0.0f : f_soft * pow2i(e_run - E);
    if (g == 0) sm.mrg_l[wave][m] = l_wave * f_soft;
#pragma unroll
    for (int db = 0; db < 16; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] *= f_all;

    float *scratch = reinterpret_cast<float *>(smem_raw);     // 2 x 64 KiB inside buf[]
    auto put = [&](int slot) {
#pragma unroll
        for (int db = 0; db < 16; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r];
                *(f32x4 *)&scratch[(((size_t)slot * 64 + db * 4 + q4) * 64 + lane) * 4] = v;
            }
    };
    auto add = [&](int slot) {
#pragma unroll
        for (int db = 0; db < 16; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const f32x4 v = *(const f32x4 *)&scratch[(((size_t)slot * 64 + db * 4 + q4) * 64 + lane) * 4];
#pragma unroll
                for (int r = 0; r < 4; r++) oacc[db][4 * q4 + r] += v[r];
            }
    };
    if (wave >= 2) put(wave - 2);
    __syncthreads();
    if (wave < 2) add(wave);
    __syncthreads();
    if (wave == 1) put(0);
    __syncthreads();
    if (wave != 0) return;
    add(0);

    const int head = hb * ROWS + m;
    if (head >= p.nh) return;
    const float L = (sm.mrg_l[0][m] + sm.mrg_l[1][m]) + (sm.mrg_l[2][m] + sm.mrg_l[3][m]);
    const float unit_f = E == E_NONE ? 0.0f : pow2i(E - WEXP);
    if (p.n_splits == 1) {
        const float inv = L > 0.0f ? unit_f / L : 0.0f;
        float *o = p.out + ((size_t)y * p.nh + head) * VDIM + 4 * g;
#pragma unroll
        for (int db = 0; db < 16; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r] * inv;
                *(f32x4 *)(o + 32 * db + 8 * q4) = v;
            }
    } else {
        const size_t pr = ((size_t)y * p.n_splits + split) * p.nh + head;
        float *o = p.part_acc + pr * VDIM + 4 * g;
#pragma unroll
        for (int db = 0; db < 16; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = oacc[db][4 * q4 + r] * unit_f;
                *(f32x4 *)(o + 32 * db + 8 * q4) = v;
            }
        if (g == 0) {
            p.part_ml[pr * 2 + 0] = M * 0.69314718055994530942f;   // the merge pass works in e-units
            p.part_ml[pr * 2 + 1] = L;
        }
    }
}

int run(Params &p, hipStream_t s) {
    static bool attr_set = false;
    const size_t smem = sizeof(Smem);
    if (!attr_set) {
        CWICK_HIP_CALL(hipFuncSetAttribute((const void *)mla_stream_kernel,
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
        mla_stream_kernel<<<dim3((unsigned)total), THREADS, smem, s>>>(p);
    }
    CWICK_HIP_CALL(hipGetLastError());
    if (p.n_splits > 1) {
        ProfScope ps(CWICK_HIP_PROF_MLA_MERGE, s);
        splitk_merge_kernel<VDIM><<<dim3(p.nh, p.nq), 256, 0, s>>>(p.part_acc, p.part_ml, p.n_splits, p.nh, p.out);
        CWICK_HIP_CALL(hipGetLastError());
    }
    return 1;
}

}  // namespace

int launch_mla_decode_v2(const uint8_t *rows, const float *scales, int64_t row_bstride,
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
    // one workgroup per CU is resident (LDS): aim for one round of workgroups, each
    // slice a whole number of 4-wave rounds
    const int n_hb = (n_heads + ROWS - 1) / ROWS;
    int64_t want = num_cus() / ((int64_t)n_hb * batch);
    if (want < 1) want = 1;
    if (want > MERGE_MAX_SPLITS) want = MERGE_MAX_SPLITS;
    int64_t per = (n_list + want - 1) / want;
    per = ((per + 4 * TKW - 1) / (4 * TKW)) * (4 * TKW);
    p.keys_per_split = per;
    p.n_splits = (int)((n_list + per - 1) / per);
    return run(p, s);
}

int launch_mla_prefill_v2(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
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
    p.keys_per_split = ((pos0 + n + 4 * TKW - 1) / (4 * TKW)) * (4 * TKW);
    return run(p, s);
}

}  // namespace cwick
