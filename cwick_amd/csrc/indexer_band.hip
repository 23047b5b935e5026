// indexer_band.hip -- the indexer scores of a fused select (indexer -> top-k) without running
// the exact vector-ALU kernel over every key.
//
// The selection has to be the one the reference makes (src/attention.c:573-598,
// src/ds_model.c:1108-1152): bit-identical scores for every key that could change it.  Most
// keys cannot.  So:
//
//   1. indexer_approx_kernel: approximate scores on the bf16 matrix cores,
//          st[t] = ks[t] * sum_h w[h] * max(q_h . e_t, 0),
//      and next to them a bound on |st[t] - s[t]|, s the reference's score.  The products
//      e*q are exact in fp32 either way (a 4-bit times an 8-bit significand); the two sides
//      differ in the order of the additions and in a handful of roundings:
//          reference dot (dot_f32: four fma chains of 32, three additions)  35 roundings
//          matrix-core dot, any order and any internal truncation          <= 256 roundings
//          scale, weight, sum over at most 64 heads, on each side          <= 2 * 66 roundings
//      each relative to A_h = sum_i |e_i||q_hi| >= |q_h . e_t|, so
//          |st - s| <= 450 u * ks[t] * sum_h |w_h| A_h[t],   u = 2^-24,
//      and sum_h |w_h| A_h[t] = sum_i |e_ti| c_i with c_i = sum_h |w_h||q_hi|: one more row
//      through the matrix core, with c rounded up to bf16.  beta[t] = 512 u * ks[t] * that row
//      (the slack covers the rounding of the bound itself); beta = max_t beta[t].
//   2. top-k machinery on st: T = the k-th largest approximate score (topk.hip).
//   3. classify: at most k-1 keys have st > T.  A key with st > T + 2 beta has s > T + beta, and
//      every key that scores at least as much has st > T: it is among at most k-2 others, so it
//      is selected whatever the ties do.  At least k keys have st >= T, hence s >= T - beta; a
//      key with st < T - 2 beta has s < T - beta and is not selected.  The first kind gets +inf,
//      the second -inf, the rest (a few hundred of 65536) are candidates.
//   4. indexer_rescore_kernel: the reference's arithmetic, instruction for instruction as in
//      indexer.hip, for the candidates only, spread over heads so that it takes microseconds.
//   5. the selection is the +inf keys (fewer than k, all selected) and the best k - (their number)
//      candidates by exact score, ties to the smaller index: topk_band_finish_kernel (topk.hip)
//      ranks the candidates and writes the indices in order.
// Whenever a row does not fit this (more candidates than the list holds, a bound that is not
// finite, NaN where T should be), the rescoring kernel's workgroups run the exact kernel's code
// on all keys of that row and the finish kernel's first workgroup the plain select.
#include "indexer_exact.hpp"

namespace cwick {

constexpr int IB_THREADS = 512;
constexpr int IB_WAVES = IB_THREADS / 64;
constexpr int IB_QROW = 128 + 8;                 // bf16 per head row of q in LDS (padded: 272 bytes)
constexpr int IB_KEYS = CWICK_INDEXER_APPROX_KEYS;   // keys per workgroup of the approximate kernel
constexpr int IB_HD = CWICK_HIP_INDEX_DIM;    // 128

typedef __attribute__((ext_vector_type(2))) float ib_f32x2;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;

// v[l] + v[l ^ 32] in every lane: the two halves of the wave trade places between two copies
__device__ __forceinline__ float ib_half_sum(float v) {
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
}

__global__ void __launch_bounds__(IB_THREADS) __attribute__((amdgpu_waves_per_eu(2)))
indexer_approx_kernel(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                      int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                      const uint16_t *__restrict__ q,   // [batch][ih][128] bf16
                      const float *__restrict__ w,      // [batch][ih]
                      int ih, float *__restrict__ scores, float *__restrict__ beta_slots,
                      IndexerBandRow *__restrict__ rows,
                      uint32_t *__restrict__ digit0, size_t digit0_row) {   // optional: first-digit counts for the radix select
    __shared__ __attribute__((aligned(16))) float cpart_sh[IB_THREADS / 16][IB_HD];
    __shared__ __attribute__((aligned(16))) uint16_t cb_sh[IB_HD + 64];          // coefficients, then 128 bytes of zeros
    __shared__ uint32_t hist0[256 * 8];
    __shared__ __attribute__((aligned(16))) uint16_t q_sh[64 * IB_QROW];
    __shared__ float w_sh[64];
    __shared__ float bmax_sh[IB_THREADS / 64];
    const int b = blockIdx.y, wg = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint16_t *qb = q + (size_t)b * ih * IB_HD;
    const float *wb = w + (size_t)b * ih;
    if (wg == 0 && tid == 0) {
        rows[b].n_cand = 0u;
        rows[b].fallback = 0u;
    }
    // Contraction slot j of k-step ks in lane half g is dimension 64 g + 8 ks + j (the same on
    // both operands, so the order is free): a lane reads 64 contiguous bytes of its key row,
    // four 16-byte loads, and a wave reads 32 whole rows.
    const int row = lane & 31, g = lane >> 5;
    const uint8_t *kb = keys + (size_t)b * key_bstride;
    const float *ksb = kscale + (size_t)b * kscale_bstride;
    const int64_t wbase = (int64_t)wg * IB_KEYS + (int64_t)wave * (IB_KEYS / IB_WAVES);
    constexpr int N_IT = IB_KEYS / IB_WAVES / 32;
    // the key bytes and the scale of an iteration are loaded two iterations ahead
    u32x4 raw_a[4], raw_b[4], raw_c[4];
    float kst_a, kst_b, kst_c;
    auto load_keys = [&](int it, u32x4 (&raw)[4], float &kst) {
        int64_t tc = wbase + (it < N_IT ? it : N_IT - 1) * 32 + row;
        tc = tc < n_keys ? tc : n_keys - 1;
        const uint8_t *krow = kb + (size_t)tc * IB_HD + 64 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) raw[i] = *(const u32x4 *)(krow + 16 * i);
        kst = ksb[tc];
    };
    // A operands (rows = heads): every wave needs all of q, so the workgroup fetches it once
    // (sixteen bytes per thread and step) and the waves take their fragments from LDS; rows are
    // 272 bytes apart there, which spreads the sixteen-byte reads of consecutive heads over the
    // banks.  The loads go out first and the first two key iterations right behind them.
    // c_i = sum_h |w_h| |q_hi| starts from the same registers: thread (group = tid / 16, part =
    // tid % 16) holds dims 8 part .. +7 of heads group + 16 j, adds up its four heads and leaves
    // the eight sums in LDS; after the barrier thread i < 128 adds the sixteen groups of dim i.
    bf16x8 qa[2][8];
    {
        // (the weights first: a load that is waited for drags every load issued before it along)
        const float w_mine = (tid < 64 && tid < ih) ? wb[tid] : 0.0f;
        constexpr int NST = 1024 / IB_THREADS;              // sixteen-byte pieces of q per thread
        float w4[NST];
        u32x4 stage[NST];
#pragma unroll
        for (int j = 0; j < NST; j++) {
            const int head = (tid >> 4) + (IB_THREADS / 16) * j;
            w4[j] = head < ih ? fabsf(wb[head]) : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < NST; j++) {
            const int c = tid + IB_THREADS * j, head = c >> 4, part = c & 15;
            const int hc = head < ih ? head : ih - 1;           // clamped load, zeroed afterwards
            stage[j] = *(const u32x4 *)(qb + (size_t)hc * IB_HD + 8 * part);
            if (head >= ih) stage[j] = (u32x4){0u, 0u, 0u, 0u};
        }
        load_keys(0, raw_a, kst_a);
        load_keys(1, raw_b, kst_b);
        float cp[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < NST; j++) {
            const int c = tid + IB_THREADS * j;
            *(u32x4 *)&q_sh[(c >> 4) * IB_QROW + 8 * (c & 15)] = stage[j];
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t x = stage[j][d];
                cp[2 * d] = __builtin_fmaf(w4[j], __builtin_bit_cast(float, (x << 16) & 0x7FFFFFFFu), cp[2 * d]);
                cp[2 * d + 1] = __builtin_fmaf(w4[j], __builtin_bit_cast(float, x & 0x7FFF0000u), cp[2 * d + 1]);
            }
        }
        *(f32x4 *)&cpart_sh[tid >> 4][8 * (tid & 15)] = (f32x4){cp[0], cp[1], cp[2], cp[3]};
        *(f32x4 *)&cpart_sh[tid >> 4][8 * (tid & 15) + 4] = (f32x4){cp[4], cp[5], cp[6], cp[7]};
        if (tid < 64) w_sh[tid] = w_mine;
    }
#pragma unroll
    for (int j = 0; j < 2048 / IB_THREADS; j++) hist0[tid + IB_THREADS * j] = 0u;
    __syncthreads();
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int ks = 0; ks < 8; ks++)
            qa[mb][ks] = *(const bf16x8 *)&q_sh[(mb * 32 + row) * IB_QROW + 64 * g + 8 * ks];
    if (tid < IB_HD) {
        float part[IB_THREADS / 16], c = 0.0f;
#pragma unroll
        for (int k = 0; k < IB_THREADS / 16; k++) part[k] = cpart_sh[k][tid];
#pragma unroll
        for (int k = 0; k < IB_THREADS / 16; k++) c += part[k];
        cb_sh[tid] = (uint16_t)((__builtin_bit_cast(uint32_t, c) + 0xFFFFu) >> 16);     // rounded up to bf16
        if (tid < 64) cb_sh[IB_HD + tid] = 0;
    }
    __syncthreads();
    // the bound row's A fragments are read from LDS step by step: lanes of row 0 from the
    // coefficients, all others from a stretch of zeros behind them
    const char __attribute__((address_space(3))) *c_lane =
        (const char __attribute__((address_space(3))) *)&cb_sh[row == 0 ? 64 * g : IB_HD];
    // the heads this lane holds after the MFMAs: register i of block mb is head
    // 32 mb + 8 (i / 4) + 4 g + i % 4
    float wl[2][16];
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int i = 0; i < 16; i++) wl[mb][i] = w_sh[mb * 32 + (i >> 2) * 8 + 4 * g + (i & 3)];

    float bmax = 0.0f;
    auto iteration = [&](int it, const u32x4 (&raw)[4], float kst) {
        const int64_t t = wbase + it * 32 + row;
        const bool live = t < n_keys;
        // The accumulators are pinned to VGPRs (through the builtin they land in AGPRs and cost a
        // read each).  The compiler does not see these as MFMAs and leaves out the wait states
        // they need (one state = four cycles = one pass of the matrix pipe): two between a VALU
        // write of an operand and the MFMA that reads it, up to nineteen between the issue of
        // an MFMA and a VALU read of its result.  The first is met by converting the keys
        // of k-step ks + 1 before the MFMAs of k-step ks are issued (which also puts the
        // conversions in the shadow of the matrix pipe), the second by the s_nop behind the loop.
        f32x16 d0, d1, ab;
        typedef __attribute__((ext_vector_type(2))) __bf16 ib_bf16x2;
        u32x4 e[2], ea[2], cfrag[2];
        auto convert = [&](int ks, u32x4 &eo, u32x4 &eao) {
#pragma unroll
            for (int j = 0; j < 2; j++) {                          // exact: E4M3 fits bf16
                const int dw = raw[ks >> 1][2 * (ks & 1) + j];
                eo[2 * j] = __builtin_bit_cast(uint32_t, (ib_bf16x2)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(dw, 1.0f, false));
                eo[2 * j + 1] = __builtin_bit_cast(uint32_t, (ib_bf16x2)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(dw, 1.0f, true));
            }
#pragma unroll
            for (int j = 0; j < 4; j++) eao[j] = eo[j] & 0x7FFF7FFFu;
        };
        convert(0, e[0], ea[0]);
        cfrag[0] = *(const lds_u32x4 *)(c_lane);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            const int cur = ks & 1, nxt = cur ^ 1;
            const u32x4 ea_before = ea[nxt], c_before = cfrag[nxt];   // operands of the last MFMA issued
            if (ks + 1 < 8) {
                convert(ks + 1, e[nxt], ea[nxt]);
                cfrag[nxt] = *(const lds_u32x4 *)(c_lane + 16 * (ks + 1));
            }
            // Everything above is in its registers before the first MFMA below is issued; the
            // operands of the step before stay allocated up to here (an MFMA goes on reading its
            // operands for a while after it has been issued, and the compiler, which does not
            // know, would hand their registers to the conversions above).
            if (ks == 0)
                asm volatile("s_nop 1" : "+v"(e[nxt]), "+v"(ea[nxt]), "+v"(e[cur]), "+v"(ea[cur]), "+v"(cfrag[cur]));
            else
                asm volatile("" : "+v"(e[nxt]), "+v"(ea[nxt]), "+v"(e[cur]), "+v"(ea[cur]), "+v"(cfrag[cur])
                             : "v"(ea_before), "v"(c_before));
            if (ks == 0) {
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d0) : "v"(qa[0][ks]), "v"(e[cur]));
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d1) : "v"(qa[1][ks]), "v"(e[cur]));
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(ab) : "v"(cfrag[cur]), "v"(ea[cur]), "v"(e[cur]));
            } else {
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d0) : "v"(qa[0][ks]), "v"(e[cur]));
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d1) : "v"(qa[1][ks]), "v"(e[cur]));
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(ab) : "v"(cfrag[cur]), "v"(ea[cur]), "v"(e[cur]));
            }
        }
        // Nothing may read the results or write a register that these MFMAs read before the last
        // one is through: the wait carries the accumulators, so that nothing that reads them can
        // be scheduled above it either.
        asm volatile("s_nop 15\n\ts_nop 2" : "+v"(d0), "+v"(d1), "+v"(ab)::"memory");
        float sp = 0.0f, sq = 0.0f, sr = 0.0f, ss = 0.0f;      // four chains: a dependent FMA waits for the one before it
#pragma unroll
        for (int i = 0; i < 16; i++) {
            // one instruction per ReLU (through fmaxf or fmed3 the compiler adds a second one
            // that quiets NaNs; a NaN dot counts as 0 here, and the bound row turns NaN with it)
            float r0, r1;
            asm("v_max_f32 %0, 0, %1" : "=v"(r0) : "v"(d0[i]));
            asm("v_max_f32 %0, 0, %1" : "=v"(r1) : "v"(d1[i]));
            if (i & 1) {
                sr = __builtin_fmaf(wl[0][i], r0, sr);
                ss = __builtin_fmaf(wl[1][i], r1, ss);
            } else {
                sp = __builtin_fmaf(wl[0][i], r0, sp);
                sq = __builtin_fmaf(wl[1][i], r1, sq);
            }
        }
        sp = (sp + sq) + (sr + ss);
        // lane l + lane l ^ 32 without a trip through LDS
        sp = ib_half_sum(sp);
        const float band = ib_half_sum(ab[0]);                     // row 0 sits in the g = 0 lanes
        const float st = sp * kst;
        const float beta = band * fabsf(kst) * (512.0f / 16777216.0f);
        if (live && g == 0) {
            scores[(size_t)b * n_keys + t] = st;
            // the select's first pass over the scores, done here: the leading byte of the order
            // key, counted in eight copies picked by lane (scores crowd into a few bins)
            atomicAdd(&hist0[(topk_key(st) >> 24) * 8 + (lane & 7)], 1u);
        }
        if (live) bmax = (beta <= bmax) ? bmax : beta;             // NaN sticks
    };
    // three register sets in turn, so that the loads of iteration it + 2 go out before
    // iteration it computes and nothing is copied between sets (a copy waits for its load);
    // unrolled, so that every wait counts exactly the loads behind the one it needs
#pragma unroll
    for (int it = 0; it < N_IT; it += 3) {
        if (wbase + it * 32 >= n_keys) break;                      // wave-uniform
        load_keys(it + 2, raw_c, kst_c);
        iteration(it, raw_a, kst_a);
        if (it + 1 >= N_IT || wbase + (it + 1) * 32 >= n_keys) break;
        load_keys(it + 3, raw_a, kst_a);
        iteration(it + 1, raw_b, kst_b);
        if (it + 2 >= N_IT || wbase + (it + 2) * 32 >= n_keys) break;
        load_keys(it + 4, raw_b, kst_b);
        iteration(it + 2, raw_c, kst_c);
    }
    // (never negative: the bit patterns order like the values as unsigned integers, NaNs on top)
    bmax = __builtin_bit_cast(float, wave_max_u32(__builtin_bit_cast(uint32_t, bmax)));
    if (lane == 0) bmax_sh[wave] = bmax;
    __syncthreads();
    if (tid == 0) {
        float m = bmax_sh[0];
#pragma unroll
        for (int i = 1; i < IB_THREADS / 64; i++) m = (bmax_sh[i] <= m) ? m : bmax_sh[i];
        beta_slots[(size_t)b * gridDim.x + wg] = m;
    }
    if (digit0 && tid < 256) {
        uint32_t c = 0u;
#pragma unroll
        for (int j = 0; j < 8; j++) c += hist0[tid * 8 + ((j + tid) & 7)];
        digit0[(size_t)b * digit0_row + (size_t)wg * 256 + tid] = c;
    }
}

// The reference's score of each candidate, written over its approximate one.  One workgroup
// = 16 candidates x 16 groups of four heads: lane j of a row of sixteen lanes holds candidate
// j's key, the row its four heads; the dot products run exactly as in indexer_scores_kernel
// (the q values of a head come to the FMAs through DPP row broadcasts); the 64 weighted terms
// of a candidate meet in LDS and one lane adds them in head order.
__global__ void __launch_bounds__(256)
indexer_rescore_kernel(const uint8_t *__restrict__ keys, const float *__restrict__ kscale,
                       int64_t key_bstride, int64_t kscale_bstride, int64_t n_keys,
                       const uint16_t *__restrict__ q, const float *__restrict__ w, int ih,
                       const int32_t *__restrict__ cand, int cap,
                       const IndexerBandRow *__restrict__ rows, float *__restrict__ scores,
                       float *__restrict__ cand_score) {   // [batch][cap]: the same scores in list order
    __shared__ float terms[16][65];
    const int b = blockIdx.y, tid = threadIdx.x;
    int c0 = blockIdx.x * 16;
    const int j = tid & 15, hg = tid >> 4;                          // candidate, head group
    // The list entry is fetched next to the row's state, not behind it (one round trip less in
    // front of the key's bytes): an entry past the end of the list is whatever the workspace
    // held, so it is clamped to a key of the row; what is computed for it is not stored.
    int64_t t_guess = cand[(size_t)b * cap + c0 + j];
    IndexerBandRow st;                                              // the two words in use, not the padding
    st.n_cand = rows[b].n_cand;
    st.fallback = rows[b].fallback;
    t_guess = t_guess < 0 ? 0 : (t_guess >= n_keys ? n_keys - 1 : t_guess);
    if (indexer_band_failed(st, cap)) {
        // the row did not fit the band: the workgroups of this launch score all of its keys
        // with the exact kernel's code instead
        for (int64_t block = blockIdx.x; block * IDX_THREADS < n_keys; block += gridDim.x) {
            indexer_exact_block(keys, kscale, key_bstride, kscale_bstride, n_keys, q, w, ih, scores, b, block);
            __syncthreads();
        }
        return;
    }
    // a list longer than the launch covers in one go (rare) takes further rounds
    for (; c0 < (int)st.n_cand; c0 += (int)gridDim.x * 16) {
    int64_t t = t_guess;                                            // (a slot past the end scores some key of the row: not stored)
    if (c0 != (int)blockIdx.x * 16) {
        t = cand[(size_t)b * cap + c0 + j];
        t = t < 0 ? 0 : (t >= n_keys ? n_keys - 1 : t);
    }
    const uint8_t *krow = keys + (size_t)b * key_bstride + (size_t)t * IB_HD;
    const float ks = kscale[(size_t)b * kscale_bstride + t];
    const uint16_t *qb = q + (size_t)b * ih * IB_HD;
    const float *wb = w + (size_t)b * ih;
    float e[IB_HD];
#pragma unroll
    for (int c = 0; c < IB_HD / 16; c++) {
        const u32x4 v = *(const u32x4 *)(krow + c * 16);
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const f32x2 lo = e4m3x2_to_f32<false>(v[jj]);
            const f32x2 hi = e4m3x2_to_f32<true>(v[jj]);
            e[c * 16 + jj * 4 + 0] = lo[0];
            e[c * 16 + jj * 4 + 1] = lo[1];
            e[c * 16 + jj * 4 + 2] = hi[0];
            e[c * 16 + jj * 4 + 3] = hi[1];
        }
    }
    // q of the group's four heads, all loads in flight at once: lane j holds q[h][16 c + j]
    float qall[4][IB_HD / 16], wh[4];
#pragma unroll
    for (int hh = 0; hh < 4; hh++) {
        const int h = hg * 4 + hh;
        const int hc = h < ih ? h : ih - 1;
#pragma unroll
        for (int c = 0; c < IB_HD / 16; c++) qall[hh][c] = bf16_to_f32(qb[(size_t)hc * IB_HD + 16 * c + j]);
        wh[hh] = wb[hc];
    }
#pragma unroll
    for (int hh = 0; hh < 4; hh++) {
        const int h = hg * 4 + hh;
        float qv[IB_HD / 16];
#pragma unroll
        for (int c = 0; c < IB_HD / 16; c++) qv[c] = qall[hh][c];
        // the loaded values pass through an (empty) VALU instruction: what the DPP reads below
        // is then ordinary data to the compiler, which sees to the waits; the two wait states a
        // DPP read needs after a VALU write are spent in the accumulator initialisation
#pragma unroll
        for (int c = 0; c < IB_HD / 16; c++) asm volatile("" : "+v"(qv[c]));
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
        asm volatile("s_nop 1" ::: "memory");
#pragma unroll
        for (int c = 0; c < IB_HD / 16; c++) {
#define CWICK_IB_FMA(acc, n)                                                                       \
    asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #n " row_mask:0xf bank_mask:0xf"       \
                 : "+v"(acc) : "v"(qv[c]), "v"(e[16 * c + n]))
            CWICK_IB_FMA(s0, 0);  CWICK_IB_FMA(s1, 1);  CWICK_IB_FMA(s2, 2);  CWICK_IB_FMA(s3, 3);
            CWICK_IB_FMA(s0, 4);  CWICK_IB_FMA(s1, 5);  CWICK_IB_FMA(s2, 6);  CWICK_IB_FMA(s3, 7);
            CWICK_IB_FMA(s0, 8);  CWICK_IB_FMA(s1, 9);  CWICK_IB_FMA(s2, 10); CWICK_IB_FMA(s3, 11);
            CWICK_IB_FMA(s0, 12); CWICK_IB_FMA(s1, 13); CWICK_IB_FMA(s2, 14); CWICK_IB_FMA(s3, 15);
#undef CWICK_IB_FMA
        }
        float d = (s0 + s1) + (s2 + s3);
        d = d * ks;
        d = d < 0.0f ? 0.0f : d;
        const float prod = d * wh[hh];
        terms[j][h] = h < ih ? prod : 0.0f;
    }
    __syncthreads();
    if (tid < 16 && c0 + tid < (int)st.n_cand) {
        float s = 0.0f;
        for (int h = 0; h < ih; h++) s = s + terms[tid][h];
        scores[(size_t)b * n_keys + cand[(size_t)b * cap + c0 + tid]] = s;
        cand_score[(size_t)b * cap + c0 + tid] = s;
    }
    __syncthreads();                                                // before the next round's terms
    }
}

// the approximate scores and the per-workgroup maxima of their error bound (the first stage of
// the banded select on its own; n_keys / IB_KEYS slots per row, rounded up)
int launch_indexer_approx(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys, const uint16_t *q_idx,
                          const float *w, int n_idx_heads, float *scores, float *beta_slots,
                          IndexerBandRow *rows, uint32_t *digit0_slices, size_t digit0_row_dwords,
                          hipStream_t s) {
    static_assert(IB_THREADS >= 256 && 1024 % IB_THREADS == 0, "a thread per first-digit bin, whole pieces of q per thread");
    CWICK_REQUIRE(keys && kscale && q_idx && w && scores && beta_slots && rows, "indexer_approx: null pointer");
    CWICK_REQUIRE(n_keys >= 1 && n_idx_heads >= 1 && n_idx_heads <= 64, "indexer_approx: shape out of range");
    CWICK_REQUIRE((uintptr_t)keys % 16 == 0 && key_bstride % 16 == 0 && (uintptr_t)q_idx % 16 == 0,
                  "indexer_approx: keys and q must be 16-byte aligned");
    const int n_wg = indexer_approx_slots(n_keys);
    {
        ProfKernel pk(CWICK_HIP_PROF_INDEXER_APPROX, s);
        pk.launch(indexer_approx_kernel, dim3(n_wg, batch), dim3(IB_THREADS), 0,
                  keys, kscale, key_bstride, kscale_bstride, n_keys, q_idx, w, n_idx_heads, scores, beta_slots, rows,
                  digit0_slices, digit0_row_dwords);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_indexer_banded(const uint8_t *keys, const float *kscale, int64_t key_bstride,
                          int64_t kscale_bstride, int batch, int64_t n_keys, const uint16_t *q_idx,
                          const float *w, int n_idx_heads, int64_t k, float *scores, int32_t *out_idx,
                          hipStream_t s) {
    CWICK_REQUIRE(keys && kscale && q_idx && w && scores && out_idx, "indexer_banded: null pointer");
    CWICK_REQUIRE(indexer_band_applies(n_keys, k, n_idx_heads), "indexer_banded: shape out of range");
    CWICK_REQUIRE((uintptr_t)keys % 16 == 0 && key_bstride % 16 == 0 && (uintptr_t)q_idx % 16 == 0,
                  "indexer_banded: keys and q must be 16-byte aligned");
    const int n_wg = indexer_approx_slots(n_keys);
    constexpr int cap = CWICK_INDEXER_BAND_CAP;
    // workspace: [the top-k's slices and states][beta slots][row states][+inf counts][candidate lists][their exact scores]
    const size_t topk_bytes = topk_mw_workspace_bytes(batch, n_keys);
    size_t off_beta = (topk_bytes + 255) & ~(size_t)255;
    size_t off_rows = off_beta + (((size_t)batch * n_wg * sizeof(float) + 255) & ~(size_t)255);
    size_t off_hi = off_rows + (((size_t)batch * sizeof(IndexerBandRow) + 255) & ~(size_t)255);
    size_t off_cand = off_hi + (size_t)batch * 64 * sizeof(uint32_t);
    size_t off_cs = off_cand + (size_t)batch * cap * sizeof(int32_t);
    const size_t total = off_cs + (size_t)batch * cap * sizeof(float);
    char *ws = (char *)workspace(s, total);
    if (!ws) return 0;                      // workspace() has recorded why
    float *beta_slots = (float *)(ws + off_beta);
    IndexerBandRow *rows = (IndexerBandRow *)(ws + off_rows);
    uint32_t *hi_count = (uint32_t *)(ws + off_hi);
    int32_t *cand = (int32_t *)(ws + off_cand);
    float *cand_score = (float *)(ws + off_cs);
    {
    ProfScope ps(CWICK_HIP_PROF_INDEXER, s);
    if (!launch_indexer_approx(keys, kscale, key_bstride, kscale_bstride, batch, n_keys, q_idx, w, n_idx_heads,
                               scores, beta_slots, rows, (uint32_t *)ws, topk_mw_band_row_dwords(n_keys), s))
        return 0;
    if (!launch_topk_band_classify(scores, batch, n_keys, k, (uint32_t *)ws, beta_slots, n_wg, cand, cap, rows,
                                   hi_count, true, s))
        return 0;
    // Sixteen candidates per workgroup and round.  About one workgroup per CU over all rows: a
    // list is a few hundred entries, and the launch of workgroups that find nothing to do is what
    // this kernel's time was mostly made of (256 per row: 7.3 us, 32 per row: 5.4 us for 8 rows).
    int rescore_wgs = num_cus() / batch;
    rescore_wgs = rescore_wgs < 8 ? 8 : (rescore_wgs > cap / 16 ? cap / 16 : rescore_wgs);
    indexer_rescore_kernel<<<dim3(rescore_wgs, batch), 256, 0, s>>>(
        keys, kscale, key_bstride, kscale_bstride, n_keys, q_idx, w, n_idx_heads, cand, cap, rows, scores, cand_score);
    CWICK_HIP_CALL(hipGetLastError());
    }
    return launch_topk_band_finish(scores, batch, n_keys, k, cand, cand_score, cap, rows, hi_count, out_idx, s);
}

}  // namespace cwick
