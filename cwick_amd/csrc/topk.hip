// topk.hip -- exact top-k by radix select (ds_topk_scores, src/ds_ops.c:310-338,
// under the contract of src/ds_ops.h:110-112; the threshold-then-ties selector
// of src/attention.c:585-598 computes the same set).
//
// Order: (score descending, index ascending); the k best are written in
// ascending index order.  Scores map to order-preserving 32-bit keys
// (-0.0 folded into +0.0, NaN below everything), so the selection is integer
// work and bit-exact by construction:
//
//   1. four 8-bit histogram passes, most significant digit first, find the key
//      T of the k-th best element and r = how many elements equal to T belong
//      to the selection;
//   2. one ordered pass emits every index with key > T and the first r indices
//      with key == T, in ascending index order, through a block-wide scan.
//
// Rows of 16 K to 128 K scores (the indexer's case) are split over many
// workgroups that meet at kernel boundaries: four digit-histogram launches and
// one ordered emit (see topk_mw_hist_kernel below).  Other rows take one
// workgroup of 1024 threads.  Up to 65536 scores
// are read once: every thread keeps its 64 consecutive keys in
// registers for all five passes, the first histogram pass counts into one of 32
// lane-indexed copies (scores cluster in a few exponent buckets, and same-address
// LDS atomics serialise), and the ordered emit places elements with ballots
// inside a wave and one pass over the wave totals.  Longer rows take the streaming kernel,
// which reads the row five times from L2.  Rows past min(k, n) are filled with -1.
#include "common.hpp"
#include "topk_row.hpp"

namespace cwick {

__global__ void __launch_bounds__(TOPK_THREADS)
topk_radix_kernel(const float *__restrict__ scores, int64_t n, int64_t k, int32_t *__restrict__ out) {
    topk_radix_row(scores + (size_t)blockIdx.x * n, n, k, out + (size_t)blockIdx.x * k);
}

// ---- rows that fit the register file (topk_radix_reg_row, topk_row.hpp) ----
template <int EPT>
__global__ void __launch_bounds__(TOPK_THREADS)
topk_radix_reg_kernel(const float *__restrict__ scores, int64_t n, int64_t k,
                      int32_t *__restrict__ out) {
    topk_radix_reg_row<EPT>(scores + (size_t)blockIdx.x * n, n, k, out + (size_t)blockIdx.x * k);
}

// ---- rows of 16 K .. 128 K scores: many workgroups per row ----
// One workgroup of TOPK_MW_THREADS takes TOPK_MW_KEYS consecutive scores, so a batch of eight
// 64 K rows fills the chip instead of eight CUs.  Workgroups of a row meet only at kernel
// boundaries: kernel p (p = 0..3) counts the p-th digit of the keys that match the digits
// chosen so far into the workgroup's own 256-bin slice (no atomics across workgroups, nothing
// to clear), and every workgroup of kernel p+1 first adds up the slices of its row and picks
// digit p exactly as the single-workgroup kernels do.  The last kernel knows T and the tie
// budget r, derives the output offset of its workgroup from the slices (the keys above T of
// an earlier workgroup are those that left the chosen path at some digit with a larger bin)
// and writes its indices in ascending order.
constexpr int TOPK_MW_THREADS = 256;
constexpr int TOPK_MW_EPT = 8;
constexpr int TOPK_MW_KEYS = TOPK_MW_THREADS * TOPK_MW_EPT;     // 2048
constexpr int TOPK_MW_MAX_WGS = 64;                              // per row

struct TopkMwState { uint32_t prefix, remaining; };

// sum of p[w * 256] over w < count with thirty-two loads in flight (the slices sit in L2: a
// dependent chain of loads would cost a round trip each, and so does every further batch)
__device__ __forceinline__ uint32_t topk_mw_colsum(const uint32_t *__restrict__ p, int count) {
    uint32_t c = 0u;
    for (int w0 = 0; w0 < count; w0 += 32) {
        uint32_t v[32];
#pragma unroll
        for (int j = 0; j < 32; j++) {
            const int w = w0 + j < count ? w0 + j : count - 1;      // clamped, not guarded: a guarded load is a branch
            v[j] = p[(size_t)w * 256];
        }
#pragma unroll
        for (int j = 0; j < 32; j++) c += w0 + j < count ? v[j] : 0u;
    }
    return c;
}

// adds up the slices of pass p of this row, picks the digit that holds the remaining-th best
// key; all threads return the new (prefix, remaining)
__device__ __forceinline__ TopkMwState
topk_mw_pick(const uint32_t *__restrict__ slices, int n_wg, int shift, TopkMwState st,
             uint32_t *hist /* LDS, 256 */, TopkMwState *sh_state /* LDS */) {
    const int tid = threadIdx.x;
    hist[tid] = topk_mw_colsum(slices + tid, n_wg);
    __syncthreads();
    if (tid < 64) {
        // walk the 256 buckets from the largest digit down; lane b owns buckets 255-4b .. 252-4b
        uint32_t cc[4], sum = 0u;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            cc[j] = hist[255 - (tid * 4 + j)];
            sum += cc[j];
        }
        uint32_t inc = wave_scan_u32(sum);
        uint32_t before = inc - sum;       // elements in strictly larger buckets
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (before < st.remaining && st.remaining <= before + cc[j]) {
                sh_state->prefix = st.prefix | ((uint32_t)(255 - (tid * 4 + j)) << shift);
                sh_state->remaining = st.remaining - before;
            }
            before += cc[j];
        }
    }
    __syncthreads();
    const TopkMwState out = *sh_state;
    __syncthreads();
    return out;
}

// workspace of a row: slices[4][sl][256], then state[4], then above[3][n_wg].  sl >= n_wg slices
// are laid out per pass; passes 1..3 use n_wg of them, pass 0 uses n_s0: its counts may come
// from another kernel that cut the row into more pieces (each an equal share of a workgroup's
// keys here).
__global__ void __launch_bounds__(TOPK_MW_THREADS)
topk_mw_hist_kernel(const float *__restrict__ scores, int64_t n, int64_t k, int n_wg, int pass,
                    uint32_t *__restrict__ ws, size_t ws_row, int sl, int n_s0) {
    __shared__ uint32_t hist[256];
    __shared__ uint32_t hist8[256 * 8];
    __shared__ TopkMwState sh_state;
    const int row = blockIdx.y, wg = blockIdx.x, tid = threadIdx.x;
    uint32_t *slices = ws + (size_t)row * ws_row;
    TopkMwState *state = (TopkMwState *)(slices + (size_t)4 * sl * 256);
    const int64_t kk = k < n ? k : n;
    // the workgroup's scores: issued first, they travel while the previous digit is picked
    const float *sc = scores + (size_t)row * n;
    const int64_t base = (int64_t)wg * TOPK_MW_KEYS;
    float v[TOPK_MW_EPT];
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        v[j] = i < n ? sc[i] : 0.0f;
    }
    TopkMwState st{0u, (uint32_t)kk};
    if (pass > 0) {
        if (pass > 1) st = state[pass - 1];
        // this workgroup's own bin of the previous pass: issued before the pick, used after it
        uint32_t own_prev;
        if (pass == 1) {
            const int per = (n_s0 + n_wg - 1) / n_wg;             // pass-0 slices per workgroup
            own_prev = 0u;
            for (int j = 0; j < per; j++)
                if (wg * per + j < n_s0) own_prev += slices[((size_t)wg * per + j) * 256 + tid];
        } else {
            own_prev = slices[((size_t)(pass - 1) * sl + wg) * 256 + tid];
        }
        st = topk_mw_pick(slices + (size_t)(pass - 1) * sl * 256, pass == 1 ? n_s0 : n_wg, 32 - 8 * pass, st, hist, &sh_state);
        if (wg == 0 && tid == 0) state[pass] = st;
        // how many of this workgroup's keys left the chosen path at the previous digit with a
        // larger bin, i.e. lie above T whatever the later digits are: the emit kernel adds
        // these up over the workgroups before it
        const uint32_t dig = (st.prefix >> (32 - 8 * pass)) & 0xFFu;
        uint32_t above = (uint32_t)tid > dig ? own_prev : 0u;
        above = wave_sum_u32(above);
        if ((tid & 63) == 0) hist8[tid >> 6] = above;
        __syncthreads();
        if (tid == 0) {
            uint32_t *abv = (uint32_t *)(state + 4);
            abv[(size_t)(pass - 1) * n_wg + wg] = hist8[0] + hist8[1] + hist8[2] + hist8[3];
        }
        __syncthreads();
    }
    const int shift = 24 - 8 * pass;
    const uint32_t mask = pass == 0 ? 0u : (0xFFFFFFFFu << (32 - 8 * pass));
#pragma unroll
    for (int j = 0; j < 8; j++) hist8[tid + 256 * j] = 0u;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        if (i < n) {
            const uint32_t key = topk_key(v[j]);
            // eight copies picked by lane: scores cluster in a few buckets and same-address
            // LDS atomics of one instruction serialise
            if ((key & mask) == st.prefix) atomicAdd(&hist8[((key >> shift) & 0xFFu) * 8 + (tid & 7)], 1u);
        }
    }
    __syncthreads();
    uint32_t c = 0u;
#pragma unroll
    for (int j = 0; j < 8; j++) c += hist8[tid * 8 + ((j + tid) & 7)];
    slices[((size_t)pass * sl + wg) * 256 + tid] = c;
}

__global__ void __launch_bounds__(TOPK_MW_THREADS)
topk_mw_emit_kernel(const float *__restrict__ scores, int64_t n, int64_t k, int n_wg,
                    const uint32_t *__restrict__ ws, size_t ws_row, int sl, int32_t *__restrict__ out) {
    __shared__ uint32_t hist[256];
    __shared__ TopkMwState sh_state;
    __shared__ uint32_t sh_red[2][TOPK_MW_THREADS / 64];
    __shared__ uint32_t sh_gt[TOPK_MW_EPT][TOPK_MW_THREADS / 64], sh_eq[TOPK_MW_EPT][TOPK_MW_THREADS / 64];
    const int row = blockIdx.y, wg = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t *slices = ws + (size_t)row * ws_row;
    const TopkMwState *state = (const TopkMwState *)(slices + (size_t)4 * sl * 256);
    int32_t *dst = out + (size_t)row * k;
    const int64_t kk = k < n ? k : n;
    if (wg == 0)
        for (int64_t i = kk + tid; i < k; i += TOPK_MW_THREADS) dst[i] = -1;
    const float *sc = scores + (size_t)row * n;
    const int64_t base = (int64_t)wg * TOPK_MW_KEYS;
    uint32_t keys[TOPK_MW_EPT];                 // issued first: they travel while T is picked
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        keys[j] = i < n ? topk_key(sc[i]) : 0u;
    }
    // keys above T in the workgroups before this one, part 1: bin b of pass p of workgroup w
    // counts keys that match the chosen digits 0..p-1 and have digit p = b; they are above T if
    // b is larger than the chosen digit p
    const TopkMwState st3 = state[3];
    uint32_t gt = 0u, eq = 0u;
    {   // digits 0..2: the histogram kernels left one count per workgroup and digit
        const uint32_t *abv = (const uint32_t *)(state + 4);
        const int p = tid / TOPK_MW_MAX_WGS, w = tid % TOPK_MW_MAX_WGS;     // 3 x 64 <= 256 threads
        if (p < 3 && w < wg) gt = abv[(size_t)p * n_wg + w];
    }
    const TopkMwState st = topk_mw_pick(slices + (size_t)3 * sl * 256, n_wg, 0, st3, hist, &sh_state);
    const uint32_t T = st.prefix, r = st.remaining;   // r ties belong to the selection
    {   // part 2: the last digit; equal to T if it is the digit itself
        const uint32_t dig = T & 0xFFu;
        const bool above = (uint32_t)tid > dig, same = (uint32_t)tid == dig;
        const uint32_t c = topk_mw_colsum(slices + (size_t)3 * sl * 256 + tid, (above || same) ? wg : 0);
        if (above) gt += c;
        if (same) eq += c;
    }
    gt = wave_sum_u32(gt);
    eq = wave_sum_u32(eq);
    if (lane == 0) {
        sh_red[0][wave] = gt;
        sh_red[1][wave] = eq;
    }
    // own keys, in index order: element (j, tid) is index base + 256 j + tid, so the order of
    // the workgroup is (j, wave, lane).  Ballots give the counts of every (j, wave) cell, one
    // walk over the 32 cells the position of this wave's cells.
    uint64_t m_gt[TOPK_MW_EPT], m_eq[TOPK_MW_EPT];
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        m_gt[j] = __ballot(i < n && keys[j] > T);
        m_eq[j] = __ballot(i < n && keys[j] == T);
        if (lane == 0) {
            sh_gt[j][wave] = (uint32_t)__builtin_popcountll(m_gt[j]);
            sh_eq[j][wave] = (uint32_t)__builtin_popcountll(m_eq[j]);
        }
    }
    __syncthreads();
    uint32_t gt_before = 0u, eq_before = 0u;
#pragma unroll
    for (int w = 0; w < TOPK_MW_THREADS / 64; w++) {
        gt_before += sh_red[0][w];
        eq_before += sh_red[1][w];
    }
    uint32_t run_pos = gt_before + (eq_before < r ? eq_before : r), run_eq = eq_before;
    uint32_t my_pos[TOPK_MW_EPT], my_eq[TOPK_MW_EPT];
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++)
#pragma unroll
        for (int w = 0; w < TOPK_MW_THREADS / 64; w++) {
            const uint32_t g = sh_gt[j][w], e = sh_eq[j][w];
            if (w == wave) {
                my_pos[j] = run_pos;
                my_eq[j] = run_eq;
            }
            run_pos += g + (run_eq >= r ? 0u : (r - run_eq < e ? r - run_eq : e));
            run_eq += e;
        }
    const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        const bool is_gt = (m_gt[j] >> lane) & 1, is_eq = (m_eq[j] >> lane) & 1;
        // ties first get their rank, then every taken element its slot
        const uint32_t my_eq_rank = my_eq[j] + (uint32_t)__builtin_popcountll(m_eq[j] & lt);
        const bool take = is_gt || (is_eq && my_eq_rank < r);
        const uint64_t m_take = __ballot(take);
        if (take) dst[my_pos[j] + (uint32_t)__builtin_popcountll(m_take & lt)] = (int32_t)i;
    }
}

// The select half of the banded indexer (indexer_band.hip): T is the k-th largest approximate
// score, beta the largest error bound of the row; scores above T + 2 beta become +inf, scores
// below T - 2 beta become -inf, the rest stay and are listed for exact rescoring.
__global__ void __launch_bounds__(TOPK_MW_THREADS)
topk_mw_classify_kernel(float *__restrict__ scores, int64_t n, int64_t k, int n_wg,
                        const uint32_t *__restrict__ ws, size_t ws_row,
                        const float *__restrict__ beta_slots, int n_beta,
                        int32_t *__restrict__ cand, int cap, IndexerBandRow *__restrict__ rows, int sl,
                        uint32_t *__restrict__ hi_count) {   // [row][TOPK_MW_MAX_WGS]: keys set to +inf per workgroup
    __shared__ uint32_t hist[256];
    __shared__ TopkMwState sh_state;
    __shared__ float sh_beta[TOPK_MW_THREADS / 64];
    const int row = blockIdx.y, wg = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const uint32_t *slices = ws + (size_t)row * ws_row;
    const TopkMwState *state = (const TopkMwState *)(slices + (size_t)4 * sl * 256);
    float *sc = scores + (size_t)row * n;
    const int64_t base = (int64_t)wg * TOPK_MW_KEYS;
    float v[TOPK_MW_EPT];
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        v[j] = i < n ? sc[i] : 0.0f;
    }
    float beta = tid < n_beta ? beta_slots[(size_t)row * n_beta + tid] : 0.0f;
    // (bounds are never negative: as unsigned integers their bit patterns order like the values,
    // with every NaN on top, where it sticks)
    beta = __builtin_bit_cast(float, wave_max_u32(__builtin_bit_cast(uint32_t, beta)));
    if (lane == 0) sh_beta[tid >> 6] = beta;
    // two digits are enough here: the k-th largest key lies in the bucket [T_lo, T_hi] of the
    // 16-bit prefix (sign, exponent, seven bits of the fraction); at most k-1 keys lie above the
    // bucket and at least k in or above it, which is all the argument needs.  The bucket is 2^-7
    // of the threshold wide, about as much as beta on the indexer's scores: a third digit pass
    // (5.4 us) would trim the candidate list by a quarter, which costs the rescoring less.
    const TopkMwState st = topk_mw_pick(slices + (size_t)1 * sl * 256, n_wg, 16, state[1], hist, &sh_state);
    beta = sh_beta[0];
#pragma unroll
    for (int i = 1; i < TOPK_MW_THREADS / 64; i++) beta = (sh_beta[i] <= beta) ? beta : sh_beta[i];
    // the floats behind the order keys
    auto key_float = [](uint32_t key) -> float {
        return __builtin_bit_cast(float, (key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
    };
    const float T_lo = key_float(st.prefix), T_hi = key_float(st.prefix | 0xFFFFu);
    const bool ok = (st.prefix >> 16) != 0u && beta >= 0.0f && beta < INFINITY && T_lo == T_lo && T_hi == T_hi;
    if (!ok) {
        if (wg == 0 && tid == 0) rows[row].fallback = 1u;
        return;
    }
    const float hi = T_hi + 2.004f * beta, lo = T_lo - 2.004f * beta;
    // candidates take a place in the workgroup first (LDS counter), the workgroup then takes its
    // run of the row's list with one atomic: a few hundred returning atomics on one address from
    // all over the chip would queue up behind each other
    uint32_t *wg_count = &hist[0], *wg_base = &hist[1], *wg_hi = &hist[2];   // the pick is done with hist
    if (tid == 0) *wg_count = 0u, *wg_hi = 0u;
    __syncthreads();
    uint32_t is_cand = 0u, n_hi = 0u;
#pragma unroll
    for (int j = 0; j < TOPK_MW_EPT; j++) {
        const int64_t i = base + j * TOPK_MW_THREADS + tid;
        if (i < n) {
            if (v[j] > hi) sc[i] = INFINITY, n_hi++;
            else if (v[j] < lo) sc[i] = -INFINITY;
            else is_cand |= 1u << j;
        }
    }
    uint32_t my_first = 0u;
    const uint32_t mine = (uint32_t)__builtin_popcount(is_cand);
    if (mine) my_first = atomicAdd(wg_count, mine);
    // (one atomic per wave: a few dozen on one address from one instruction queue up)
    n_hi = wave_sum_u32(n_hi);
    if (lane == 0 && n_hi) atomicAdd(wg_hi, n_hi);
    __syncthreads();
    if (tid == 0) {
        *wg_base = *wg_count ? atomicAdd(&rows[row].n_cand, *wg_count) : 0u;
        hi_count[(size_t)row * TOPK_MW_MAX_WGS + wg] = *wg_hi;
    }
    __syncthreads();
    if (mine) {
        uint32_t slot = *wg_base + my_first;
#pragma unroll
        for (int j = 0; j < TOPK_MW_EPT; j++)
            if (is_cand >> j & 1u) {
                if (slot < (uint32_t)cap) cand[(size_t)row * cap + slot] = (int32_t)(base + j * TOPK_MW_THREADS + tid);
                slot++;
            }
    }
}

// ---- the end of the banded select: no second radix select over the whole row ----
// After the classify kernel and the exact rescoring a row consists of keys that are certainly
// selected (+inf, hi_count[w] of them in workgroup w's stretch), keys that are certainly not
// (-inf) and at most `cap` candidates with their exact scores.  The selection is the +inf keys
// and the best need = k - (number of +inf keys) candidates, ties to the smaller index as
// everywhere.  The workgroups of a row are those of the classify kernel (2048 keys each).  Every
// one of them ranks the candidates for itself (a radix select on the order keys of their
// scores, and, if the need-th key has ties that do not all fit, a second one on the inverted
// indices of the tied): the list is at most 4096 entries, and knowing the outcome everywhere
// saves a launch, the write-back of the decisions and the atomics that would count them.  A
// workgroup then starts writing after the +inf keys of the stretches before it (hi_count) and
// the chosen candidates among them (counted out of the list), and writes its own keys that
// are +inf or chosen candidates in index order.
constexpr int TOPK_BAND_THREADS = 1024;
constexpr int TOPK_BAND_EPT = CWICK_INDEXER_BAND_CAP / TOPK_BAND_THREADS;     // 4

struct TopkBandShared {
    uint32_t hist[256];
    uint32_t mn[TOPK_BAND_THREADS / 64], mx[TOPK_BAND_THREADS / 64], cnt[TOPK_BAND_THREADS / 64];
    uint32_t digit, remaining, eq;
};

// Radix select inside one workgroup over up to four 32-bit values per thread (`act` marks
// the live ones): T = the need-th largest, r = how many of the values equal to T belong to
// the need largest, e = how many values equal T.  1 <= need <= number of live values.  The
// values of a candidate list agree in their leading bits (scores from a narrow band, indices
// from one row), and digits that all values share would put every LDS atomic on one word: the
// passes start at the first byte in which the largest and the smallest value differ.
__device__ __forceinline__ void topk_band_select(const uint32_t (&val)[TOPK_BAND_EPT], uint32_t act, uint32_t need,
                                                 TopkBandShared &sh, uint32_t &T, uint32_t &r, uint32_t &e) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t mn = 0xFFFFFFFFu, mx = 0u, cnt = (uint32_t)__builtin_popcount(act);
#pragma unroll
    for (int j = 0; j < TOPK_BAND_EPT; j++)
        if (act >> j & 1u) {
            mn = val[j] < mn ? val[j] : mn;
            mx = val[j] > mx ? val[j] : mx;
        }
    mn = wave_min_u32(mn);
    mx = wave_max_u32(mx);
    cnt = wave_sum_u32(cnt);
    if (lane == 0) sh.mn[wave] = mn, sh.mx[wave] = mx, sh.cnt[wave] = cnt;
    __syncthreads();
    cnt = 0u;
#pragma unroll
    for (int w = 0; w < TOPK_BAND_THREADS / 64; w++) {
        mn = sh.mn[w] < mn ? sh.mn[w] : mn;
        mx = sh.mx[w] > mx ? sh.mx[w] : mx;
        cnt += sh.cnt[w];
    }
    const uint32_t diff = mn ^ mx;
    const int passes = diff ? (31 - __builtin_clz(diff)) / 8 + 1 : 0;
    uint32_t mask = passes >= 4 ? 0u : 0xFFFFFFFFu << (8 * passes);
    uint32_t prefix = mx & mask, remaining = need;
    e = cnt;                                              // all values equal: every one is a tie
    for (int p = passes - 1; p >= 0; p--) {
        const int shift = 8 * p;
        if (tid < 256) sh.hist[tid] = 0u;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < TOPK_BAND_EPT; j++)
            if ((act >> j & 1u) && (val[j] & mask) == prefix) atomicAdd(&sh.hist[(val[j] >> shift) & 0xFFu], 1u);
        __syncthreads();
        if (tid < 64) {
            // walk the 256 buckets from the largest digit down; lane b owns buckets 255-4b .. 252-4b
            uint32_t c[4], sum = 0u;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                c[j] = sh.hist[255 - (tid * 4 + j)];
                sum += c[j];
            }
            uint32_t inc = wave_scan_u32(sum);
            uint32_t before = inc - sum;   // values in strictly larger buckets
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (before < remaining && remaining <= before + c[j]) {
                    sh.digit = (uint32_t)(255 - (tid * 4 + j));
                    sh.remaining = remaining - before;
                    sh.eq = c[j];
                }
                before += c[j];
            }
        }
        __syncthreads();
        prefix |= sh.digit << shift;
        remaining = sh.remaining;
        e = sh.eq;
        mask |= 0xFFu << shift;
    }
    __syncthreads();                                      // sh is free again
    T = prefix;
    r = remaining;
}

__global__ void __launch_bounds__(TOPK_BAND_THREADS)
topk_band_finish_kernel(const float *__restrict__ scores, int64_t n, int64_t k, int n_wg,
                        const int32_t *__restrict__ cand, const float *__restrict__ cand_score, int cap,
                        const IndexerBandRow *__restrict__ rows, const uint32_t *__restrict__ hi_count,
                        int32_t *__restrict__ out) {
    constexpr int KPT = TOPK_MW_KEYS / TOPK_BAND_THREADS;           // own keys per thread: 2
    __shared__ TopkBandShared sh;
    __shared__ uint32_t sh_hi, sh_before;
    __shared__ uint32_t sh_cnt[KPT][TOPK_BAND_THREADS / 64];
    const int row = blockIdx.y, wg = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const float *sc = scores + (size_t)row * n;
    int32_t *dst = out + (size_t)row * k;
    const int64_t base = (int64_t)wg * TOPK_MW_KEYS;
    // every load first, one round trip: the whole candidate list whatever its length (the
    // thread count times four is its capacity), this stretch's scores, the counts, the row state
    int32_t idx[TOPK_BAND_EPT];
    float val[TOPK_BAND_EPT], v[KPT];
#pragma unroll
    for (int j = 0; j < TOPK_BAND_EPT; j++) {
        idx[j] = cand[(size_t)row * cap + tid + TOPK_BAND_THREADS * j];
        val[j] = cand_score[(size_t)row * cap + tid + TOPK_BAND_THREADS * j];
    }
#pragma unroll
    for (int j = 0; j < KPT; j++) {
        const int64_t i = base + j * TOPK_BAND_THREADS + tid;
        v[j] = sc[i < n ? i : n - 1];
    }
    const uint32_t hi_part = tid < n_wg ? hi_count[(size_t)row * TOPK_MW_MAX_WGS + tid] : 0u;
    IndexerBandRow st;                                          // the two words in use, not the padding
    st.n_cand = rows[row].n_cand;
    st.fallback = rows[row].fallback;
    if (indexer_band_failed(st, cap)) {
        // the row did not fit the band: its scores are the exact kernel's by now, and its first
        // workgroup selects from all of them
        if (wg == 0) topk_radix_row(sc, n, k, dst);
        return;
    }
    const int n_cand = (int)st.n_cand;
    static_assert(TOPK_MW_MAX_WGS <= 64, "the first wave holds a count per stretch");
    if (tid < 64) {                                             // the first wave adds up the stretches' counts
        const uint32_t all = wave_sum_u32(hi_part), before = wave_sum_u32(tid < wg ? hi_part : 0u);
        if (tid == 0) sh_hi = all, sh_before = before;
    }
    uint32_t key[TOPK_BAND_EPT], inv[TOPK_BAND_EPT], live = 0u;
#pragma unroll
    for (int j = 0; j < TOPK_BAND_EPT; j++) {
        key[j] = topk_key(val[j]);
        inv[j] = ~(uint32_t)idx[j];
        if (tid + TOPK_BAND_THREADS * j < n_cand) live |= 1u << j;
    }
    __syncthreads();
    const int64_t want = k - (int64_t)sh_hi;
    const uint32_t need = want <= 0 ? 0u : (want < n_cand ? (uint32_t)want : (uint32_t)n_cand);
    uint32_t T = 0u, r = 0u, e = 0u, T2 = 0u;
    if (need > 0u) {                                            // uniform
        topk_band_select(key, live, need, sh, T, r, e);
        if (r < e) {                                            // uniform: ties at T, the smaller indices win
            uint32_t tied = 0u, r2, e2;
#pragma unroll
            for (int j = 0; j < TOPK_BAND_EPT; j++)
                if ((live >> j & 1u) && key[j] == T) tied |= 1u << j;
            topk_band_select(inv, tied, r, sh, T2, r2, e2);
        }
    }
    // a candidate is chosen if it is above the need-th, or ties with it and has a small enough index
    auto chosen = [&](uint32_t kk, uint32_t ii) { return need > 0u && (kk > T || (kk == T && ii >= T2)); };
    // chosen candidates in the stretches before this one
    uint32_t earlier = 0u;
#pragma unroll
    for (int j = 0; j < TOPK_BAND_EPT; j++)
        if ((live >> j & 1u) && (int64_t)idx[j] < base && chosen(key[j], inv[j])) earlier++;
    // (added up per wave first: hundreds of atomics on one address would queue up)
    earlier = wave_sum_u32(earlier);
    if (lane == 0 && earlier) atomicAdd(&sh_before, earlier);
    // own keys: +inf is in, -inf is out, anything else is a candidate with its exact score.
    // Element (j, tid) is index base + 1024 j + tid: the order of the workgroup is (j, wave, lane)
    uint64_t m[KPT];
#pragma unroll
    for (int j = 0; j < KPT; j++) {
        const int64_t i = base + j * TOPK_BAND_THREADS + tid;
        const bool in = i < n && (v[j] == INFINITY || (v[j] != -INFINITY && chosen(topk_key(v[j]), ~(uint32_t)i)));
        m[j] = __ballot(in);
        if (lane == 0) sh_cnt[j][wave] = (uint32_t)__builtin_popcountll(m[j]);
    }
    __syncthreads();
    uint32_t run = sh_before, my_pos[KPT];
#pragma unroll
    for (int j = 0; j < KPT; j++)
#pragma unroll
        for (int w = 0; w < TOPK_BAND_THREADS / 64; w++) {
            if (w == wave) my_pos[j] = run;
            run += sh_cnt[j][w];
        }
    const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int j = 0; j < KPT; j++)
        if ((m[j] >> lane) & 1) {
            const uint32_t pos = my_pos[j] + (uint32_t)__builtin_popcountll(m[j] & lt);
            if (pos < (uint32_t)k) dst[pos] = (int32_t)(base + j * TOPK_BAND_THREADS + tid);
        }
}

// a row's workspace in dwords: slices[4][sl][256], four states, above[3][n_wg] (+ padding to
// keep the rows 8-byte aligned)
static size_t topk_mw_row_dwords(int64_t n_wg, int64_t sl) { return (size_t)4 * sl * 256 + 2 * 4 + (size_t)((3 * n_wg + 1) & ~(int64_t)1); }
static int64_t topk_mw_wgs(int64_t n) { return (n + TOPK_MW_KEYS - 1) / TOPK_MW_KEYS; }
// the banded select's layout: room for the approximate kernel's pass-0 slices
static int64_t topk_mw_band_sl(int64_t n) {
    const int64_t n_wg = topk_mw_wgs(n), n_s0 = indexer_approx_slots(n);
    return n_wg > n_s0 ? n_wg : n_s0;
}
size_t topk_mw_band_row_dwords(int64_t n) { return topk_mw_row_dwords(topk_mw_wgs(n), topk_mw_band_sl(n)); }

// enough for either layout
size_t topk_mw_workspace_bytes(int batch, int64_t n) {
    return (size_t)batch * topk_mw_band_row_dwords(n) * sizeof(uint32_t);
}

int launch_topk_band_classify(float *scores, int batch, int64_t n, int64_t k, uint32_t *ws,
                              const float *beta_slots, int n_beta, int32_t *cand, int cap,
                              IndexerBandRow *rows, uint32_t *hi_count, bool digit0_done, hipStream_t s) {
    const int64_t n_wg = topk_mw_wgs(n);
    CWICK_REQUIRE(n_wg >= 8 && n_wg <= TOPK_MW_MAX_WGS && n_beta <= TOPK_MW_THREADS,
                  "topk_band_classify: n %lld out of range", (long long)n);
    const int sl = (int)topk_mw_band_sl(n);
    const int n_s0 = digit0_done ? indexer_approx_slots(n) : (int)n_wg;
    CWICK_REQUIRE(n_s0 <= 2 * TOPK_MW_MAX_WGS, "topk_band_classify: %d first-digit slices", n_s0);
    const size_t ws_row = topk_mw_band_row_dwords(n);
    const dim3 grid((unsigned)n_wg, (unsigned)batch);
    for (int pass = digit0_done ? 1 : 0; pass < 2; pass++)
        topk_mw_hist_kernel<<<grid, TOPK_MW_THREADS, 0, s>>>(scores, n, k, (int)n_wg, pass, ws, ws_row, sl, n_s0);
    topk_mw_classify_kernel<<<grid, TOPK_MW_THREADS, 0, s>>>(scores, n, k, (int)n_wg, ws, ws_row, beta_slots,
                                                            n_beta, cand, cap, rows, sl, hi_count);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_topk_band_finish(float *scores, int batch, int64_t n, int64_t k, const int32_t *cand,
                            const float *cand_score, int cap, const IndexerBandRow *rows, uint32_t *hi_count,
                            int32_t *out_idx, hipStream_t s) {
    static_assert(TOPK_BAND_EPT * TOPK_BAND_THREADS == CWICK_INDEXER_BAND_CAP, "a workgroup holds the whole list");
    static_assert(TOPK_BAND_THREADS == TOPK_THREADS, "the workgroup runs the one-workgroup select for rows off the band");
    static_assert(TOPK_MW_KEYS % TOPK_BAND_THREADS == 0, "whole keys per thread");
    const int64_t n_wg = topk_mw_wgs(n);
    CWICK_REQUIRE(n_wg >= 8 && n_wg <= TOPK_MW_MAX_WGS && cap == CWICK_INDEXER_BAND_CAP && k < n,
                  "topk_band_finish: n %lld out of range", (long long)n);
    ProfScope ps(CWICK_HIP_PROF_TOPK, s);
    topk_band_finish_kernel<<<dim3((unsigned)n_wg, (unsigned)batch), TOPK_BAND_THREADS, 0, s>>>(
        scores, n, k, (int)n_wg, cand, cand_score, cap, rows, hi_count, out_idx);
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_topk(const float *scores, int batch, int64_t n, int64_t k, int32_t *out_idx,
                hipStream_t s) {
    CWICK_REQUIRE(scores && out_idx, "topk: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535, "topk: batch %d", batch);
    CWICK_REQUIRE(n >= 1 && n <= ((int64_t)1 << 24), "topk: n %lld (1..2^24)", (long long)n);
    CWICK_REQUIRE(k >= 1 && k <= 65536, "topk: k %lld (1..65536)", (long long)k);
    const int64_t n_wg = topk_mw_wgs(n);
    if (n_wg >= 8 && n_wg <= TOPK_MW_MAX_WGS) {
        const size_t ws_row = topk_mw_row_dwords(n_wg, n_wg);       // dwords: slices, four states, above counts
        // its own slot: the callers that select among block scores keep those in the main one
        uint32_t *ws = (uint32_t *)workspace(s, (size_t)batch * ws_row * sizeof(uint32_t), WS_NESTED);
        if (!ws) return 0;                      // workspace() has recorded why
        const dim3 grid((unsigned)n_wg, (unsigned)batch);
        ProfScope ps(CWICK_HIP_PROF_TOPK, s);
        for (int pass = 0; pass < 4; pass++)
            topk_mw_hist_kernel<<<grid, TOPK_MW_THREADS, 0, s>>>(scores, n, k, (int)n_wg, pass, ws, ws_row, (int)n_wg, (int)n_wg);
        topk_mw_emit_kernel<<<grid, TOPK_MW_THREADS, 0, s>>>(scores, n, k, (int)n_wg, ws, ws_row, (int)n_wg, out_idx);
        CWICK_HIP_CALL(hipGetLastError());
        return 1;
    }
    {
        ProfScope ps(CWICK_HIP_PROF_TOPK, s);
        if (n <= (int64_t)TOPK_THREADS)
            topk_radix_reg_kernel<1><<<batch, TOPK_THREADS, 0, s>>>(scores, n, k, out_idx);
        else if (n <= (int64_t)TOPK_THREADS * 4)
            topk_radix_reg_kernel<4><<<batch, TOPK_THREADS, 0, s>>>(scores, n, k, out_idx);
        else if (n <= (int64_t)TOPK_THREADS * 16)
            topk_radix_reg_kernel<16><<<batch, TOPK_THREADS, 0, s>>>(scores, n, k, out_idx);
        else if (n <= (int64_t)TOPK_THREADS * TOPK_EPT)
            topk_radix_reg_kernel<TOPK_EPT><<<batch, TOPK_THREADS, 0, s>>>(scores, n, k, out_idx);
        else
            topk_radix_kernel<<<batch, TOPK_THREADS, 0, s>>>(scores, n, k, out_idx);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
