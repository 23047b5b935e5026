// topk_row.hpp -- the radix select of one row by one workgroup of TOPK_THREADS threads, shared by
// the top-k kernels (topk.hip) and by kernels that select inside a larger step (mm_select.hip).
// Order: (score descending, index ascending); the k best are written in ascending index order;
// entries past min(k, n) are filled with -1.
#pragma once
#include "common.hpp"

namespace cwick {

constexpr int TOPK_THREADS = 1024;
constexpr int TOPK_WAVES = TOPK_THREADS / 64;

// exclusive scan of one value per thread across the block; returns the
// exclusive prefix and writes the block total to *total
__device__ __forceinline__ uint32_t block_exscan(uint32_t v, uint32_t *sh_wave, uint32_t *total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inc = wave_scan_u32(v);
    if (lane == 63) sh_wave[wave] = inc;
    __syncthreads();
    uint32_t wave_off = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < TOPK_WAVES; w++) {
        const uint32_t c = sh_wave[w];
        if (w < wave) wave_off += c;
        tot += c;
    }
    __syncthreads();
    *total = tot;
    return wave_off + inc - v;
}

// one row by one workgroup of TOPK_THREADS; sc and dst are the row's
__device__ __forceinline__ void topk_radix_row(const float *__restrict__ sc, int64_t n, int64_t k,
                                               int32_t *__restrict__ dst) {
    // 16 copies of the histogram, picked by lane, so that the lanes of a wave
    // that hit one digit (scores cluster in a few exponent buckets) do not all
    // serialise on one LDS word
    __shared__ uint32_t hist16[256 * 16];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t sh_wave[TOPK_WAVES];
    __shared__ uint32_t sh_prefix, sh_remaining;
    const int tid = threadIdx.x;
    const int64_t kk = k < n ? k : n;

    for (int64_t i = kk + tid; i < k; i += TOPK_THREADS) dst[i] = -1;

    if (tid == 0) {
        sh_prefix = 0u;
        sh_remaining = (uint32_t)kk;
    }
    // ---- 1. find the key of the kk-th best element ----
    uint32_t prefix = 0u, mask = 0u;
    for (int shift = 24; shift >= 0; shift -= 8) {
#pragma unroll
        for (int j = 0; j < 4; j++) hist16[tid * 4 + j] = 0u;
        __syncthreads();
        for (int64_t i = tid; i < n; i += TOPK_THREADS) {
            const uint32_t key = topk_key(sc[i]);
            if ((key & mask) == prefix)
                atomicAdd(&hist16[((key >> shift) & 0xFFu) * 16 + (tid & 15)], 1u);
        }
        __syncthreads();
        if (tid < 256) {
            uint32_t c = 0u;
#pragma unroll
            for (int j = 0; j < 16; j++) c += hist16[tid * 16 + j];
            hist[tid] = c;
        }
        __syncthreads();
        if (tid < 64) {
            // walk the 256 buckets from the largest digit down; lane b owns
            // buckets 255-4b .. 252-4b
            const uint32_t remaining = sh_remaining;
            uint32_t c[4], sum = 0u;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                c[j] = hist[255 - (tid * 4 + j)];
                sum += c[j];
            }
            uint32_t inc = wave_scan_u32(sum);
            uint32_t before = inc - sum;   // elements in strictly larger buckets
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (before < remaining && remaining <= before + c[j]) {
                    sh_prefix = prefix | ((uint32_t)(255 - (tid * 4 + j)) << shift);
                    sh_remaining = remaining - before;
                }
                before += c[j];
            }
        }
        __syncthreads();
        prefix = sh_prefix;
        mask |= 0xFFu << shift;
    }
    const uint32_t T = prefix;
    const uint32_t r = sh_remaining;   // elements equal to T that belong to the selection

    // ---- 2. ordered emit ----
    uint32_t out_base = 0u, eq_base = 0u;
    for (int64_t base = 0; base < n; base += (int64_t)TOPK_THREADS * 4) {
        const int64_t i0 = base + (int64_t)tid * 4;
        uint32_t key[4];
#pragma unroll
        for (int j = 0; j < 4; j++) key[j] = (i0 + j < n) ? topk_key(sc[i0 + j]) : 0u;
        uint32_t n_eq = 0u;
#pragma unroll
        for (int j = 0; j < 4; j++) n_eq += (i0 + j < n && key[j] == T) ? 1u : 0u;
        uint32_t eq_total;
        uint32_t eq_before = eq_base + block_exscan(n_eq, sh_wave, &eq_total);
        uint32_t take[4], n_take = 0u;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const bool in = i0 + j < n;
            const bool gt = in && key[j] > T;
            const bool eq = in && key[j] == T;
            take[j] = (gt || (eq && eq_before < r)) ? 1u : 0u;
            if (eq) eq_before++;
            n_take += take[j];
        }
        uint32_t take_total;
        uint32_t pos = out_base + block_exscan(n_take, sh_wave, &take_total);
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (take[j]) dst[pos++] = (int32_t)(i0 + j);
        out_base += take_total;
        eq_base += eq_total;
    }
}

// ---- rows that fit the register file: n <= TOPK_THREADS * TOPK_EPT ----
// Wave w owns the consecutive elements [w * 64 * ept, (w + 1) * 64 * ept); inside it lane l
// holds elements base + 64 j + l, so the loads are coalesced and index order is (j, lane):
// positions inside a wave come from ballots, positions of the waves from one block scan.
constexpr int TOPK_EPT = 64;                   // keys per thread at most; shorter rows take a kernel unrolled for fewer

template <int EPT>
__device__ __forceinline__ void topk_radix_reg_row(const float *__restrict__ sc, int64_t n, int64_t k,
                                                   int32_t *__restrict__ dst) {
    // first pass: 32 copies of the histogram, one per lane (mod 32): scores cluster in a few
    // exponent buckets and same-address LDS atomics of one instruction serialise
    __shared__ uint32_t hist32[256 * 32];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t sh_gt[TOPK_WAVES], sh_eq[TOPK_WAVES];
    __shared__ uint32_t sh_prefix, sh_remaining;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t kk = k < n ? k : n;
    for (int64_t i = kk + tid; i < k; i += TOPK_THREADS) dst[i] = -1;

    const int ept = (int)((n + TOPK_THREADS - 1) / TOPK_THREADS);     // <= EPT
    const int64_t wbase = (int64_t)wave * 64 * ept;
    // this lane holds elements j < jv
    int64_t left = n - wbase - lane;
    const int jv = left <= 0 ? 0 : (int)((left + 63) / 64 < ept ? (left + 63) / 64 : ept);
    uint32_t key[EPT];
#pragma unroll
    for (int j = 0; j < EPT; j++) key[j] = j < jv ? topk_key(sc[wbase + 64 * j + lane]) : 0u;
    if (tid == 0) {
        sh_prefix = 0u;
        sh_remaining = (uint32_t)kk;
    }
    // ---- 1. find the key of the kk-th best element ----
    uint32_t prefix = 0u, mask = 0u;
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0u;
        if (shift == 24) {
#pragma unroll
            for (int c = 0; c < 8; c++) hist32[tid + TOPK_THREADS * c] = 0u;
        }
        __syncthreads();
        if (shift == 24) {
#pragma unroll
            for (int j = 0; j < EPT; j++)
                if (j < jv) atomicAdd(&hist32[(key[j] >> 24) * 32 + (lane & 31)], 1u);
            __syncthreads();
            if (tid < 256) {
                uint32_t c = 0u;
#pragma unroll
                for (int i = 0; i < 32; i++) c += hist32[tid * 32 + ((i + tid) & 31)];
                hist[tid] = c;
            }
        } else {
#pragma unroll
            for (int j = 0; j < EPT; j++)
                if (j < jv && (key[j] & mask) == prefix) atomicAdd(&hist[(key[j] >> shift) & 0xFFu], 1u);
        }
        __syncthreads();
        if (tid < 64) {
            // walk the 256 buckets from the largest digit down; lane b owns
            // buckets 255-4b .. 252-4b
            const uint32_t remaining = sh_remaining;
            uint32_t c[4], sum = 0u;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                c[j] = hist[255 - (tid * 4 + j)];
                sum += c[j];
            }
            uint32_t inc = wave_scan_u32(sum);
            uint32_t before = inc - sum;   // elements in strictly larger buckets
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (before < remaining && remaining <= before + c[j]) {
                    sh_prefix = prefix | ((uint32_t)(255 - (tid * 4 + j)) << shift);
                    sh_remaining = remaining - before;
                }
                before += c[j];
            }
        }
        __syncthreads();
        prefix = sh_prefix;
        mask |= 0xFFu << shift;
    }
    const uint32_t T = prefix;
    const uint32_t r = sh_remaining;       // elements equal to T that belong to the selection

    // ---- 2. ordered emit ----
    uint32_t w_gt = 0u, w_eq = 0u;         // wave totals (uniform)
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        w_gt += (uint32_t)__builtin_popcountll(__ballot(j < jv && key[j] > T));
        w_eq += (uint32_t)__builtin_popcountll(__ballot(j < jv && key[j] == T));
    }
    if (lane == 0) {
        sh_gt[wave] = w_gt;
        sh_eq[wave] = w_eq;
    }
    __syncthreads();
    uint32_t eq_before = 0u, pos = 0u;     // ties / outputs of the waves before this one
    for (int w = 0; w < wave; w++) {
        const uint32_t e = sh_eq[w];
        const uint32_t take_e = eq_before >= r ? 0u : (r - eq_before < e ? r - eq_before : e);
        pos += sh_gt[w] + take_e;
        eq_before += e;
    }
    const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int j = 0; j < EPT; j++) {
        const bool gt = j < jv && key[j] > T;
        const bool eq = j < jv && key[j] == T;
        const uint64_t m_eq = __ballot(eq);
        const uint32_t my_eq_rank = eq_before + (uint32_t)__builtin_popcountll(m_eq & lt);
        const bool take = gt || (eq && my_eq_rank < r);
        const uint64_t m_take = __ballot(take);
        if (take) dst[pos + (uint32_t)__builtin_popcountll(m_take & lt)] = (int32_t)(wbase + 64 * j + lane);
        pos += (uint32_t)__builtin_popcountll(m_take);
        eq_before += (uint32_t)__builtin_popcountll(m_eq);
    }
}

}  // namespace cwick
