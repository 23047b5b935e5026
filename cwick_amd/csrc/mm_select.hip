// Block selection of the block-sparse GQA decode (the MiniMax family of the reference).
//
// Replaces, for one query or a chunk of consecutive ones, mm_index_scores (src/mm_model.c:
// 1764-1780), mm_select_blocks (:1733-1761) and the loop that writes the chosen blocks out as
// positions (:1969-1976).  What leaves is a position list per query, padded with -1, that
// launch_gqa_decode takes as its `sel`: the whole selection stays on the device.
//
//   1. mm_index_scores_kernel   one thread per (position, index head): the dot of the head's fp32
//      query with the position's bf16 key, a fused multiply-add per dimension in dimension order
//      from zero (the reference's serial loop: a chain belongs to one thread, but the heads of a
//      position are independent chains), then ReLU and the heads added in head order by the
//      first wave.  A workgroup is 64 positions x one wave per head; a wave's query is uniform
//      and read through the scalar unit; a thread requests its whole 256-byte key row in
//      16-byte pieces before it uses the first.
//   2. block maxima, started from -1e30 like the reference.  The scoring kernel leaves the
//      maximum of every group of 64 positions; when a block is a whole number of groups (128 in
//      the reference's configuration) mm_pick_kernel, one workgroup per query, makes the block
//      maxima from them, selects the `keep` best blocks (the one-workgroup radix select, lowest
//      index first among equal maxima -- the reference's heap makes that choice on tie-free
//      input) and writes the list: one launch.  Other block sizes take mm_blockmax_kernel (one
//      wave per block over the scores; blocks past a query's last one get -inf so that rows of
//      a chunk with different block counts share one top-k launch), launch_topk and
//      mm_expand_kernel.
//   3. the list: block limit / block is added when it is not among the chosen (for a limit that
//      is a multiple of the block size this is a block without a written position, which
//      contributes nothing -- the reference's rule, kept as it is); chosen blocks are full
//      except the last, so position p of the list is block[p / block] * block + p % block, or
//      -1 past the limit.
#include "common.hpp"
#include "topk_row.hpp"

namespace cwick {
namespace {

constexpr int MM_THREADS = 256;
constexpr int MM_SCORE_THREADS = 64;        // positions per workgroup of the scoring kernel (one wave per index head)
constexpr int MM_MAX_HEADS = 8;
constexpr int64_t MM_SHORT_POSITIONS = 32768;   // up to here the scoring kernel takes a wave per head
constexpr int MM_MAX_DIM = 512;

__global__ void __launch_bounds__(MM_SCORE_THREADS * MM_MAX_HEADS)
mm_index_scores_kernel(const uint16_t *__restrict__ keys, const float *__restrict__ iq, int64_t limit0, int ih, int id,
                       float *__restrict__ scores, int64_t score_stride,
                       float *__restrict__ gmax, int64_t gmax_stride) {
    // workgroup = 64 positions x ih waves: wave h runs head h's chain for the 64 positions (the
    // heads are independent until the sum), its lanes the positions
    __shared__ float sh_d[MM_MAX_HEADS][MM_SCORE_THREADS];
    const int row = blockIdx.y;
    const int64_t limit = limit0 + row;
    if ((int64_t)blockIdx.x * MM_SCORE_THREADS >= limit) return;          // the whole workgroup: before the barrier
    const int lane = threadIdx.x & 63;
    const int h = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t s = (int64_t)blockIdx.x * MM_SCORE_THREADS + lane;
    const int64_t sc = s < limit ? s : limit - 1;                   // threads past the end read the last row
    const u32x4 *kp = (const u32x4 *)(keys + (size_t)sc * id);
    const int chunks = id / 8;
    // sixteen pieces of the row (a whole 128-dimension key) are requested before the first is
    // used: one round trip to memory per key
    constexpr int G = 16;
    u32x4 kw[G];
#pragma unroll
    for (int g = 0; g < G; g++) kw[g] = kp[g < chunks ? g : chunks - 1];
    // the head's query is the same for every lane of the wave: its address is uniform, so it
    // arrives through the scalar unit, eight values a load, and enters the multiply-adds as a
    // scalar operand
    const float *__restrict__ q = iq + ((size_t)row * ih + h) * id;
    float d = 0.0f;
    for (int c0 = 0; c0 < chunks; c0 += G) {
        if (c0) {
#pragma unroll
            for (int g = 0; g < G; g++) kw[g] = kp[c0 + g < chunks ? c0 + g : chunks - 1];
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (c0 + g < chunks) {                                  // uniform
                const float *qc = q + (c0 + g) * 8;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    d = __builtin_fmaf(qc[2 * i], bf16lo_to_f32(kw[g][i]), d);
                    d = __builtin_fmaf(qc[2 * i + 1], bf16hi_to_f32(kw[g][i]), d);
                }
            }
        }
    }
    sh_d[h][lane] = d;
    __syncthreads();
    if (h != 0) return;
    float tot = 0.0f;
    for (int j = 0; j < ih; j++) {
        const float dj = sh_d[j][lane];
        if (dj > 0.0f) tot = tot + dj;
    }
    if (s < limit) scores[(size_t)row * score_stride + s] = tot;
    // the largest score of this group of 64 positions: what the block maxima are made of when a
    // block is a whole number of groups
    if (gmax) {
        const float gm = wave_max(s < limit ? fmaxf(-1e30f, tot) : -INFINITY);
        if ((threadIdx.x & 63) == 0) gmax[(size_t)row * gmax_stride + blockIdx.x] = gm;
    }
}

// The same for long contexts: one thread per position runs the chains of all heads (a key row is
// read by one wave instead of one per head, which is what counts once the rows come from HBM
// rather than out of a cache that the head waves share).
__global__ void __launch_bounds__(MM_SCORE_THREADS)
mm_index_scores_long_kernel(const uint16_t *__restrict__ keys, const float *__restrict__ iq, int64_t limit0, int ih, int id,
                       float *__restrict__ scores, int64_t score_stride,
                       float *__restrict__ gmax, int64_t gmax_stride) {
    const int row = blockIdx.y;
    const int64_t limit = limit0 + row;
    if ((int64_t)blockIdx.x * MM_SCORE_THREADS >= limit) return;
    const int64_t s = (int64_t)blockIdx.x * MM_SCORE_THREADS + threadIdx.x;
    const int64_t sc = s < limit ? s : limit - 1;                   // threads past the end read the last row
    const u32x4 *kp = (const u32x4 *)(keys + (size_t)sc * id);
    const int chunks = id / 8;
    // sixteen pieces of the row (a whole 128-dimension key) are requested before the first is
    // used: one round trip to memory per key
    constexpr int G = 16;
    u32x4 kw[G];
#pragma unroll
    for (int g = 0; g < G; g++) kw[g] = kp[g < chunks ? g : chunks - 1];
    // the query is the same for every thread: its address is uniform, so it arrives through the
    // scalar unit, eight values a load, and enters the multiply-adds as a scalar operand
    const float *__restrict__ q = iq + (size_t)row * ih * id;
    float d[MM_MAX_HEADS];
#pragma unroll
    for (int h = 0; h < MM_MAX_HEADS; h++) d[h] = 0.0f;
    for (int c0 = 0; c0 < chunks; c0 += G) {
        if (c0) {
#pragma unroll
            for (int g = 0; g < G; g++) kw[g] = kp[c0 + g < chunks ? c0 + g : chunks - 1];
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (c0 + g < chunks) {                                  // uniform
                const int c = c0 + g;
                float kf[8];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    kf[2 * i] = bf16lo_to_f32(kw[g][i]);
                    kf[2 * i + 1] = bf16hi_to_f32(kw[g][i]);
                }
#pragma unroll
                for (int h = 0; h < MM_MAX_HEADS; h++) {
                    if (h < ih) {                                   // uniform
                        const float *qh = q + h * id + c * 8;
#pragma unroll
                        for (int i = 0; i < 8; i++) d[h] = __builtin_fmaf(qh[i], kf[i], d[h]);
                    }
                }
            }
        }
    }
    float tot = 0.0f;
#pragma unroll
    for (int h = 0; h < MM_MAX_HEADS; h++)
        if (h < ih && d[h] > 0.0f) tot = tot + d[h];
    if (s < limit) scores[(size_t)row * score_stride + s] = tot;
    // the largest score of this group of 64 positions: what the block maxima are made of when a
    // block is a whole number of groups
    if (gmax) {
        const float gm = wave_max(s < limit ? fmaxf(-1e30f, tot) : -INFINITY);
        if ((threadIdx.x & 63) == 0) gmax[(size_t)row * gmax_stride + blockIdx.x] = gm;
    }
}

__global__ void __launch_bounds__(MM_THREADS)
mm_blockmax_kernel(const float *__restrict__ scores, int64_t score_stride, int64_t limit0, int bs, int64_t nblk_max,
                   float *__restrict__ bsc) {
    const int lane = threadIdx.x & 63;
    const int64_t b = (int64_t)blockIdx.x * (MM_THREADS / 64) + (threadIdx.x >> 6);
    const int row = blockIdx.y;
    if (b >= nblk_max) return;
    const int64_t limit = limit0 + row;
    const int64_t lo = b * bs, hi = lo + bs < limit ? lo + bs : limit;
    float mx = lo < limit ? -1e30f : -INFINITY;
    const float *sc = scores + (size_t)row * score_stride;
    for (int64_t t = lo + lane; t < hi; t += 64) mx = fmaxf(mx, sc[t]);
    mx = wave_max(mx);
    if (lane == 0) bsc[(size_t)row * nblk_max + b] = mx;
}

// The list of one query, by all NT threads of a workgroup: `mine` holds the kb chosen blocks in
// ascending order, -1 padded.
template <int NT>
__device__ __forceinline__ void mm_expand_row(const int32_t *__restrict__ mine, int kb, int64_t limit, int bs,
                                              int32_t *__restrict__ blk_out, int32_t *__restrict__ sel, int64_t max_sel,
                                              int32_t *__restrict__ n_sel) {
    __shared__ uint32_t sh_nv, sh_has;
    const int tid = threadIdx.x;
    const int64_t nblk = (limit + bs - 1) / bs;
    const int32_t newest = (int32_t)(limit / bs);
    if (tid == 0) sh_nv = 0, sh_has = 0;
    __syncthreads();
    // the chosen blocks come in ascending order, blocks this query does not have (and the -1
    // padding of a short row) after the ones it has: the valid entries are a prefix
    for (int j0 = 0; j0 < kb; j0 += NT) {
        const int j = j0 + tid;
        const int32_t b = j < kb ? mine[j] : -1;
        const uint32_t ok = b >= 0 && b < nblk;
        const uint32_t cnt = wave_sum_u32(ok), has = wave_sum_u32(ok && b == newest);
        if ((tid & 63) == 0 && cnt) atomicAdd(&sh_nv, cnt);
        if ((tid & 63) == 0 && has) atomicAdd(&sh_has, has);
    }
    __syncthreads();
    const int nv = (int)sh_nv;
    const int nb = nv + (sh_has ? 0 : 1);
    if (blk_out)
        for (int j = tid; j <= kb; j += NT) blk_out[j] = j < nv ? mine[j] : j < nb ? newest : -1;
    // every block of the list but its last is full
    for (int64_t p = tid; p < max_sel; p += NT) {
        const int64_t j = p / bs;
        int64_t pos = -1;
        if (j < nb) {
            const int64_t b = j < nv ? mine[j] : newest;
            pos = b * bs + (p - j * bs);
            if (pos >= limit) pos = -1;
        }
        sel[p] = (int32_t)pos;
    }
    if (n_sel && tid == 0) {
        const int64_t last = nb - 1 < nv ? mine[nb - 1] : newest;
        int64_t in_last = limit - last * bs;
        in_last = in_last < 0 ? 0 : in_last > bs ? bs : in_last;
        const int64_t total = (int64_t)(nb - 1) * bs + in_last;
        *n_sel = (int32_t)(total < max_sel ? total : max_sel);
    }
}

__global__ void __launch_bounds__(MM_THREADS)
mm_expand_kernel(const int32_t *__restrict__ blk, int kb, int64_t limit0, int bs, int32_t *__restrict__ blk_out,
                 int32_t *__restrict__ sel, int64_t max_sel, int32_t *__restrict__ n_sel) {
    const int row = blockIdx.x;
    mm_expand_row<MM_THREADS>(blk + (size_t)row * kb, kb, limit0 + row, bs,
                              blk_out ? blk_out + (size_t)row * (kb + 1) : nullptr, sel + (size_t)row * max_sel, max_sel,
                              n_sel ? n_sel + row : nullptr);
}

// Block maxima, the kept blocks and the list of one query in one workgroup, for blocks that are
// a whole number of the scoring kernel's 64-position groups: a block's maximum is that of its
// groups (a few KB per query instead of the scores themselves), the selection is the
// one-workgroup radix select, the list follows.  Three launches less than the general path.
__global__ void __launch_bounds__(TOPK_THREADS)
mm_pick_kernel(const float *__restrict__ gmax, int64_t gmax_stride, int64_t limit0, int bs, int64_t nblk_max, int kb,
               float *__restrict__ bsc, int32_t *__restrict__ blk, int32_t *__restrict__ blk_out,
               int32_t *__restrict__ sel, int64_t max_sel, int32_t *__restrict__ n_sel) {
    const int row = blockIdx.x, tid = threadIdx.x;
    const int64_t limit = limit0 + row;
    const int64_t nblk = (limit + bs - 1) / bs, ngrp = (limit + 63) / 64;
    const int gpb = bs / 64;                                          // groups per block
    const float *gm = gmax + (size_t)row * gmax_stride;
    float *mybsc = bsc + (size_t)row * nblk_max;
    for (int64_t b = tid; b < nblk; b += TOPK_THREADS) {
        float mx = -1e30f;
        for (int u = 0; u < gpb; u++) {
            const int64_t gi = b * gpb + u;
            if (gi < ngrp) mx = fmaxf(mx, gm[gi]);
        }
        mybsc[b] = mx;
    }
    __syncthreads();                                                  // the workgroup reads what it wrote
    int32_t *myblk = blk + (size_t)row * kb;
    if (nblk <= TOPK_THREADS) topk_radix_reg_row<1>(mybsc, nblk, kb, myblk);     // a score per thread, kept in a register
    else topk_radix_row(mybsc, nblk, kb, myblk);
    __syncthreads();
    mm_expand_row<TOPK_THREADS>(myblk, kb, limit, bs, blk_out ? blk_out + (size_t)row * (kb + 1) : nullptr,
                                sel + (size_t)row * max_sel, max_sel, n_sel ? n_sel + row : nullptr);
}

}  // namespace

int launch_mm_select(const uint16_t *idx_keys, const float *iq, int batch, int64_t limit0, int index_heads,
                     int index_dim, int block, int keep_blocks, float *scores, int64_t score_stride,
                     int32_t *blk_out, int32_t *sel, int64_t max_sel, int32_t *n_sel, hipStream_t s) {
    CWICK_REQUIRE(idx_keys && iq && scores && sel, "mm_select: null pointer");
    CWICK_REQUIRE(batch >= 1 && batch <= 65535 && limit0 >= 1 && limit0 + batch - 1 <= ((int64_t)1 << 30),
                  "mm_select: batch %d, first limit %lld", batch, (long long)limit0);
    CWICK_REQUIRE(index_heads >= 1 && index_heads <= MM_MAX_HEADS && index_dim >= 8 && index_dim <= MM_MAX_DIM &&
                      index_dim % 8 == 0,
                  "mm_select: %d index heads of %d dims (1..%d heads, dims a multiple of 8 up to %d)", index_heads,
                  index_dim, MM_MAX_HEADS, MM_MAX_DIM);
    CWICK_REQUIRE(block >= 1 && keep_blocks >= 1 && keep_blocks <= 4096, "mm_select: block %d, blocks kept %d", block,
                  keep_blocks);
    const int64_t limit_max = limit0 + batch - 1;
    CWICK_REQUIRE(score_stride >= limit_max, "mm_select: score rows of %lld hold fewer than %lld positions",
                  (long long)score_stride, (long long)limit_max);
    CWICK_REQUIRE(max_sel >= 1 && max_sel <= ((int64_t)1 << 24), "mm_select: max_sel %lld", (long long)max_sel);
    CWICK_REQUIRE(((uintptr_t)idx_keys) % 16 == 0, "mm_select: index keys must be 16-byte aligned");
    const int64_t nblk_max = (limit_max + block - 1) / block;
    // (the top-k below keeps its own workspace slot, so the block scores can sit in this call's)
    CWICK_REQUIRE(nblk_max < 16384, "mm_select: %lld blocks (at most 16383)", (long long)nblk_max);
    const bool fused = block % MM_SCORE_THREADS == 0;          // a block is whole groups of the scoring kernel
    const int64_t ng_max = (limit_max + MM_SCORE_THREADS - 1) / MM_SCORE_THREADS;
    const size_t bsc_b = ((size_t)batch * nblk_max * 4 + 255) & ~(size_t)255;
    const size_t blk_b = ((size_t)batch * keep_blocks * 4 + 255) & ~(size_t)255;
    char *ws = (char *)workspace(s, bsc_b + blk_b + (fused ? (size_t)batch * ng_max * 4 : 0));
    if (!ws) return 0;                      // workspace() has recorded why
    float *bsc = (float *)ws;
    int32_t *blk = (int32_t *)(ws + bsc_b);
    float *gmax = fused ? (float *)(ws + bsc_b + blk_b) : nullptr;
    {
        ProfScope ps(CWICK_HIP_PROF_MM_SELECT, s);
        const dim3 sgrid((unsigned)ng_max, batch);
        // up to 32 K positions a wave per head (8 192 positions: 8.5 -> 5.5 us); beyond, the head
        // waves' reads of the same key rows cost more than their parallelism gains (262 144
        // positions: 19 us against 32)
        if (limit_max * batch <= MM_SHORT_POSITIONS)
            mm_index_scores_kernel<<<sgrid, MM_SCORE_THREADS * index_heads, 0, s>>>(
                idx_keys, iq, limit0, index_heads, index_dim, scores, score_stride, gmax, ng_max);
        else
            mm_index_scores_long_kernel<<<sgrid, MM_SCORE_THREADS, 0, s>>>(idx_keys, iq, limit0, index_heads, index_dim,
                                                                       scores, score_stride, gmax, ng_max);
        if (fused)
            mm_pick_kernel<<<dim3(batch), TOPK_THREADS, 0, s>>>(gmax, ng_max, limit0, block, nblk_max, keep_blocks, bsc,
                                                                blk, blk_out, sel, max_sel, n_sel);
        else
            mm_blockmax_kernel<<<dim3((unsigned)((nblk_max + 3) / 4), batch), MM_THREADS, 0, s>>>(
                scores, score_stride, limit0, block, nblk_max, bsc);
    }
    CWICK_HIP_CALL(hipGetLastError());
    if (fused) return 1;
    if (!launch_topk(bsc, batch, nblk_max, keep_blocks, blk, s)) return 0;
    {
        ProfScope ps(CWICK_HIP_PROF_MM_SELECT, s);
        mm_expand_kernel<<<dim3(batch), MM_THREADS, 0, s>>>(blk, keep_blocks, limit0, block, blk_out, sel, max_sel, n_sel);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
