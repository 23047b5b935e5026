// gqa_decode.hip -- split-K flash-decoding for one query position over a bf16
// K/V cache (the decode branch of the reference's mixer_attn,
// src/q35_model.c:1656-1701: dec_scores / dec_softmax / dec_out_slices).
//
// HBM-bound: every K and V row is read exactly once.
//
//   grid  = (n_splits, n_kv_heads), 256 threads (4 waves)
//   A workgroup owns one kv head and one contiguous slice of keys and serves
//   the `group` query heads that share the kv head (the reference walks cache
//   rows for the same reason: one row serves every head of its group,
//   src/q35_model.c:1417-1423).
//   A key row of head_dim bf16 is read by LPK = head_dim/8 lanes, 16 bytes
//   (8 dims) per lane, so a wave covers 64/LPK consecutive rows with full
//   1 KiB coalesced loads.  Each lane keeps `group` partial dots, an xor
//   butterfly over the LPK lanes leaves the full score in every lane of the
//   row, so the weight exp(s - m) is available where the V row lands without a
//   broadcast.  Online softmax per lane group, KB rows per step to amortise
//   the rescale; the lane groups of a workgroup are merged through LDS, then
//   (m, l, acc) goes to the workspace and a second kernel merges the splits.
//   With a position list (sel[]: the block-sparse decode of src/mm_model.c:1962-2047, whose
//   selected blocks the caller has expanded to positions) list entry i names cache row sel[i];
//   entries that name no row (negative, or beyond n_rows) carry no weight.
#include "common.hpp"
#include "merge.hpp"

#include <cstdlib>

namespace cwick {

constexpr int GQA_DEC_THREADS = 256;
constexpr int GQA_DEC_KB = 4;      // key rows per lane group per step

template <int HD, int GROUP>
__global__ void __launch_bounds__(GQA_DEC_THREADS)
gqa_decode_split_kernel(const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
                        const uint16_t *__restrict__ Q, int64_t n_keys, int n_kv_heads,
                        const int32_t *__restrict__ sel, int64_t n_rows,
                        int keys_per_split, int kv_shift, float scale,
                        float *__restrict__ part_acc,   // [n_splits][n_heads][HD]
                        float *__restrict__ part_ml) {  // [n_splits][n_heads][2]
    constexpr int LPK = HD / 8;                 // lanes per key row
    constexpr int NGRP = GQA_DEC_THREADS / LPK; // lane groups per workgroup
    // a kv head whose group is larger than GROUP is served by 1 << kv_shift workgroups, each with
    // GROUP of its query heads
    const int g = blockIdx.y;
    const int gk = g >> kv_shift;
    const int split = blockIdx.x;
    const int n_heads = (n_kv_heads << kv_shift) * GROUP;
    const int tid = threadIdx.x;
    const int sub = tid % LPK;                  // which 8 dims of the row
    const int grp = tid / LPK;                  // which lane group
    const int64_t k_begin = (int64_t)split * keys_per_split;
    const int64_t k_end = (k_begin + keys_per_split < n_keys) ? k_begin + keys_per_split : n_keys;
    const int64_t row_stride = (int64_t)n_kv_heads * HD;

    // this lane's 8 query dims for each head of the group, pre-scaled
    float q[GROUP][8];
#pragma unroll
    for (int j = 0; j < GROUP; j++) {
        const u32x4 w = *(const u32x4 *)(Q + ((size_t)(g * GROUP + j) * HD + sub * 8));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            q[j][2 * i] = bf16lo_to_f32(w[i]) * scale;
            q[j][2 * i + 1] = bf16hi_to_f32(w[i]) * scale;
        }
    }

    float m[GROUP], l[GROUP], acc[GROUP][8];
#pragma unroll
    for (int j = 0; j < GROUP; j++) {
        m[j] = -INFINITY;
        l[j] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[j][i] = 0.0f;
    }

    const uint16_t *Kg = K + (size_t)gk * HD + sub * 8;
    const uint16_t *Vg = V + (size_t)gk * HD + sub * 8;

    for (int64_t base = k_begin + (int64_t)grp * GQA_DEC_KB; base < k_end;
         base += (int64_t)NGRP * GQA_DEC_KB) {
        u32x4 kw[GQA_DEC_KB], vw[GQA_DEC_KB];
        bool dead[GQA_DEC_KB];
#pragma unroll
        for (int r = 0; r < GQA_DEC_KB; r++) {
            // rows past the slice are clamped (their weight is forced to zero below)
            int64_t t = base + r < k_end ? base + r : k_end - 1;
            dead[r] = base + r >= k_end;
            if (sel) {
                t = sel[t];
                if (t < 0 || t >= n_rows) dead[r] = true, t = 0;
            }
            kw[r] = *(const u32x4 *)(Kg + t * row_stride);
            vw[r] = *(const u32x4 *)(Vg + t * row_stride);
        }
        float s[GQA_DEC_KB][GROUP];
#pragma unroll
        for (int r = 0; r < GQA_DEC_KB; r++) {
            float kf[8];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                kf[2 * i] = bf16lo_to_f32(kw[r][i]);
                kf[2 * i + 1] = bf16hi_to_f32(kw[r][i]);
            }
#pragma unroll
            for (int j = 0; j < GROUP; j++) {
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) d = __builtin_fmaf(q[j][i], kf[i], d);
                s[r][j] = d;
            }
        }
        // the LPK lanes of the row add up their parts, every lane ending with the full dot
        // (through DPP and lane swaps: no trips through LDS)
#pragma unroll
        for (int r = 0; r < GQA_DEC_KB; r++)
#pragma unroll
            for (int j = 0; j < GROUP; j++) {
                float t = s[r][j];
                t = group_step_sum<2>(t);
                t = group_step_sum<4>(t);
                t = group_step_sum<8>(t);
                t = group_step_sum<16>(t);
                if (LPK == 32) t = group_step_sum<32>(t);
                s[r][j] = t;
            }
#pragma unroll
        for (int r = 0; r < GQA_DEC_KB; r++)
            if (dead[r])
#pragma unroll
                for (int j = 0; j < GROUP; j++) s[r][j] = -INFINITY;

#pragma unroll
        for (int j = 0; j < GROUP; j++) {
            float mx = m[j];
#pragma unroll
            for (int r = 0; r < GQA_DEC_KB; r++) mx = fmaxf(mx, s[r][j]);
            // all of a step's rows can be dead in a list: then nothing moves (exp(-inf) = 0)
            const float corr = __expf(m[j] - (mx == -INFINITY ? 0.0f : mx));
            m[j] = mx;
            l[j] *= corr;
#pragma unroll
            for (int i = 0; i < 8; i++) acc[j][i] *= corr;
#pragma unroll
            for (int r = 0; r < GQA_DEC_KB; r++) {
                const float p = __expf(s[r][j] - (mx == -INFINITY ? 0.0f : mx));
                l[j] += p;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    acc[j][2 * i] = __builtin_fmaf(p, bf16lo_to_f32(vw[r][i]), acc[j][2 * i]);
                    acc[j][2 * i + 1] = __builtin_fmaf(p, bf16hi_to_f32(vw[r][i]), acc[j][2 * i + 1]);
                }
            }
        }
    }

    // merge the lane groups of one wave with shuffles (lanes l and l^o hold the
    // same 8 dims of different key subsets) ...
    // A swap leaves the values of the two lane groups that meet in two registers, the same
    // pair in every lane: all lanes merge (first, second) in that order.
    auto meet = [&](float v, int o, float &first, float &second) {
        uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
        if (o == 16) lanes_swap16(a, b); else lanes_swap32(a, b);
        first = __builtin_bit_cast(float, a);
        second = __builtin_bit_cast(float, b);
    };
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
        for (int j = 0; j < GROUP; j++) {
            float m1, m2, l1, l2;
            meet(m[j], o, m1, m2);
            meet(l[j], o, l1, l2);
            const float mx = fmaxf(m1, m2);
            const float c1 = mx > -INFINITY ? __expf(m1 - mx) : 0.0f;
            const float c2 = mx > -INFINITY ? __expf(m2 - mx) : 0.0f;
            l[j] = l1 * c1 + l2 * c2;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float a1, a2;
                meet(acc[j][i], o, a1, a2);
                acc[j][i] = a1 * c1 + a2 * c2;
            }
            m[j] = mx;
        }
    }
    // ... and the waves of the workgroup through LDS
    constexpr int NW = GQA_DEC_THREADS / 64;
    __shared__ __attribute__((aligned(16))) float sh_acc[NW][GROUP][HD];
    __shared__ float sh_m[NW][GROUP], sh_l[NW][GROUP];
    const int wave = tid >> 6;
    if ((tid & 63) < LPK) {
#pragma unroll
        for (int j = 0; j < GROUP; j++) {
#pragma unroll
            for (int i = 0; i < 8; i++) sh_acc[wave][j][sub * 8 + i] = acc[j][i];
            if (sub == 0) {
                sh_m[wave][j] = m[j];
                sh_l[wave][j] = l[j];
            }
        }
    }
    __syncthreads();
    // a thread takes four consecutive dims of one head: the waves' weights once per four values,
    // the values in 16-byte LDS reads, two 8-byte stores
    for (int i4 = tid; i4 < GROUP * HD / 4; i4 += GQA_DEC_THREADS) {
        const int j = i4 / (HD / 4), d = (i4 % (HD / 4)) * 4;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; w++) mx = fmaxf(mx, sh_m[w][j]);
        f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
        float ls = 0.0f;
        if (mx > -INFINITY) {
#pragma unroll
            for (int w = 0; w < NW; w++) {
                const float c = __expf(sh_m[w][j] - mx);   // exp(-inf) = 0 for idle waves
                const f32x4 t = *(const f32x4 *)&sh_acc[w][j][d];
#pragma unroll
                for (int r = 0; r < 4; r++) a[r] += t[r] * c;
                ls += sh_l[w][j] * c;
            }
        }
        const int h = g * GROUP + j;
        // written through: the merge kernel reads it from other XCDs, and a dirty line would be
        // written back at the end of this kernel
        uint64_t *dst = (uint64_t *)&part_acc[((size_t)split * n_heads + h) * HD + d];
        __hip_atomic_store(dst, __builtin_bit_cast(uint64_t, (f32x2){a[0], a[1]}), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(dst + 1, __builtin_bit_cast(uint64_t, (f32x2){a[2], a[3]}), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        if (d == 0) {
            part_ml[((size_t)split * n_heads + h) * 2 + 0] = mx;
            part_ml[((size_t)split * n_heads + h) * 2 + 1] = ls;
        }
    }
}

template <int HD, int GROUP>
static int run_gqa_decode(const uint16_t *k, const uint16_t *v, int64_t n_keys, int n_kv_heads,
                          const int32_t *sel, int64_t n_rows, const uint16_t *q, float scale, float *out,
                          hipStream_t s, int kv_shift = 0) {
    const int n_units = n_kv_heads << kv_shift;            // (kv head, GROUP query heads) pairs
    const int n_heads = n_units * GROUP;
    constexpr int LPK = HD / 8, NGRP = GQA_DEC_THREADS / LPK;
    constexpr int step = NGRP * GQA_DEC_KB;   // rows one workgroup consumes per iteration
    // About one workgroup per CU, each with whole steps: a slice is the share of a workgroup
    // rounded DOWN to whole steps (a few workgroups more than CUs are cheaper than workgroups
    // half as many and twice as long; twice as many with one step each cost a microsecond in
    // partials written and merged).  4096 keys on 4 kv heads: 64 slices of two steps.
    const char *env = getenv("CWICK_HIP_GQA_WG_PER_CU");
    int per_cu = env ? atoi(env) : 1;
    if (per_cu < 1 || per_cu > 8) per_cu = 1;
    int64_t want = (int64_t)per_cu * num_cus() / n_units;
    if (want < 1) want = 1;
    if (want > MERGE_MAX_SPLITS / 2) want = MERGE_MAX_SPLITS / 2;
    int64_t per = (n_keys / want) / step * step;
    if (per < step) per = step;
    const int n_splits = (int)((n_keys + per - 1) / per);
    const size_t acc_bytes = (size_t)n_splits * n_heads * HD * sizeof(float);
    const size_t ml_bytes = (size_t)n_splits * n_heads * 2 * sizeof(float);
    char *ws = (char *)workspace(s, acc_bytes + ml_bytes);
    if (!ws) return 0;                      // workspace() has recorded why
    float *part_acc = (float *)ws, *part_ml = (float *)(ws + acc_bytes);
    {
        ProfKernel pk(CWICK_HIP_PROF_GQA_DECODE, s);
        pk.launch(gqa_decode_split_kernel<HD, GROUP>, dim3(n_splits, n_units), dim3(GQA_DEC_THREADS), 0,
                  k, v, q, n_keys, n_kv_heads, sel, n_rows, (int)per, kv_shift, scale, part_acc, part_ml);
    }
    CWICK_HIP_CALL(hipGetLastError());
    {
        ProfKernel pk(CWICK_HIP_PROF_GQA_DECODE_MERGE, s);
        pk.launch(splitk_merge_wide_kernel<HD>, dim3(n_heads, 1), dim3(64 * (n_splits < 16 ? n_splits : 16)), 0,
                  part_acc, part_ml, n_splits, n_heads, out);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

int launch_gqa_decode(const uint16_t *k, const uint16_t *v, int64_t n_keys, int n_kv_heads,
                      int head_dim, const uint16_t *q, int n_heads, float scale, float *out,
                      hipStream_t s, const int32_t *sel, int64_t n_rows) {
    CWICK_REQUIRE(k && v && q && out, "gqa_decode: null pointer");
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= ((int64_t)1 << 30), "gqa_decode: n_keys %lld",
                  (long long)n_keys);
    CWICK_REQUIRE(n_kv_heads >= 1 && n_kv_heads <= 64 && n_heads >= n_kv_heads &&
                      n_heads % n_kv_heads == 0,
                  "gqa_decode: n_heads %d is not a multiple of n_kv_heads %d", n_heads, n_kv_heads);
    CWICK_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)q) % 16 == 0,
                  "gqa_decode: K, V and q must be 16-byte aligned");
    const int group = n_heads / n_kv_heads;
#define CASE(HD, G)                                      \
    if (head_dim == HD && group == G)                    \
        return run_gqa_decode<HD, G>(k, v, n_keys, n_kv_heads, sel, n_rows, q, scale, out, s)
    CASE(256, 1); CASE(256, 2); CASE(256, 4); CASE(256, 8);
    CASE(128, 1); CASE(128, 2); CASE(128, 4); CASE(128, 8);
#undef CASE
    // sixteen query heads per kv head (the block-sparse family's 64/4): two workgroups of eight
    if (group == 16 && head_dim == 256) return run_gqa_decode<256, 8>(k, v, n_keys, n_kv_heads, sel, n_rows, q, scale, out, s, 1);
    if (group == 16 && head_dim == 128) return run_gqa_decode<128, 8>(k, v, n_keys, n_kv_heads, sel, n_rows, q, scale, out, s, 1);
    set_error("gqa_decode: head_dim %d with group %d is not supported (head_dim 128/256, group 1/2/4/8/16)",
              head_dim, group);
    return 0;
}

}  // namespace cwick
