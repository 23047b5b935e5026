// mla_roles.hip -- absorbed-latent MLA over the FP8 latent (decode, sparse decode and chunked
// prefill of src/attention.c:749-811 / :1010-1019).
//
//   workgroup = 12 waves, 32 query rows (heads of one query) x one key slice, walked in tiles
//   of 64 keys.  The waves take one of two roles:
//     waves 0..7  score: wave (kb, hh) takes keys 16 kb..+15 of the tile and heads 16 hh..+15:
//                 S^T = K Q^T on v_mfma_scale_f32_16x16x128_f8f6f4 with K as stored (E4M3) and Q
//                 as two E4M3 terms with a shared E8M0 scale per head and 128-dim block; the five
//                 block products are combined with the keys' fp32 block scales, exponentiated
//                 against the wave's reference m, and published through LDS as fp16
//                 probabilities exp2(s - m), already in the fragment order of the value MFMA,
//                 together with m;
//     waves 8..11 accumulate: wave cw owns output dims 128 cw..+127 (one scale block) for all 32
//                 heads: it turns the probabilities into weights p * scale[key][cw] * 2^(10 - e)
//                 (packed fp16 multiplies; 2^e is above every scale the wave has seen, so the
//                 weights fit fp16) and runs O^T += V^T W^T on v_mfma_f32_16x16x32_f16, V^T read
//                 transposed from the tile (ds_read_b64_tr_b8) and widened E4M3 -> fp16 (exact).
//   The roles are one tile apart (tile t+1 is scored while tile t is accumulated), so a step has
//   a single workgroup barrier and nobody waits for an exchange inside it.  The softmax
//   reference is lazy: a scoring wave keeps the reference every wave knows (m_ref) unless its own
//   tile exceeds it by 2^LAZY; the m it used travels with the probabilities together with one
//   flag per scoring wave ("my reference for this tile is not the common one").  One step later
//   every wave reads the eight flags: all clear (almost always) means nothing to do; otherwise
//   the accumulating waves (and the scorers, for their sums) bring everything to the common
//   maximum.  Each scoring lane keeps the sum of its own keys; the sums meet once, after the loop.
//   Tiles are copied global -> LDS by global_load_lds (no registers) into four stages.  Tile 0 is
//   fetched by all twelve waves at kernel start, tile 1 behind it by the two waves that have no
//   part in the preparation of Q, tile 2 by the value waves behind the first barrier; from step 0
//   on every wave copies its share of tile t+3 during step t
//   (three sixteen-byte columns of the 64 rows, plus a scale block for five of the waves): the
//   value waves at the top of the step, the scoring waves at the end of theirs, when they would
//   otherwise wait at the barrier.  The copies are issued from inline assembly and the barrier
//   waits for LDS traffic only, so the compiler never makes anything wait for the tiles in
//   flight.  LDS is addressed by integer byte offsets throughout (a generic pointer into LDS costs
//   a null check and a 64-bit add per use), and the kernel exists in two instantiations: dense
//   lists (rows are k_begin + i, only the last tile can be ragged) and lists given by sel[].
//
//   Where the time goes (counters and ablation builds, 12 waves on 256 CUs): a 64-key step takes
//   about 3 000 cycles against 1 088 of matrix-core work.  Leaving out the tile copies, the score
//   MFMAs or the value MFMAs with their conversions takes about a quarter off each, all three
//   together two thirds; what remains (barrier, exchange, softmax, weights) is the last third.
//   No single unit is saturated: vector ALU 56 % busy, matrix core 37 %, LDS 32 %.  A copy
//   instruction here has one lane per row (64 cache lines touched); alone on the machine that
//   pattern moves 54 bytes per ns and compute unit from L2 and 18 from HBM, a pattern that walks
//   along the rows 125 and 25.  Inside this kernel it makes no difference: tile layouts filled
//   sixteen lines per instruction ([16-key block][piece][key]) or row by row were built, pass
//   parity and run 4 to 7 % slower, because they spend more vector instructions per copy on
//   addresses, and the vector ALU, not the copy path, is what a step waits for most.  With 32
//   query rows per tile the per-tile work that does not depend on the rows (copies, scale
//   handling, conversions of V) is paid per 1 088 matrix cycles; 64 rows would halve it per
//   flop.  Eight or sixteen waves per workgroup (the same work split differently) were measured
//   and are no faster.
//
//   LDS tile layout [16-byte column][key 0..63][16 B]: the K fragment is two 16-byte reads per
//   lane, 256 B contiguous per 16 keys; the V^T fragment of 32 keys x 16 dims is one
//   ds_read_b64_tr_b8, 128 B contiguous per 16-lane group (keys 8 g..8 g+7 of the half).
//
//   Split-K partials are stored per 16 heads in accumulator-fragment order
//   [split][16-head block][dim block][lane][4] (every store 1 KiB contiguous);
//   mla_merge_frag16_kernel reads them in the same order with all loads in flight.
#include "common.hpp"

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace cwick {
namespace {

constexpr int KDIM = CWICK_HIP_LATENT_KDIM;   // 576
constexpr int VDIM = CWICK_HIP_LATENT_VDIM;   // 512
constexpr int NBLK = CWICK_HIP_LATENT_NBLK;   // 5
constexpr int THREADS = 768;                  // waves 0..7 score, waves 8..11 accumulate values
constexpr int TK = 64;                        // keys per tile
constexpr int HB = 16;                        // heads per head half (partials are laid out per 16 heads)
constexpr int HW = 32;                        // heads per workgroup
constexpr int NST = 4;                        // tile stages
constexpr int NCOL = KDIM / 16;               // 36 sixteen-byte columns per row
constexpr int NDB = VDIM / 16;                // 32 sixteen-dim output blocks
constexpr float LAZY = 4.0f;                  // the reference moves when a tile exceeds it by 2^LAZY
constexpr int WEXP = 10;                      // fp16 weights are p * scale * 2^(WEXP - e), scale < 2^e
constexpr int E_NONE = -1000;                 // no scale seen yet
constexpr int MERGE_MAX_SPLITS = 1024;

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
// max(v[l], v[l ^ 16]) and max(v[l], v[l ^ 32]) in every lane
__device__ __forceinline__ uint32_t lanes_xor16_max(uint32_t v) {
    uint32_t a = v, b = v;
    lanes_swap16(a, b);
    return a > b ? a : b;
}
__device__ __forceinline__ uint32_t lanes_xor32_max(uint32_t v) {
    uint32_t a = v, b = v;
    lanes_swap32(a, b);
    return a > b ? a : b;
}
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef __attribute__((address_space(3))) void lds_void;

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
    int64_t keys_per_split;   // multiple of TK
    const float *sink;        // per head, natural-log units of the scaled scores, or null
    float *out, *part_ml;
    uint32_t *part_acc;
};

// What a masked position of a tile (past the end of the list, a -1 or out-of-range entry of
// sel[]) is fetched from: a row of zero bytes with zero scales.  Its weight is zero already;
// with zero values and zero scales nothing of any cache row that is not in the list (a NaN
// byte, a scale many binades above the others) can reach the products or the fp16 normaliser.
__device__ __attribute__((aligned(16))) uint8_t g_zero_row[KDIM + 64] = {0};
__device__ __attribute__((aligned(16))) float g_zero_scales[8] = {0.0f};

struct Tile {
    uint8_t kv[NCOL][TK][16];     // [16-byte column][key][16]     36864 B
    float sc[NBLK][TK];           // [block][key]                   1280 B
    uint32_t valid[2];            // list kernels: bit k = position k of the tile holds a row
    uint32_t pad[2];
};
struct Xch {                       // what the scoring waves publish per tile
    // fp16 probabilities exp2(s - m), laid out as the B fragments of the value MFMA:
    // [head half][32-key half][slot group g][head n][4 dwords]; contraction slot 8 g + j of a
    // half is key 8 g + j of that half
    uint32_t p[2][2][4][16][4];
    float m[2][16][4];            // [head half][head][key block]: the reference m they are relative to
    uint32_t moved[8];            // per scoring wave: its reference for this tile is not the common one
};
struct Smem {
    Tile tile[NST];
    Xch x[2];
};
// Q of one (head half, 128-dim block) in MFMA operand order, dword-interleaved by lane; for the
// rope block `hi` is the combined hi|lo register set
struct QPark { int hi[8][64]; int lo[8][64]; int sc[64]; };
static_assert(10 * sizeof(QPark) <= sizeof(Tile) + 2 * sizeof(Xch), "Q park area");
static_assert(sizeof(Tile) * NST + 2 * sizeof(Xch) <= 160 * 1024, "LDS");

__device__ __forceinline__ float pow2i(int e) {
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
    return __builtin_bit_cast(float, (uint32_t)(e + 127) << 23);
}

// both fp16 halves of a dword times f
__device__ __forceinline__ uint32_t scale_f16x2(uint32_t x, float f) {
    const _Float16 h = (_Float16)f;
    const f16x2 r = __builtin_bit_cast(f16x2, x) * (f16x2){h, h};
    return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ uint32_t mul_f16x2(uint32_t a, uint32_t b) {
    const f16x2 r = __builtin_bit_cast(f16x2, a) * __builtin_bit_cast(f16x2, b);
    return __builtin_bit_cast(uint32_t, r);
}

#define LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

// one instruction per max: the compiler's fmaxf quiets both operands first (a v_max of the
// operand with itself) because it may not assume they are not signalling NaNs
__device__ __forceinline__ float vmax(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float vmax3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ uint32_t umax3(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r;
    asm("v_max3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) u32x2 lds_u32x2;
typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
typedef __attribute__((address_space(3))) f32x2 lds_f32x2;
typedef __attribute__((address_space(3))) float lds_f32;
typedef __attribute__((address_space(3))) uint32_t lds_u32;
// LDS is addressed by byte offsets held in ordinary integers (a generic pointer into LDS costs a
// null check and a 64-bit add at every use)
#define LDS_AT(type, a) (*(type *)(size_t)(uint32_t)(a))

// LDS offsets of the parts of Smem
constexpr uint32_t TILE_B = sizeof(Tile);
constexpr uint32_t SC_OFF = NCOL * TK * 16;                       // Tile::sc
constexpr uint32_t VALID_OFF = SC_OFF + NBLK * TK * 4;            // Tile::valid
constexpr uint32_t X_OFF = NST * TILE_B;                          // Smem::x
constexpr uint32_t XCH_B = sizeof(Xch);
constexpr uint32_t XM_OFF = 2 * 2 * 4 * 16 * 4 * 4;               // Xch::m
constexpr uint32_t XF_OFF = XM_OFF + 2 * 16 * 4 * 4;              // Xch::moved

template <bool SEL>
__global__ void __launch_bounds__(THREADS) mla_roles_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    Smem &sm = *reinterpret_cast<Smem *>(smem_raw);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_void *)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool scorer = wave < 8;
    const int kb = wave & 3;         // scoring role: keys 16 kb .. 16 kb + 15 of the tile
    const int hh = (wave >> 2) & 1;  //               heads 16 hh .. 16 hh + 15
    const int cw = wave & 3;         // value role: dims 128 cw .. +127 = scale block cw
    const int n = lane & 15;         // head column / key row of a 16-block / dim row
    const int g = lane >> 4;         // 32-wide contraction block (QK) / 8-wide (PV)

    const int n_hb = (p.nh + HW - 1) / HW;
    const uint32_t total = gridDim.x, u_hb = (uint32_t)n_hb, u_sp = (uint32_t)p.n_splits;
    // Workgroups go to the eight XCDs round robin.  Decode: an XCD takes a contiguous eighth of
    // the units (the head blocks of a slice, the slices of a query: what they share stays in one
    // L2).  Causal prefill: queries differ in length, so consecutive queries go to consecutive
    // XCDs instead (a contiguous eighth would leave the XCD with the longest queries behind).
    // (32-bit arithmetic: a 64-bit division is a hundred instructions in front of the first load)
    uint32_t unit = blockIdx.x;
    if (p.list_step > 0 && p.n_splits == 1) {
        if (total % (8 * u_hb) == 0) {
            const uint32_t grp = unit / (8 * u_hb), r = unit % (8 * u_hb);
            unit = (8 * grp + r % 8) * u_hb + r / 8;
        }
    } else if (total % 8 == 0) {
        unit = (unit % 8) * (total / 8) + unit / 8;
    }
    const int hb = (int)(unit % u_hb);
    const int split = (int)((unit / u_hb) % u_sp);
    int y = (int)(unit / (u_hb * u_sp));
    if (p.list_step > 0) y = p.nq - 1 - y;          // causal prefill: the queries with the most keys start first

    const uint8_t *rows = p.rows + (size_t)y * p.row_bstride;
    const float *scales = p.scales + (size_t)y * p.scale_bstride;
    const int32_t *sel = SEL ? p.sel + (size_t)y * p.n_list : nullptr;
    const int64_t limit = p.n_list + (int64_t)y * p.list_step;
    const int64_t k_begin = (int64_t)split * p.keys_per_split;
    int64_t k_end = k_begin + p.keys_per_split;
    if (k_end > limit) k_end = limit;
    const int n_keys = k_end > k_begin ? (int)(k_end - k_begin) : 0;     // of this workgroup
    const int n_tiles = (n_keys + TK - 1) / TK;

    // The zero row and its scales: where masked positions of a tile are fetched from.  The
    // addresses are taken once, here: inside the loops every mention would be a load from the
    // global offset table.
    uint64_t zrow = (uint64_t)(uintptr_t)g_zero_row, zsc = (uint64_t)(uintptr_t)g_zero_scales;
    asm volatile("" : "+s"(zrow), "+s"(zsc));

    // copy role: lane = key of the tile; row of the cache or -1
    auto row_of = [&](int t) -> int {
        const int i = t * TK + lane;
        if (!SEL) return (t < n_tiles && i < n_keys) ? (int)(k_begin + i) : -1;    // rows fit 31 bits (checked by the launcher)
        int r = -1;
        if (t < n_tiles && i < n_keys) {
            r = sel[k_begin + i];
            if (r < 0 || r >= p.n_rows) r = -1;
        }
        return r;
    };
    // global -> LDS copies in assembly: the compiler keeps no account of them, so nothing in the
    // loop waits for the tile in flight except the s_waitcnt before the barrier.  Each statement
    // writes M0 itself right before the copy that reads it.  M0 is a reserved register to the
    // compiler (it cannot be named as clobbered); what keeps this safe is that nothing else in
    // this file makes the compiler use M0, which tests/test_mfma_wait_states.py checks on the
    // compiled code.
    auto dma16 = [&](uint64_t gp, uint32_t lds_off) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gp), "s"(lds_off) : "memory");
    };
    auto dma4 = [&](uint64_t gp, uint32_t lds_off) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gp), "s"(lds_off) : "memory");
    };
    // pieces 0..35 = sixteen-byte columns of the 64 rows, 36..40 = scale blocks
    auto piece = [&](int pc, uint64_t rowp, uint64_t scp, uint32_t tile_off) {
        if (pc < NCOL) dma16(rowp + 16 * pc, tile_off + pc * (TK * 16));
        else if (pc < NCOL + NBLK) dma4(scp + 4 * (pc - NCOL), tile_off + SC_OFF + (pc - NCOL) * (TK * 4));
    };
    auto row_ptr = [&](int r) -> uint64_t { return r >= 0 ? (uint64_t)(uintptr_t)rows + (uint64_t)(uint32_t)r * KDIM : zrow; };
    auto sc_ptr = [&](int r) -> uint64_t { return r >= 0 ? (uint64_t)(uintptr_t)scales + (uint64_t)(uint32_t)r * (NBLK * 4) : zsc; };
    // this wave's share of a tile: three columns, and a scale block for the first five waves
    // which of the 64 positions of the tile hold a row (the scoring waves mask the others)
    auto mark = [&](int r, uint32_t tile_off) {
        const uint64_t v = __ballot(r >= 0);
        LDS_AT(lds_u32x2, tile_off + VALID_OFF) = (u32x2){(uint32_t)v, (uint32_t)(v >> 32)};
    };
    auto share = [&](int r, uint32_t tile_off) {
        const uint64_t rp = row_ptr(r), sp = sc_ptr(r);
        // columns wave, wave + 12, wave + 24 (all below 36) and, for the first five waves, scale block `wave`
        const uint32_t col_off = tile_off + (uint32_t)wave * (TK * 16);
        const uint64_t col_src = rp + 16 * wave;
        // (the 192 and 384 bytes to the lane's source are the instruction's immediate offset, which
        // the hardware also adds to the LDS address: M0 is set that much below the column)
        dma16(col_src, col_off);
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:192"
                     ::"v"(col_src), "s"(col_off + 12 * (TK * 16) - 192u) : "memory");
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:384"
                     ::"v"(col_src), "s"(col_off + 24 * (TK * 16) - 384u) : "memory");
        if (wave < NBLK) dma4(sp + 4 * wave, tile_off + SC_OFF + (uint32_t)wave * (TK * 4));
        if (SEL && wave == 0) mark(r, tile_off);
    };
    // pieces first, first + stride, ... of a tile
    auto part = [&](int r, uint32_t tile_off, int first, int stride) {
        const uint64_t rp = row_ptr(r), sp = sc_ptr(r);
#pragma unroll
        for (int pc = 0; pc < NCOL + NBLK; pc++)
            if (pc >= first && (pc - first) % stride == 0) piece(pc, rp, sp, tile_off);
        if (SEL && first == 0) mark(r, tile_off);
    };
    // Tile 0 is fetched by everybody at once, and tile 1 right behind it by waves 10 and 11,
    // which have no part in the preparation of Q (the memory pipeline takes a copy every few
    // dozen cycles while every workgroup starts cold, and the first tiles of all workgroups are
    // a third of the cache: the memory system has to start on them at once).  Tile 2 follows
    // behind the first barrier, a quarter from each value wave while the scoring waves read
    // their Q back: two waves that issued tiles 1 and 2 whole held that barrier back by
    // 3 000 cycles.  From step 0 on tile t+3 is fetched during step t, every wave its share.
    int r12[2] = {row_of(1), row_of(2)};
    // (list entries are loads: in before the first copy goes out, or the wait for them would
    // sit out the copies)
    int r0 = row_of(0);
    if (SEL) asm volatile("" : "+v"(r0), "+v"(r12[0]), "+v"(r12[1])::"memory");
    // The query goes first: the copies of a compute unit queue up in one memory pipeline, and a
    // Q load behind forty of them arrives thousands of cycles late (the preparation of Q is
    // what the first barrier waits for).  Its loads are written in assembly like the copies, so
    // that the wait for them can leave the copies issued behind them in flight (a wait that the
    // compiler places counts only the loads it knows).
    u32x4 qraw[4];            // (no initialiser and one definition: a second one would make the compiler copy registers whose loads are still in flight)
    if (wave < 10) {
        const int hhu = wave / 5, b = wave % 5;
        int head = hb * HW + 16 * hhu + n;
        if (head >= p.nh) head = p.nh - 1;
        const uint16_t *src = p.q + ((size_t)y * p.nh + head) * KDIM + (b < 4 ? 128 * b + 32 * g : 512 + 32 * (g & 1));
        asm volatile("global_load_dwordx4 %0, %4, off\n\t"
                     "global_load_dwordx4 %1, %4, off offset:16\n\t"
                     "global_load_dwordx4 %2, %4, off offset:32\n\t"
                     "global_load_dwordx4 %3, %4, off offset:48"
                     : "=&v"(qraw[0]), "=&v"(qraw[1]), "=&v"(qraw[2]), "=&v"(qraw[3]) : "v"(src) : "memory");
    }
    if (n_tiles > 0) share(r0, lds0);
    const bool half_of_1 = wave >= 10 && n_tiles > 1;
    if (half_of_1) part(r12[0], lds0 + TILE_B, wave == 10 ? 0 : 1, 2);      // 21 pieces or 20

    // ---- Q for 2 x 16 heads as two E4M3 terms per 32-dim block with one E8M0 scale per head and
    // 128-dim block (the hardware pairs the scale of lane (n, g) with k-elements that live in other
    // lanes of the same head, so the four lanes must agree; both terms use it).
    // lane (n, g) holds head n of the half, dims 128 b + 32 g + [0, 32); the rope block is one
    // register set: lanes g < 2 hold the hi term of dims 512 + 32 g.., lanes g >= 2 the lo term of
    // dims 512 + 32 (g - 2).. (the key side repeats its bytes).  Unit u = 5 hhu + b is prepared
    // by wave u and parked in the last tile stage and the exchange area (neither in use yet).
    {
        QPark *park = reinterpret_cast<QPark *>(&sm.tile[NST - 1]);
        if (wave < 10) {
            const int u = wave;
            const int b = u % 5;
            // the share of tile 0 (three columns, and a scale block for the first five waves) stays in flight
            if (n_tiles <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else if (wave < NBLK) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
            // the registers count as written here, behind the waits
            asm volatile("" : "+v"(qraw[0]), "+v"(qraw[1]), "+v"(qraw[2]), "+v"(qraw[3])::"memory");
            float qv[32];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const u32x4 w = qraw[c];
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    qv[8 * c + 2 * d] = bf16lo_to_f32(w[d]);
                    qv[8 * c + 2 * d + 1] = bf16hi_to_f32(w[d]);
                }
            }
            float am4[4] = {0.0f, 0.0f, 0.0f, 0.0f};      // four chains: a link waits for the one before it
#pragma unroll
            for (int j = 0; j < 32; j++) am4[j & 3] = fmaxf(am4[j & 3], __builtin_fabsf(qv[j]));
            float amax = fmaxf(fmaxf(am4[0], am4[1]), fmaxf(am4[2], am4[3]));
            amax = xor16_max(amax);
            amax = xor32_max(amax);
            int s = amax > 0.0f ? (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFFu) - 127 - 7 : 0;
            s = s < -110 ? -110 : s;
            const float inv = pow2i(-s), mul = pow2i(s);
            QPark *qp = park + u;
            const bool rope_lo = b == 4 && g >= 2;
#pragma unroll
            for (int d = 0; d < 8; d++) {
                int wh = 0, wl = 0;
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++) {
                    const float a0 = qv[4 * d + 2 * h2], a1 = qv[4 * d + 2 * h2 + 1];
                    if (h2 == 0) wh = __builtin_amdgcn_cvt_pk_fp8_f32(a0 * inv, a1 * inv, wh, false);
                    else wh = __builtin_amdgcn_cvt_pk_fp8_f32(a0 * inv, a1 * inv, wh, true);
                    const f32x2 back = h2 == 0 ? __builtin_amdgcn_cvt_pk_f32_fp8(wh, false) : __builtin_amdgcn_cvt_pk_f32_fp8(wh, true);
                    const float r0 = a0 - back[0] * mul, r1 = a1 - back[1] * mul;
                    if (h2 == 0) wl = __builtin_amdgcn_cvt_pk_fp8_f32(r0 * inv, r1 * inv, wl, false);
                    else wl = __builtin_amdgcn_cvt_pk_fp8_f32(r0 * inv, r1 * inv, wl, true);
                }
                qp->hi[d][lane] = rope_lo ? wl : wh;
                qp->lo[d][lane] = wl;
            }
            qp->sc[lane] = 127 + s;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // tile 0 has landed (this wave's share)
        } else if (half_of_1) {
            // the share of tile 0 was issued before the copies of tile 1, which stay in flight
            if (wave == 10) asm volatile("s_waitcnt vmcnt(21)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        LDS_BARRIER();
    }
    static_assert(NCOL + NBLK == 41, "the counts of copies in flight above and below");

    const float c0 = p.scale * 1.44269504088896340736f;   // scores in log2 units
    float m_ref[2] = {-INFINITY, -INFINITY};          // of head 16 h2 + n; every wave tracks the same values

    if (scorer) {
        i32x8 qhi[4], qlo[4], qrope;
        int qsc0 = 0, qsc1 = 0;                           // scale bytes of blocks 0..3 / of the rope block
        QPark *park = reinterpret_cast<QPark *>(&sm.tile[NST - 1]);
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const QPark *qp = park + 5 * hh + b;
#pragma unroll
            for (int d = 0; d < 8; d++) {
                qhi[b][d] = qp->hi[d][lane];
                qlo[b][d] = qp->lo[d][lane];
            }
            qsc0 |= qp->sc[lane] << (8 * b);
        }
        {
            const QPark *qp = park + 5 * hh + 4;
#pragma unroll
            for (int d = 0; d < 8; d++) qrope[d] = qp->hi[d][lane];
            qsc1 = qp->sc[lane];
        }
        LDS_BARRIER();                                // before copies or weights land in the park area
        // Nothing the compiler has in flight may cross into the loop: its waits would also wait
        // for the copies.
        asm volatile("" : "+v"(qhi[0]), "+v"(qhi[1]), "+v"(qhi[2]), "+v"(qhi[3]), "+v"(qlo[0]), "+v"(qlo[1]), "+v"(qlo[2]), "+v"(qlo[3]), "+v"(qrope), "+v"(qsc0), "+v"(qsc1));

        float l_priv = 0.0f, l_pend = 0.0f;               // sum over this lane's keys (head 16 hh + n), relative to m_ref / to the tile's m_loc
        float mr = -INFINITY;                             // m_ref of this wave's head half
        // per-lane LDS offsets inside a tile: K fragment (key 16 kb + n, columns 8 b + 2 g and the
        // next), the rope block's (columns 32 + 2 (g & 1)), this lane's four keys' scales
        const uint32_t k_off = (uint32_t)((2 * g) * (TK * 16) + (16 * kb + n) * 16);
        const uint32_t kr_off = (uint32_t)((32 + 2 * (g & 1)) * (TK * 16) + (16 * kb + n) * 16);
        const uint32_t s_off = SC_OFF + (uint32_t)((16 * kb + 4 * g) * 4);
        // where this lane's four probabilities go: keys 16 (kb & 1) + 4 g + i of half kb >> 1
        const uint32_t xp_off = (uint32_t)(((((hh * 2 + (kb >> 1)) * 4 + 2 * (kb & 1) + (g >> 1)) * 16 + n) * 4 + 2 * (g & 1)) * 4);
        const uint32_t xm_off = XM_OFF + (uint32_t)(((hh * 16 + n) * 4 + kb) * 4);
        const uint32_t xmr_off = XM_OFF + (uint32_t)((hh * 16 + n) * 4 * 4);
        const uint32_t xf_off = XF_OFF + (uint32_t)(wave * 4);
        const int tail_tile = n_tiles - 1;
        const bool ragged = (n_keys & (TK - 1)) != 0;

#pragma clang loop unroll(disable)
        for (int t = -1; t < n_tiles; t++) {
            const uint32_t xb = lds0 + X_OFF + (uint32_t)(t & 1) * XCH_B;         // exchange area of tile t
            const bool do_copy = t >= 0 && t + 3 < n_tiles;
            const int r_cp = do_copy ? row_of(t + 3) : -1;    // fetched here (a list entry is a load), used at the end of the step
            if (t >= 0) {
                // did any scoring wave move its reference in tile t?  (rare after the first tiles)
                const u32x4 f0 = LDS_AT(lds_u32x4, xb + XF_OFF), f1 = LDS_AT(lds_u32x4, xb + XF_OFF + 16);
                const uint32_t any_moved = (f0[0] | f0[1] | f0[2] | f0[3]) | (f1[0] | f1[1] | f1[2] | f1[3]);
                if (__builtin_amdgcn_readfirstlane(any_moved) != 0u) {
                    const f32x4 ml = LDS_AT(lds_f32x4, xb + xmr_off);
                    const float m_new = fmaxf(mr, fmaxf(fmaxf(ml[0], ml[1]), fmaxf(ml[2], ml[3])));
                    const float mo = kb == 0 ? ml[0] : kb == 1 ? ml[1] : kb == 2 ? ml[2] : ml[3];
                    const float fo = mo == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mo - m_new);
                    const float c = mr == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(mr - m_new);
                    l_priv = l_priv * c + fo * l_pend;
                    mr = m_new;
                } else {
                    l_priv += l_pend;
                }
            }
            if (t + 1 < n_tiles) {
                // ---- scores S^T[key][head] for keys 16 kb.., heads 16 hh.. of tile t+1 ----
                const uint32_t tb = lds0 + (uint32_t)((t + 1) & (NST - 1)) * TILE_B;
                const uint32_t xn = lds0 + X_OFF + (uint32_t)((t + 1) & 1) * XCH_B;
                const uint32_t ka = tb + k_off, kr = tb + kr_off, sa = tb + s_off;
                auto kfrag = [&](int b) -> i32x8 {
                    const uint32_t a = b < 4 ? ka + (uint32_t)(8 * b) * (TK * 16) : kr;
                    const u32x4 k0 = LDS_AT(lds_u32x4, a);
                    const u32x4 k1 = LDS_AT(lds_u32x4, a + TK * 16);
                    return (i32x8){(int)k0[0], (int)k0[1], (int)k0[2], (int)k0[3], (int)k1[0], (int)k1[1], (int)k1[2], (int)k1[3]};
                };
                const f32x4 z4 = {0.0f, 0.0f, 0.0f, 0.0f};
                f32x4 S;
                i32x8 kA = kfrag(0);
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const i32x8 kN = kfrag(b + 1);
                    const f32x4 scb = LDS_AT(lds_f32x4, sa + (uint32_t)b * (TK * 4));
                    f32x4 acc;
                    if (b == 0) {
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qhi[b], z4, 0, 0, 0, 0x7F7F7F7F, 0, qsc0);
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qlo[b], acc, 0, 0, 0, 0x7F7F7F7F, 0, qsc0);
                    } else if (b == 1) {
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qhi[b], z4, 0, 0, 0, 0x7F7F7F7F, 1, qsc0);
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qlo[b], acc, 0, 0, 0, 0x7F7F7F7F, 1, qsc0);
                    } else if (b == 2) {
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qhi[b], z4, 0, 0, 0, 0x7F7F7F7F, 2, qsc0);
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qlo[b], acc, 0, 0, 0, 0x7F7F7F7F, 2, qsc0);
                    } else {
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qhi[b], z4, 0, 0, 0, 0x7F7F7F7F, 3, qsc0);
                        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qlo[b], acc, 0, 0, 0, 0x7F7F7F7F, 3, qsc0);
                    }
                    if (b == 0) S = acc * scb;
                    else S += acc * scb;
                    kA = kN;
                }
                {
                    const f32x4 scb = LDS_AT(lds_f32x4, sa + 4u * (TK * 4));
                    const f32x4 acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(kA, qrope, z4, 0, 0, 0, 0x7F7F7F7F, 0, qsc1);
                    S += acc * scb;
                }
                S *= c0;
                // masked positions: past the end of the list (only the last tile of a dense list),
                // or entries of sel[] that name no row
                if (SEL ? true : (ragged && t + 1 == tail_tile)) {
                    uint64_t valid;
                    if (SEL) {
                        const u32x2 vw = LDS_AT(lds_u32x2, tb + VALID_OFF);
                        valid = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)vw[0]) |
                                ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)vw[1]) << 32);
                    } else {
                        valid = __ballot(row_of(t + 1) >= 0);
                    }
                    if (valid != ~0ull) {
                        const uint32_t bits = (uint32_t)(valid >> (16 * kb)) >> (4 * g);
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            if (!((bits >> i) & 1u)) S[i] = -INFINITY;
                    }
                }
                float lmax = vmax3(S[0], S[1], vmax(S[2], S[3]));
                float m_loc = mr;
                const bool moves = __any(lmax > mr + LAZY);   // rare after the first tiles: only then the lanes of a head confer
                if (moves) {
                    lmax = xor16_max(lmax);
                    lmax = xor32_max(lmax);
                    m_loc = lmax > mr + LAZY ? lmax : mr;
                }
                const float m_use = m_loc == -INFINITY ? 0.0f : m_loc;
                f32x4 P;
#pragma unroll
                for (int i = 0; i < 4; i++) P[i] = __builtin_amdgcn_exp2f(S[i] - m_use);
                l_pend = (P[0] + P[1]) + (P[2] + P[3]);   // of this lane's four keys, relative to m_loc
                {
                    u32x2 d;
                    d[0] = pack_f16_rne(P[0], P[1]);
                    d[1] = pack_f16_rne(P[2], P[3]);
                    LDS_AT(lds_u32x2, xn + xp_off) = d;
                }
                // the reference this key block used (the four lanes of a head write the same word)
                // and whether it differs from the one every wave holds
                LDS_AT(lds_f32, xn + xm_off) = m_loc;
                LDS_AT(lds_u32, xn + xf_off) = moves ? 1u : 0u;
            }
            // the copies this wave issued a step ago (its share of tile t+2) have long landed; its
            // share of tile t+3 goes out now, when the wave would otherwise wait at the barrier
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (do_copy) share(r_cp, lds0 + (uint32_t)((t + 3) & (NST - 1)) * TILE_B);
            LDS_BARRIER();
        }

        // ---- the sums of the scoring role meet in LDS (the exchange area is free now) ----
        float *lsum = reinterpret_cast<float *>(&sm.x[0]);            // [head half][head][key block]
        float ls = xor16_sum(l_priv);
        ls = xor32_sum(ls);
        if (g == 0) lsum[(hh * 16 + n) * 4 + kb] = ls;
        LDS_BARRIER();
    } else {
        // tile 2 (stage 2; Q is parked in the last stage and the exchange area): pieces cw, cw + 4, ...
        const bool quarter_of_2 = n_tiles > 2;
        if (quarter_of_2) part(r12[1], lds0 + 2 * TILE_B, cw, 4);           // 11 pieces for cw = 0, else 10
        LDS_BARRIER();                                // before copies or weights land in the park area
        f32x4 oacc[2][8];                                 // [head half][dim block]: dims 128 cw + 16 j + 4 g + i, head n
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
            for (int j = 0; j < 8; j++) oacc[h2][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        int e_run = E_NONE;                               // 2^e_run is above every scale of this wave's block seen so far
        uint32_t thr_bits = 0u;                           // bits of 2^e_run: a scale whose bits reach them does not fit
        float wfac = 0.0f;                                // 2^(WEXP - e_run)
        // the value wave shares its SIMD with two scoring waves that stream MFMAs: without priority
        // its many short VALU instructions wait behind them and it becomes the long pole of the step
        __builtin_amdgcn_s_setprio(3);
        // transpose-read addressing for V^T: lane i of 16-lane group g supplies key 8 g + (i >> 1),
        // bytes 8 (i & 1) .. +7 of the sixteen-byte column
        const uint32_t tr_off = (uint32_t)((8 * cw) * (TK * 16) + (8 * g + (n >> 1)) * 16 + 8 * (n & 1));
        // the two scales this lane turns into a pair of factors (see the loop)
        const uint32_t sv_off = SC_OFF + (uint32_t)(cw * (TK * 4) + (32 * ((n & 7) >> 2) + 8 * g + 2 * (n & 3)) * 4);
        // the probabilities of this lane's slots: [head half][key half][g][n][4 dwords]
        const uint32_t pw_off = (uint32_t)((g * 16 + n) * 16);
        const uint32_t xml_off = XM_OFF + (uint32_t)(n * 16);
        asm volatile("" ::: "memory");
        int r_cp = row_of(3);                             // rows of the tile copied in step 0; a list entry is a load: fetched a step ahead
#pragma clang loop unroll(disable)
        for (int t = -1; t < n_tiles; t++) {
            const bool do_copy = t >= 0 && t + 3 < n_tiles;
            if (do_copy) {
                share(r_cp, lds0 + (uint32_t)((t + 3) & (NST - 1)) * TILE_B);   // the stage tile t-1 left at the last barrier
                r_cp = row_of(t + 4);
            }
            if (t >= 0) {
                // ---- values O^T[dim][head] += V^T W^T for dims 128 cw.., all 32 heads, tile t ----
                const uint32_t tb = lds0 + (uint32_t)(t & (NST - 1)) * TILE_B;
                const uint32_t xb = lds0 + X_OFF + (uint32_t)(t & 1) * XCH_B;
                // The sixteen lanes of a row share their contraction slots (keys 8 g .. 8 g + 7 of each
                // half), so a row needs eight fp16 pairs of scale factors per tile: lane (g, n) reads
                // the two scales of pair n & 7 (half (n & 7) >> 2, keys 8 g + 2 (n & 3) and the next),
                // forms that one pair, and every lane takes the eight pairs out of the row by DPP.
                const f32x2 sv = LDS_AT(lds_f32x2, tb + sv_off);
                u32x4 pw[2][2];                           // [head half][key half]
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
                    for (int kh = 0; kh < 2; kh++) pw[h2][kh] = LDS_AT(lds_u32x4, xb + pw_off + (uint32_t)((h2 * 2 + kh) * 1024));
                const u32x4 f0 = LDS_AT(lds_u32x4, xb + XF_OFF), f1 = LDS_AT(lds_u32x4, xb + XF_OFF + 16);
                // normaliser of the fp16 weights: a power of two above every scale seen so far (it
                // only grows, and only then the lanes confer).  Scales are compared as integers:
                // they are positive, and a negative or NaN scale has the larger bit pattern too.
                float ecorr = 1.0f;
                {
                    const uint32_t b0 = __builtin_bit_cast(uint32_t, sv[0]) & 0x7FFFFFFFu, b1 = __builtin_bit_cast(uint32_t, sv[1]) & 0x7FFFFFFFu;
                    const uint32_t smax = b0 > b1 ? b0 : b1;
                    if (__any(smax >= thr_bits && smax != 0u)) {
                        float sm_f = __builtin_bit_cast(float, smax);
                        sm_f = wave_max(sm_f);
                        const int e_tile = (int)((__builtin_bit_cast(uint32_t, sm_f) >> 23) & 0xFFu) - 126;
                        if (e_tile > e_run) {
                            if (e_run != E_NONE) ecorr = pow2i(e_run - e_tile);
                            e_run = e_tile;
                            thr_bits = __builtin_bit_cast(uint32_t, pow2i(e_run));
                            wfac = pow2i(WEXP - e_run);
                        }
                    }
                }
                const uint32_t my_pair = pack_f16_rne(sv[0] * wfac, sv[1] * wfac);
                u32x4 sw[2];                              // scale * 2^(WEXP - e_run) of the slots' keys, fp16 pairs
                sw[0][0] = row_place<0>(my_pair);
                sw[0][1] = row_place<1>(my_pair);
                sw[0][2] = row_place<2>(my_pair);
                sw[0][3] = row_place<3>(my_pair);
                sw[1][0] = row_place<4>(my_pair);
                sw[1][1] = row_place<5>(my_pair);
                sw[1][2] = row_place<6>(my_pair);
                sw[1][3] = row_place<7>(my_pair);
                const uint32_t any_moved = (f0[0] | f0[1] | f0[2] | f0[3]) | (f1[0] | f1[1] | f1[2] | f1[3]);
                if (__builtin_amdgcn_readfirstlane(any_moved) != 0u || ecorr != 1.0f) {
                    // a scoring wave left the common reference in this tile (or the weights'
                    // normaliser grew): bring accumulators and probabilities to the new maximum
#pragma unroll
                    for (int h2 = 0; h2 < 2; h2++) {
                        const f32x4 ml = LDS_AT(lds_f32x4, xb + xml_off + (uint32_t)(h2 * 256));
                        const float m_new = fmaxf(m_ref[h2], fmaxf(fmaxf(ml[0], ml[1]), fmaxf(ml[2], ml[3])));
                        float f[4];
#pragma unroll
                        for (int k = 0; k < 4; k++) f[k] = ml[k] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ml[k] - m_new);
                        const float c = (m_ref[h2] == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_ref[h2] - m_new)) * ecorr;
                        m_ref[h2] = m_new;
#pragma unroll
                        for (int j = 0; j < 8; j++) oacc[h2][j] *= c;
                        // probabilities were taken relative to each key block's own reference: bring
                        // them to m_new (slot group g of half kh holds keys of key block 2 kh + g / 2)
                        const float fsel0 = (g >> 1) ? f[1] : f[0];
                        const float fsel1 = (g >> 1) ? f[3] : f[2];
#pragma unroll
                        for (int kh = 0; kh < 2; kh++)
#pragma unroll
                            for (int d = 0; d < 4; d++) pw[h2][kh][d] = scale_f16x2(pw[h2][kh][d], kh ? fsel1 : fsel0);
                    }
                }
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
                    for (int kh = 0; kh < 2; kh++)
#pragma unroll
                        for (int d = 0; d < 4; d++) pw[h2][kh][d] = mul_f16x2(pw[h2][kh][d], sw[kh][d]);
                const uint32_t va0 = tb + tr_off;
#pragma unroll
                for (int j0 = 0; j0 < 8; j0 += 4) {
                    i32x2 vt[4][2];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int kh = 0; kh < 2; kh++)
                            vt[j][kh] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2 *)(size_t)(va0 + (uint32_t)((j0 + j) * (TK * 16) + kh * (32 * 16))));
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int kh = 0; kh < 2; kh++) {
                            u32x4 vh;
                            vh[0] = e4m3x2_to_f16x2<false>((uint32_t)vt[j][kh][0]);
                            vh[1] = e4m3x2_to_f16x2<true>((uint32_t)vt[j][kh][0]);
                            vh[2] = e4m3x2_to_f16x2<false>((uint32_t)vt[j][kh][1]);
                            vh[3] = e4m3x2_to_f16x2<true>((uint32_t)vt[j][kh][1]);
                            const f16x8 va = __builtin_bit_cast(f16x8, vh);
                            oacc[0][j0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(f16x8, pw[0][kh]), oacc[0][j0 + j], 0, 0, 0);
                            oacc[1][j0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(f16x8, pw[1][kh]), oacc[1][j0 + j], 0, 0, 0);
                        }
                }
            }
            // tile t+2 must be whole at the next barrier; the share of tile t+3 issued in this
            // step (three copies) may stay in flight, and in step -1 this wave's quarter of tile 2,
            // which is needed one step later than tile 1
            if (do_copy) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
            else if (t < 0 && quarter_of_2) {
                if (cw == 0) asm volatile("s_waitcnt vmcnt(11)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
            } else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            LDS_BARRIER();
        }

        const float *lsum = reinterpret_cast<const float *>(&sm.x[0]);
        LDS_BARRIER();
        // ---- every value wave owns its dims: write the partial (or the result) directly ----
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
            const f32x4 lv = *(const f32x4 *)&lsum[(h2 * 16 + n) * 4];
            float L = (lv[0] + lv[1]) + (lv[2] + lv[3]);
            const int head = hb * HW + 16 * h2 + n;
            if (head >= p.nh) continue;
            // the attention sink of src/ds_model.c:946: one more term in the denominator, no value
            // (with several splits the merge kernel adds it)
            if (p.sink && p.n_splits == 1 && m_ref[h2] > -INFINITY)
                L += __builtin_amdgcn_exp2f(p.sink[head] * 1.44269504088896340736f - m_ref[h2]);
            const float unit_f = e_run == E_NONE ? 0.0f : pow2i(e_run - WEXP);   // the accumulators are in units of 2^(e_run - WEXP)
            const float fin = p.n_splits == 1 ? (L > 0.0f ? unit_f / L : 0.0f) : unit_f;
            const size_t pb = ((size_t)y * p.n_splits + split) * (2 * n_hb) + 2 * hb + h2;
            if (p.n_splits == 1) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    // accumulator register i <-> dim 16 db + 4 g + i
                    const f32x4 v = oacc[h2][j] * fin;
                    *(f32x4 *)(p.out + ((size_t)y * p.nh + head) * VDIM + 16 * (8 * cw + j) + 4 * g) = v;
                }
                continue;
            }
            // The partial leaves as 16-bit fixed point: this wave's 128 dims of the head share one
            // scale, their largest magnitude, so every value is off by at most 2^-16 of that.  A
            // non-finite value makes the scale NaN and with it the head's merged output.
            // (the largest magnitude as an integer maximum of the bit patterns without their signs:
            // infinities and NaNs compare above every finite value; four chains, because each link
            // waits for the one before it, and the four lanes of a head meet without a trip
            // through LDS)
            uint32_t b0 = 0u, b1 = 0u, b2 = 0u, b3 = 0u;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const u32x4 a = __builtin_bit_cast(u32x4, oacc[h2][j]) & 0x7FFFFFFFu;
                b0 = a[0] > b0 ? a[0] : b0;
                b1 = a[1] > b1 ? a[1] : b1;
                b2 = a[2] > b2 ? a[2] : b2;
                b3 = a[3] > b3 ? a[3] : b3;
            }
            uint32_t bm = b0 > b1 ? b0 : b1;
            const uint32_t bn = b2 > b3 ? b2 : b3;
            bm = bm > bn ? bm : bn;
            bm = lanes_xor16_max(bm);
            bm = lanes_xor32_max(bm);
            float big = bm > 0x7F7FFFFFu ? __builtin_nanf("") : __builtin_bit_cast(float, bm);   // in accumulator units
            const float to_unit = big > 0.0f ? 1.0f / big : 0.0f;
            uint32_t *pq = p.part_acc + (pb * NDB + 8 * cw) * 128 + lane * 2;   // [db][lane][4 x i16]
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const f32x4 v = oacc[h2][j] * to_unit;
                u32x2 w;
                w[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pknorm_i16(v[0], v[1]));
                w[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pknorm_i16(v[2], v[3]));
                // written through to memory as it is stored: the merge runs on other XCDs, and what
                // would otherwise sit dirty in this L2 is written back at the end of the kernel,
                // on the critical path (about 1 us for the 8 MB of a full-chip launch)
                __hip_atomic_store((uint64_t *)(pq + j * 128), __builtin_bit_cast(uint64_t, w), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_SYSTEM);
            }
            if (g == 0)
                *(f32x4 *)(p.part_ml + ((pb * 4 + cw) * HB + n) * 4) =
                    (f32x4){m_ref[h2] * 0.69314718055994530942f, L, big * fin * (1.0f / 32767.0f), 0.0f};
        }
    }
}

// merge of fragment-layout partials: values [y][split][16-head block][dim block][lane][4] as
// 16-bit fixed point, and per 16-head block and quarter of the dims [head][4] floats (running
// maximum in natural-log units, weight sum, value of one fixed-point step, unused).  With more
// than eight splits a workgroup is one dim block of one 16-head block: its waves (eight up to
// 64 splits, where a wave then has its eight loads in flight at once: 4.55 -> 4.16 us; sixteen
// beyond) take splits w, w + n_waves, ... and meet in LDS.  With up to eight a wave merges a dim block alone and
// eight of them make a workgroup (a batch of queries splits each query less: one wave per
// split would be thousands of workgroups that each wait out one load).  Every wave has all its
// loads in flight at once (eight splits per batch); which splits exist is uniform per wave, so
// absent ones cost nothing.
constexpr int MW = 16;
__device__ __forceinline__ void merge_add(f32x4 &acc, float &ls, const u32x2 a, const f32x4 v, const float mx) {
    const float c = v[0] == -INFINITY ? 0.0f : __expf(v[0] - mx);
    ls = __builtin_fmaf(v[1], c, ls);
    const float cs = c * v[2];
    acc[0] = __builtin_fmaf((float)((int32_t)(a[0] << 16) >> 16), cs, acc[0]);
    acc[1] = __builtin_fmaf((float)((int32_t)a[0] >> 16), cs, acc[1]);
    acc[2] = __builtin_fmaf((float)((int32_t)(a[1] << 16) >> 16), cs, acc[2]);
    acc[3] = __builtin_fmaf((float)((int32_t)a[1] >> 16), cs, acc[3]);
}
__global__ void __launch_bounds__(64 * MW)
mla_merge_frag16_kernel(const uint32_t *__restrict__ part_acc, const float *__restrict__ part_ml,
                        int n_splits, int n_hb16, int nh, const float *__restrict__ sink,
                        float *__restrict__ out, int packed) {
    __shared__ float red_m[MW][64];
    __shared__ float red_l[MW][64];
    __shared__ f32x4 red_a[MW][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), y = blockIdx.y;
    int wv, mw, db, hb;
    if (packed) {
        // up to eight splits: a wave merges a dim block by itself, and the workgroup's eight
        // waves take the eight dim blocks of one quarter
        wv = 0, mw = 1, db = 8 * (int)(blockIdx.x & 3) + wave, hb = (int)(blockIdx.x >> 2);
    } else {
        // workgroups go to the eight XCDs round robin: the eight dim blocks that share a quarter's
        // [head][4] floats sit on one XCD, so that only one L2 fetches them (n_hb16 is even)
        const int grp = (int)(blockIdx.x & 7) + 8 * (int)(blockIdx.x >> 6);
        wv = wave, mw = (int)blockDim.x >> 6;
        db = 8 * (grp & 3) + (int)((blockIdx.x >> 3) & 7), hb = grp >> 2;
    }
    const int n = lane & 15, g = lane >> 4;
    const size_t sb = (size_t)y * n_splits;
    const float *ml = part_ml + (((sb * n_hb16 + hb) * 4 + (db >> 3)) * HB + n) * 4;
    const size_t ml_stride = (size_t)n_hb16 * 4 * HB * 4;
    const uint32_t *pa = part_acc + ((sb * n_hb16 + hb) * NDB + db) * 128 + lane * 2;
    const size_t pa_stride = (size_t)n_hb16 * NDB * 128;

    // first batch: everything in flight before anything is waited for
    u32x2 a0[8];
    f32x4 v0[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int s = wv + mw * j;
        v0[j] = (f32x4){-INFINITY, 0.0f, 0.0f, 0.0f};
        a0[j] = (u32x2){0u, 0u};
        if (s < n_splits) {
            v0[j] = *(const f32x4 *)(ml + s * ml_stride);
            a0[j] = *(const u32x2 *)(pa + s * pa_stride);
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; j++) mx = fmaxf(mx, v0[j][0]);
    for (int s = wv + 8 * mw; s < n_splits; s += mw) mx = fmaxf(mx, ml[s * ml_stride]);
    if (mw > 1) {
        red_m[wv][lane] = mx;
        __syncthreads();
        for (int w = 0; w < mw; w++) mx = fmaxf(mx, red_m[w][lane]);
    }

    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float ls = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) merge_add(acc, ls, a0[j], v0[j], mx);
    for (int s0 = wv + 8 * mw; s0 < n_splits; s0 += 8 * mw) {
        u32x2 a[8];
        f32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = s0 + mw * j;
            v[j] = (f32x4){-INFINITY, 0.0f, 0.0f, 0.0f};
            a[j] = (u32x2){0u, 0u};
            if (s < n_splits) {
                v[j] = *(const f32x4 *)(ml + s * ml_stride);
                a[j] = *(const u32x2 *)(pa + s * pa_stride);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) merge_add(acc, ls, a[j], v[j], mx);
    }
    float l = ls;
    f32x4 r4 = acc;
    if (mw > 1) {
        red_l[wv][lane] = ls;
        red_a[wv][lane] = acc;
        __syncthreads();
        if (wv != 0) return;
        l = 0.f;
        r4 = (f32x4){0.f, 0.f, 0.f, 0.f};
        for (int w = 0; w < mw; w++) {
            l += red_l[w][lane];
            const f32x4 t = red_a[w][lane];
#pragma unroll
            for (int r = 0; r < 4; r++) r4[r] += t[r];
        }
    }
    const int head = hb * HB + n;
    if (head >= nh) return;
    if (sink && mx > -INFINITY) l += __expf(sink[head] - mx);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) r4[r] *= inv;
    // accumulator register i <-> dim 16 db + 4 g + i
    *(f32x4 *)(out + ((size_t)y * nh + head) * VDIM + 16 * db + 4 * g) = r4;
}

// Split-K partials of the entry point that may not allocate (cwick_hip_mla_decode_static_dev):
// a fixed area in the library's own device image instead of the grow-only workspace.  Host code
// never uses the array's name as an address: static_scratch() asks the runtime once where the
// device's copy lives and hands out that pointer.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

static void *static_scratch() {
    static std::once_flag once;
    static void *ptr = nullptr;
    static hipError_t err = hipSuccess;
    std::call_once(once, [] {
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) ptr = nullptr;
    });
    if (!ptr) hip_ok(err != hipSuccess ? err : hipErrorInvalidSymbol, "hipGetSymbolAddress(scratch)");
    return ptr;
}

// fixed == true: partials go to the static area, nothing is allocated and no events are created
int run(Params &p, hipStream_t s, bool fixed = false) {
    static std::once_flag attr_once;
    static hipError_t attr_err = hipSuccess;
    const size_t smem = sizeof(Smem);
    std::call_once(attr_once, [&] {
        attr_err = hipFuncSetAttribute((const void *)mla_roles_kernel<false>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (attr_err == hipSuccess)
            attr_err = hipFuncSetAttribute((const void *)mla_roles_kernel<true>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    });
    CWICK_HIP_CALL(attr_err);
    const int n_hb = (p.nh + HW - 1) / HW;
    const int64_t total = (int64_t)n_hb * p.n_splits * p.nq;
    CWICK_REQUIRE(total <= 0x7FFFFFFF, "mla: grid of %lld workgroups is too large", (long long)total);
    if (p.n_splits > 1) {
        const size_t acc_b = (size_t)p.nq * p.n_splits * n_hb * HW * VDIM * sizeof(int16_t);
        const size_t ml_b = (size_t)p.nq * p.n_splits * n_hb * HW * 4 * 4 * sizeof(float);
        char *ws;
        if (fixed) {
            CWICK_REQUIRE(acc_b + ml_b <= STATIC_SCRATCH_BYTES,
                          "mla_decode_static: the split-K partials of this call (%zu bytes) exceed the "
                          "static scratch area (%zu bytes); use cwick_hip_mla_decode_dev",
                          acc_b + ml_b, STATIC_SCRATCH_BYTES);
            ws = (char *)static_scratch();
            if (!ws) return 0;
        } else {
            ws = (char *)workspace(s, acc_b + ml_b);
            if (!ws) return 0;                      // workspace() has recorded why
        }
        p.part_acc = (uint32_t *)ws;
        p.part_ml = (float *)(ws + acc_b);
    }
    {
        ProfKernel pk(fixed ? -1 : CWICK_HIP_PROF_MLA, s);
        if (p.sel) pk.launch(mla_roles_kernel<true>, dim3((unsigned)total), dim3(THREADS), smem, p);
        else pk.launch(mla_roles_kernel<false>, dim3((unsigned)total), dim3(THREADS), smem, p);
    }
    CWICK_HIP_CALL(hipGetLastError());
    if (p.n_splits > 1) {
        ProfKernel pk(fixed ? -1 : CWICK_HIP_PROF_MLA_MERGE, s);
        if (p.n_splits <= 8)
            pk.launch(mla_merge_frag16_kernel, dim3(2 * n_hb * 4, p.nq), dim3(64 * 8), 0, p.part_acc, p.part_ml,
                      p.n_splits, 2 * n_hb, p.nh, p.sink, p.out, 1);
        else
            pk.launch(mla_merge_frag16_kernel, dim3(2 * n_hb * NDB, p.nq), dim3(64 * (p.n_splits <= 64 ? 8 : MW)), 0,
                      p.part_acc, p.part_ml, p.n_splits, 2 * n_hb, p.nh, p.sink, p.out, 0);
        CWICK_HIP_CALL(hipGetLastError());
    }
    return 1;
}

int splits_per_cu() {
    static const int v = [] {
        const char *e = getenv("CWICK_HIP_MLA_WG_PER_CU");
        const int x = e ? atoi(e) : 1;
        return (x < 1 || x > 8) ? 1 : x;
    }();
    return v;
}

}  // namespace

int launch_mla_decode(const uint8_t *rows, const float *scales, int64_t row_bstride,
                      int64_t scale_bstride, int64_t n_rows, int batch, const int32_t *sel,
                      int64_t n_list, const uint16_t *q, int n_heads, float scale, const float *sink,
                      float *out, hipStream_t s, bool fixed_scratch) {
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
    p.q = q; p.nh = n_heads; p.nq = batch; p.scale = scale; p.out = out; p.sink = sink;
    // one workgroup is resident per CU: one round of workgroups
    const int n_hb = (n_heads + HW - 1) / HW;
    int64_t want = (int64_t)splits_per_cu() * num_cus() / ((int64_t)n_hb * batch);
    if (want < 1) want = 1;
    if (want > MERGE_MAX_SPLITS) want = MERGE_MAX_SPLITS;
    int64_t per = (n_list + want - 1) / want;
    per = ((per + TK - 1) / TK) * TK;
    p.keys_per_split = per;
    p.n_splits = (int)((n_list + per - 1) / per);
    return run(p, s, fixed_scratch);
}

int launch_mla_prefill(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n,
                       const uint16_t *q, int n_heads, float scale, float *out, hipStream_t s) {
    CWICK_REQUIRE(rows && scales && q && out, "mla_prefill: null pointer");
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "mla_prefill: n_heads %d (1..128)", n_heads);
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= ((int64_t)1 << 31) - 1 && n <= (1 << 22),
                  "mla_prefill: pos0 %lld n %lld", (long long)pos0, (long long)n);
    CWICK_REQUIRE(scale > 0.0f && scale < INFINITY, "mla_prefill: scale must be positive");
    CWICK_REQUIRE((uintptr_t)rows % 16 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)out % 16 == 0,
                  "mla_prefill: rows, q and out must be 16-byte aligned");
    // 64 heads per workgroup when the query has them (mla_prefill64.hip); CWICK_HIP_MLA_PREFILL=roles
    // keeps the decode kernel's 32
    static const bool wide = [] {
        const char *e = getenv("CWICK_HIP_MLA_PREFILL");
        return !(e && !strcmp(e, "roles"));
    }();
    if (wide && n_heads > HW) return launch_mla_prefill_wide(rows, scales, pos0, n, q, n_heads, scale, out, s);
    Params p{};
    p.rows = rows; p.scales = scales; p.row_bstride = 0; p.scale_bstride = 0;
    p.n_rows = pos0 + n; p.sel = nullptr; p.n_list = pos0 + 1; p.list_step = 1;
    p.q = q; p.nh = n_heads; p.nq = (int)n; p.scale = scale; p.out = out;
    p.n_splits = 1;
    p.keys_per_split = ((pos0 + n + TK - 1) / TK) * TK;
    return run(p, s);
}

}  // namespace cwick
