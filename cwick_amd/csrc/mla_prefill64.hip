// mla_prefill64.hip -- absorbed-latent MLA chunked prefill (src/attention.c:1010-1019: one
// mla_latent_decode per query of the chunk, :749-811) with 64 query rows per key tile.
//
// The decode kernel (mla_roles.hip) gives a workgroup 32 heads of one query, and what a 64-key
// tile costs it besides the matrix work -- the copy into LDS, the handling of the block scales,
// the E4M3 -> fp16 conversion of V -- does not depend on the number of rows.  A prefill chunk has
// rows to spare, so here a workgroup takes 64 heads of one query and pays that per twice the
// matrix work.
//
//   workgroup = 8 waves (two per SIMD, 256 registers each), 64 heads x all keys of the query,
//   walked in tiles of 64 keys, three LDS stages.
//     waves 0..3 score: wave hq owns heads 16 hq .. +15 and scores them against all 64 keys of
//                the tile (four 16-key blocks): S^T = K Q^T on v_mfma_scale_f32_16x16x128_f8f6f4,
//                K as stored, Q as two E4M3 terms with one E8M0 scale per head and 128-dim block
//                (as in mla_roles.hip).  The keys' block scales sit in five registers per tile (a
//                key per lane) and enter the fold of the five block products through a DPP row
//                broadcast inside the multiply-add.  Because a wave sees every key of its heads,
//                the softmax reference of a head lives in one wave: when a tile exceeds it by
//                2^LAZY the wave moves it at once, and publishes the factor by which the
//                accumulators of that head shrink together with the fp16 probabilities of the tile.
//     waves 4..7 accumulate: wave cw owns output dims 128 cw .. +127 for all 64 heads;
//                weights p * scale[key][cw] * 2^(10 - e) in fp16, O^T += V^T W^T on
//                v_mfma_f32_16x16x32_f16, every converted V^T fragment used four times.
//   The roles run one tile apart (tile t+1 is scored while tile t is accumulated): one barrier
//   per step.  Tile t+2 is copied (global_load_lds, issued from assembly) at the top of step t
//   into the stage tile t-1 left at the last barrier, by the value waves alone: a wave stalls
//   while the memory pipeline takes its copies, and the scoring waves are the longer pole of a
//   step (copies dealt to all eight waves: 36.1 ms for 4096 queries over 28672 + 4096 rows,
//   by the value waves: 31.2; spreading them over the step or issuing them a step earlier into
//   the columns a value wave has just finished with: 31.1 and 34).
//   One slice per query: no partials, the value waves write the output.
//   Per tile the workgroup reads about 275 KB from LDS (160 KB of K fragments, 32 KB of V^T, 32 KB
//   of probabilities, the scale registers) and the copies write 37 KB; with the scales as twenty
//   16-byte fragments per scoring wave it was 350 KB and the kernel 7 % slower.
//   Ablation builds at 31 ms: without the value MFMAs and conversions 21.7, without the score
//   MFMAs and K reads 22.4, without the K reads alone 27.3: the two roles weigh the same and
//   mostly add up; the matrix pipe is busy 2 176 of about 4 200 cycles per step and SIMD.
//   Every K fragment is read from LDS by all four scoring waves (160 KB per tile); a timing build
//   that read half of them ran 11 % faster (3 % since the scales are registers).  A scoring wave
//   of 32 heads x 32 keys would read each
//   fragment twice instead of four times, but its Q operands alone are 144 registers: with the
//   loop's other values that does not fit the 256 of a wave (built: 24 of them reloaded from
//   scratch every step), and Q fragments re-read from LDS give back what the K reads saved.
#include "common.hpp"

#include <cstdlib>
#include <mutex>

namespace cwick {
namespace {

constexpr int KDIM = CWICK_HIP_LATENT_KDIM;   // 576
constexpr int VDIM = CWICK_HIP_LATENT_VDIM;   // 512
constexpr int NBLK = CWICK_HIP_LATENT_NBLK;   // 5
constexpr int THREADS = 512;                  // waves 0..3 score, waves 4..7 accumulate values
constexpr int NWAVES = THREADS / 64;
constexpr int TK = 64;                        // keys per tile
constexpr int HW = 64;                        // heads per workgroup
constexpr int NHQ = HW / 16;                  // 16-head blocks = scoring waves
constexpr int NST = 3;                        // tile stages
constexpr int NCOL = KDIM / 16;               // 36 sixteen-byte columns per row
constexpr float LAZY = 10.0f;                 // the reference moves when a tile exceeds it by 2^LAZY (fp16 probabilities up to 2^10)
constexpr int WEXP = 4;                       // fp16 weights are p * scale * 2^(WEXP - e), scale < 2^e: below 2^(LAZY + WEXP) = 2^14
constexpr int E_NONE = -1000;                 // no scale seen yet

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) u32x2 lds_u32x2;
typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
typedef __attribute__((address_space(3))) f32x2 lds_f32x2;
typedef __attribute__((address_space(3))) float lds_f32;
typedef __attribute__((address_space(3))) uint32_t lds_u32;

struct WideParams {
    const uint8_t *rows;
    const float *scales;
    int64_t pos0;             // query y sees rows 0 .. pos0 + y
    const uint16_t *q;        // [nq][nh][576] bf16
    int nh, nq;
    float scale;
    float *out;               // [nq][nh][512]
};

// what a position past the end of a query's keys is fetched from (see mla_roles.hip)
__device__ __attribute__((aligned(16))) uint8_t g_zero_row64[KDIM + 64] = {0};
__device__ __attribute__((aligned(16))) float g_zero_scales64[8] = {0.0f};

struct Tile {
    uint8_t kv[NCOL][TK][16];     // [16-byte column][key][16]     36864 B
    float sc[NBLK][TK];           // [block][key]                   1280 B
    uint32_t pad[4];
};
struct Xch {                       // what the scoring waves publish per tile
    // fp16 probabilities exp2(s - m) as the B fragments of the value MFMA:
    // [16-head block][32-key half][slot group g][head n][4 dwords]; contraction slot 8 g + j of a
    // half is key 8 g + j of that half
    uint32_t p[NHQ][2][4][16][4];
    float c[NHQ][16];             // by what the accumulators of head (hq, n) shrink before this tile
    uint32_t moved[NHQ];          // scoring wave hq moved a reference in this tile
    uint32_t pad[12];
};
struct Smem {
    Tile tile[NST];
    Xch x[2];
};
// Q of one (16-head block, 128-dim block) in MFMA operand order, dword-interleaved by lane; for
// the rope block `hi` is the combined hi|lo register set
struct QPark { int hi[8][64]; int lo[8][64]; int sc[64]; };
static_assert(5 * NHQ * sizeof(QPark) <= 2 * sizeof(Tile) + 2 * sizeof(Xch), "Q park area");
static_assert(sizeof(Smem) <= 160 * 1024, "LDS");

__device__ __forceinline__ float pow2i(int e) {
    e = e > 126 ? 126 : (e < -126 ? -126 : e);
    return __builtin_bit_cast(float, (uint32_t)(e + 127) << 23);
}
__device__ __forceinline__ uint32_t mul_f16x2(uint32_t a, uint32_t b) {
    const f16x2 r = __builtin_bit_cast(f16x2, a) * __builtin_bit_cast(f16x2, b);
    return __builtin_bit_cast(uint32_t, r);
}
#define LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")
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
#define LDS_AT(type, a) (*(type *)(size_t)(uint32_t)(a))

constexpr uint32_t TILE_B = sizeof(Tile);
constexpr uint32_t SC_OFF = NCOL * TK * 16;                       // Tile::sc
constexpr uint32_t X_OFF = NST * TILE_B;                          // Smem::x
constexpr uint32_t XCH_B = sizeof(Xch);
constexpr uint32_t XC_OFF = NHQ * 2 * 4 * 16 * 4 * 4;             // Xch::c
constexpr uint32_t XF_OFF = XC_OFF + NHQ * 16 * 4;                // Xch::moved

// d = x * r[place n of the row]  /  d += x * r[place n of the row]: the factor comes out of one
// lane of each row of sixteen (DPP row broadcast inside the multiply), so a row's sixteen factors
// live in one register.  Assembly: the compiler folds a DPP move into a multiply but not into a
// multiply-add.  It does not space an assembly statement from an MFMA whose result the statement
// reads: x must have been written at least eleven instructions earlier (an 8-pass MFMA), which
// the callers arrange by the order of their (volatile) statements.
__device__ __forceinline__ void scaled_by_row_lane(float &d, float r, float x, int nsel, bool first) {
#define CWICK_SBL_CASE(n)                                                                                         \
    case n:                                                                                                       \
        if (first) asm volatile("v_mul_f32_dpp %0, %1, %2 row_newbcast:" #n " row_mask:0xf bank_mask:0xf" : "=v"(d) : "v"(r), "v"(x)); \
        else asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #n " row_mask:0xf bank_mask:0xf" : "+v"(d) : "v"(r), "v"(x));      \
        break;
    switch (nsel) {
        CWICK_SBL_CASE(0) CWICK_SBL_CASE(1) CWICK_SBL_CASE(2) CWICK_SBL_CASE(3) CWICK_SBL_CASE(4) CWICK_SBL_CASE(5)
        CWICK_SBL_CASE(6) CWICK_SBL_CASE(7) CWICK_SBL_CASE(8) CWICK_SBL_CASE(9) CWICK_SBL_CASE(10) CWICK_SBL_CASE(11)
        CWICK_SBL_CASE(12) CWICK_SBL_CASE(13) CWICK_SBL_CASE(14) CWICK_SBL_CASE(15)
        default: break;
    }
#undef CWICK_SBL_CASE
}

__global__ void __launch_bounds__(THREADS) mla_prefill64_kernel(const WideParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    Smem &sm = *reinterpret_cast<Smem *>(smem_raw);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_void *)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool scorer = wave < NHQ;
    const int hq = wave & 3;         // scoring role: heads 16 hq .. 16 hq + 15
    const int cw = wave & 3;         // value role: dims 128 cw .. +127 = scale block cw
    const int n = lane & 15;         // head column / key row of a 16-block / dim row
    const int g = lane >> 4;         // 32-wide contraction block (QK) / 8-wide (PV)

    const int n_hb = (p.nh + HW - 1) / HW;
    const int64_t total = (int64_t)gridDim.x;
    // Workgroups go to the eight XCDs round robin.  The head blocks of a query run on one XCD (they
    // read the same tiles at the same time: one fetch into that L2), and consecutive queries go
    // to consecutive XCDs, so that every XCD gets the same mix of long and short queries (a
    // contiguous eighth of the queries per XCD left the XCD with the longest ones 6 % behind).
    int64_t unit = blockIdx.x;
    if (total % (8 * n_hb) == 0) {
        const int64_t grp = unit / (8 * n_hb), r = unit % (8 * n_hb);
        unit = (8 * grp + r % 8) * n_hb + r / 8;
    }
    const int hb = (int)(unit % n_hb);
    const int y = p.nq - 1 - (int)(unit / n_hb);                      // the queries with the most keys start first

    const uint8_t *rows = p.rows;
    const float *scales = p.scales;
    const int n_keys = (int)(p.pos0 + 1 + y);
    const int n_tiles = (n_keys + TK - 1) / TK;

    uint64_t zrow = (uint64_t)(uintptr_t)g_zero_row64, zsc = (uint64_t)(uintptr_t)g_zero_scales64;
    asm volatile("" : "+s"(zrow), "+s"(zsc));

    // ---- tile copies.  lane = key of the tile; the 36 sixteen-byte columns and 5 scale blocks are
    // dealt round robin: wave w copies columns w, w + 8, w + 16, w + 24, and w + 32 when w < 4;
    // waves 4..7 scale block w - 4, wave 0 scale block 4.  M0 is written by the statement that
    // needs it (the compiler has no other use of M0 in this file; tests check the compiled code).
    auto dma16 = [&](uint64_t gp, uint32_t lds_off) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gp), "s"(lds_off) : "memory");
    };
    auto dma4 = [&](uint64_t gp, uint32_t lds_off) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gp), "s"(lds_off) : "memory");
    };
    auto share = [&](int t, uint32_t tile_off) {
        const int r = t * TK + lane;
        const bool live = r < n_keys;
        const uint64_t rp = live ? (uint64_t)(uintptr_t)rows + (uint64_t)(uint32_t)r * KDIM : zrow;
        const uint64_t sp = live ? (uint64_t)(uintptr_t)scales + (uint64_t)(uint32_t)r * (NBLK * 4) : zsc;
        const uint32_t col_off = tile_off + (uint32_t)wave * (TK * 16);
        const uint64_t col_src = rp + 16 * wave;
        dma16(col_src, col_off);
        dma16(col_src + 128, col_off + 8 * (TK * 16));
        dma16(col_src + 256, col_off + 16 * (TK * 16));
        dma16(col_src + 384, col_off + 24 * (TK * 16));
        if (wave < 4) dma16(col_src + 512, col_off + 32 * (TK * 16));
        else dma4(sp + 4 * (wave - 4), tile_off + SC_OFF + (uint32_t)(wave - 4) * (TK * 4));
        if (wave == 0) dma4(sp + 16, tile_off + SC_OFF + 4u * (TK * 4));
    };
    // a tile by the four value waves alone (the loop: the scoring waves are the longer pole of a
    // step and a wave stalls while the memory pipeline takes its copies): wave cw copies columns
    // cw, cw + 4, .. cw + 32, scale block cw, and wave 4 also scale block 4
    auto share_v = [&](int t, uint32_t tile_off) {
        const int r = t * TK + lane;
        const bool live = r < n_keys;
        const uint64_t rp = live ? (uint64_t)(uintptr_t)rows + (uint64_t)(uint32_t)r * KDIM : zrow;
        const uint64_t sp = live ? (uint64_t)(uintptr_t)scales + (uint64_t)(uint32_t)r * (NBLK * 4) : zsc;
        const uint32_t col_off = tile_off + (uint32_t)cw * (TK * 16);
        const uint64_t col_src = rp + 16 * cw;
        // the 64 k bytes to the lane's source are the instruction's immediate offset, which the
        // hardware also adds to the LDS address: M0 is set that much below the column
#define CWICK_P64_COL(k)                                                                                  \
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:" #k "*64"          \
                 ::"v"(col_src), "s"(col_off + (uint32_t)(4 * k) * (TK * 16) - 64u * k) : "memory")
        CWICK_P64_COL(0); CWICK_P64_COL(1); CWICK_P64_COL(2); CWICK_P64_COL(3); CWICK_P64_COL(4);
        CWICK_P64_COL(5); CWICK_P64_COL(6); CWICK_P64_COL(7); CWICK_P64_COL(8);
#undef CWICK_P64_COL
        dma4(sp + 4 * cw, tile_off + SC_OFF + (uint32_t)cw * (TK * 4));
        if (cw == 0) dma4(sp + 16, tile_off + SC_OFF + 4u * (TK * 4));
    };
    if (n_tiles > 0) share(0, lds0);                  // stage 0 is not part of the Q park area

    // ---- Q for 4 x 16 heads as two E4M3 terms per 32-dim block with one E8M0 scale per head and
    // 128-dim block: unit u = 5 hq + b is prepared by wave u % 8 and parked in the last two tile
    // stages and the exchange area (none in use yet).  lane (n, g) holds head n of the block, dims
    // 128 b + 32 g + [0, 32); the rope block is one register set: lanes g < 2 hold the hi term of
    // dims 512 + 32 g.., lanes g >= 2 the lo term of dims 512 + 32 (g - 2)...
    QPark *park = reinterpret_cast<QPark *>(&sm.tile[1]);
    for (int u = wave; u < 5 * NHQ; u += NWAVES) {
        const int hqu = u / 5, b = u % 5;
        int head = hb * HW + 16 * hqu + n;
        if (head >= p.nh) head = p.nh - 1;
        const uint16_t *qrow = p.q + ((size_t)y * p.nh + head) * KDIM;
        const uint16_t *src = qrow + (b < 4 ? 128 * b + 32 * g : 512 + 32 * (g & 1));
        float qv[32];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const u32x4 w = *(const u32x4 *)(src + 8 * c);
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
    }
    __syncthreads();

    i32x8 qhi[4], qlo[4], qrope;
    int qsc0 = 0, qsc1 = 0;                           // scale bytes of blocks 0..3 / of the rope block
    if (scorer) {
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const QPark *qp = park + 5 * hq + b;
#pragma unroll
            for (int d = 0; d < 8; d++) {
                qhi[b][d] = qp->hi[d][lane];
                qlo[b][d] = qp->lo[d][lane];
            }
            qsc0 |= qp->sc[lane] << (8 * b);
        }
        const QPark *qp = park + 5 * hq + 4;
#pragma unroll
        for (int d = 0; d < 8; d++) qrope[d] = qp->hi[d][lane];
        qsc1 = qp->sc[lane];
    }
    __syncthreads();                                  // the park area becomes tiles and exchange again
    // Nothing the compiler has in flight may cross into the loops: its waits would also wait for
    // the copies.
    if (scorer)
        asm volatile("" : "+v"(qhi[0]), "+v"(qhi[1]), "+v"(qhi[2]), "+v"(qhi[3]), "+v"(qlo[0]), "+v"(qlo[1]), "+v"(qlo[2]), "+v"(qlo[3]), "+v"(qrope), "+v"(qsc0), "+v"(qsc1));

    if (n_tiles > 1) share(1, lds0 + TILE_B);         // tiles 0 and 1 are whole when the loops start
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    LDS_BARRIER();

    const float c0 = p.scale * 1.44269504088896340736f;   // scores in log2 units
    // The stages rotate in scalar registers: st_val holds tile t, st_sc tile t+1, st_cp is where
    // tile t+2 goes (t % 3 as an induction variable made the compiler keep a dozen per-lane
    // addresses alive).
    uint32_t st_val = lds0 + 2 * TILE_B, st_sc = lds0, st_cp = lds0 + TILE_B;    // at t = -1
    auto rotate = [&]() {
        const uint32_t v = st_val;
        st_val = st_sc;
        st_sc = st_cp;
        st_cp = v;
        st_val = (uint32_t)__builtin_amdgcn_readfirstlane((int)st_val);
        st_sc = (uint32_t)__builtin_amdgcn_readfirstlane((int)st_sc);
        st_cp = (uint32_t)__builtin_amdgcn_readfirstlane((int)st_cp);
    };

    if (scorer) {
        float l_priv = 0.0f;                              // sum over this lane's keys of head 16 hq + n, relative to mr
        float mr = -INFINITY;                             // the reference of head 16 hq + n (the four lanes of a head agree)
        // per-lane LDS offsets inside a tile: K fragment of key block 0 (key n, columns 8 b + 2 g and
        // the next), the rope block's (columns 32 + 2 (g & 1)), this lane's four keys' scales
        const uint32_t k_off = (uint32_t)((2 * g) * (TK * 16) + n * 16);
        const uint32_t kr_off = (uint32_t)((32 + 2 * (g & 1)) * (TK * 16) + n * 16);
        // the scales of the tile's keys: lane (row g, place j) holds the scale of key
        // 16 (j / 4) + 4 g + j % 4, the key that accumulator register j % 4 of key block j / 4 holds in
        // this row: one register per dim block covers the tile (five 4-byte reads instead of twenty
        // 16-byte ones, a quarter of what the four scoring waves read from LDS per tile), and the
        // combination of the block products takes its factor from place 4 kb + i of the row
        const uint32_t sr_off = SC_OFF + (uint32_t)((16 * (n >> 2) + 4 * g + (n & 3)) * 4);
        // where this lane's four probabilities of key block kb go: keys 16 (kb & 1) + 4 g + i of half kb >> 1
        const uint32_t xp_off = (uint32_t)(((hq * 2 * 4 + (g >> 1)) * 16 + n) * 16 + 2 * (g & 1) * 4);
        const uint32_t xc_off = XC_OFF + (uint32_t)((hq * 16 + n) * 4);
        const uint32_t xf_off = XF_OFF + (uint32_t)(hq * 4);
        const int tail_tile = n_tiles - 1;
        const int tail_keys = n_keys - tail_tile * TK;    // 1..64

#pragma clang loop unroll(disable)
        for (int t = -1; t < n_tiles; t++) {
            if (t + 1 < n_tiles) {
                // ---- scores S^T[key][head] for all 64 keys, heads 16 hq.. of tile t+1 ----
                const uint32_t tb = st_sc;
                const uint32_t xn = lds0 + X_OFF + (uint32_t)((t + 1) & 1) * XCH_B;
                f32x4 S[4];
                float rsc[NBLK];
#pragma unroll
                for (int b = 0; b < NBLK; b++) rsc[b] = LDS_AT(lds_f32, tb + sr_off + (uint32_t)b * (TK * 4));
                // Fragment j = 5 kb + b (b = 4: the rope block).  Its MFMAs (hi and lo term, or the one
                // rope instruction) are issued from assembly in a fixed order, its block product is
                // folded into S three fragments later: between an MFMA and the statement that reads its
                // result lie the MFMAs and folds of three other fragments (fifteen instructions or
                // more, where an 8-pass MFMA asks for eleven), and a lo term accumulates into the
                // registers its hi term wrote.
                const uint32_t kbase = tb + k_off, krbase = tb + kr_off;
                auto kfrag = [&](int j) -> i32x8 {
                    const int kb = j / 5, b = j % 5;
                    const uint32_t a = (b < 4 ? kbase + (uint32_t)(8 * b) * (TK * 16) : krbase) + (uint32_t)kb * 256u;
                    const u32x4 k0 = LDS_AT(lds_u32x4, a);
                    const u32x4 k1 = LDS_AT(lds_u32x4, a + TK * 16);
                    return (i32x8){(int)k0[0], (int)k0[1], (int)k0[2], (int)k0[3], (int)k1[0], (int)k1[1], (int)k1[2], (int)k1[3]};
                };
                const int one_scales = 0x7F7F7F7F;
#define CWICK_P64_PAIR(A, K, QH, QL, SEL)                                                                         \
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %4, %5 " SEL "\n\t"                             \
                 "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %3, %0, %4, %5 " SEL                                    \
                 : "=&v"(A) : "v"(K), "v"(QH), "v"(QL), "v"(one_scales), "v"(qsc0))
                f32x4 acc[4];
                i32x8 kfr[3];
                kfr[0] = kfrag(0);
                kfr[1] = kfrag(1);
#pragma unroll
                for (int j = 0; j < 23; j++) {
                    if (j < 20) {
                        const int b = j % 5;
                        if (j + 2 < 20) kfr[(j + 2) % 3] = kfrag(j + 2);
                        switch (b) {
                            case 0: CWICK_P64_PAIR(acc[j % 4], kfr[j % 3], qhi[0], qlo[0], "op_sel:[0,0,0] op_sel_hi:[0,0,0]"); break;
                            case 1: CWICK_P64_PAIR(acc[j % 4], kfr[j % 3], qhi[1], qlo[1], "op_sel:[0,1,0] op_sel_hi:[0,0,0]"); break;
                            case 2: CWICK_P64_PAIR(acc[j % 4], kfr[j % 3], qhi[2], qlo[2], "op_sel:[0,0,0] op_sel_hi:[0,1,0]"); break;
                            case 3: CWICK_P64_PAIR(acc[j % 4], kfr[j % 3], qhi[3], qlo[3], "op_sel:[0,1,0] op_sel_hi:[0,1,0]"); break;
                            default:
                                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[0,0,0] op_sel_hi:[0,0,0]"
                                             : "=&v"(acc[j % 4]) : "v"(kfr[j % 3]), "v"(qrope), "v"(one_scales), "v"(qsc1));
                                break;
                        }
                    } else {
                        asm volatile("s_nop 3" ::: "memory");          // the last three folds have no MFMAs behind them
                    }
                    if (j >= 3) {
                        const int f = j - 3, kb = f / 5, b = f % 5;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            float d = S[kb][i];
                            scaled_by_row_lane(d, rsc[b], acc[f % 4][i], 4 * kb + i, b == 0);
                            S[kb][i] = d;
                        }
                    }
                }
#undef CWICK_P64_PAIR
                // positions past the query's last key (only in its last tile; the empty statement keeps
                // this a branch: as sixteen selects it would run in every step)
                if (t + 1 == tail_tile && tail_keys < TK) {
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int kb = 0; kb < 4; kb++)
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            if (16 * kb + 4 * g + i >= tail_keys) S[kb][i] = -INFINITY;
                }
                float lmax = vmax3(S[0][0], S[0][1], vmax(S[0][2], S[0][3]));
#pragma unroll
                for (int kb = 1; kb < 4; kb++) lmax = vmax3(lmax, S[kb][0], vmax3(S[kb][1], S[kb][2], S[kb][3]));
                lmax *= c0;                                   // S stays unscaled: c0 > 0 goes into the exponent's multiply-add
                const bool moves = __any(lmax > mr + LAZY);   // rare after the first tiles: only then the lanes of a head confer
                if (moves) {
                    lmax = xor16_max(lmax);
                    lmax = xor32_max(lmax);
                    const float m_new = lmax > mr + LAZY ? lmax : mr;
                    const float cf = (mr == -INFINITY || m_new == mr) ? 1.0f : __builtin_amdgcn_exp2f(mr - m_new);
                    l_priv *= cf;
                    mr = m_new;
                    LDS_AT(lds_f32, xn + xc_off) = cf;        // the four lanes of a head write the same word
                }
                const float m_use = mr == -INFINITY ? 0.0f : mr;
                float lsum = 0.0f;
#pragma unroll
                for (int kb = 0; kb < 4; kb++) {
                    f32x4 P;
#pragma unroll
                    for (int i = 0; i < 4; i++) P[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[kb][i], c0, -m_use));
                    lsum += (P[0] + P[1]) + (P[2] + P[3]);
                    u32x2 d;
                    d[0] = pack_f16_rne(P[0], P[1]);
                    d[1] = pack_f16_rne(P[2], P[3]);
                    // [hq][kb >> 1][2 (kb & 1) + (g >> 1)][n][2 (g & 1) ..]
                    LDS_AT(lds_u32x2, xn + xp_off + (uint32_t)(((kb >> 1) * 4 + 2 * (kb & 1)) * 256)) = d;
                }
                l_priv += lsum;
                LDS_AT(lds_u32, xn + xf_off) = moves ? 1u : 0u;
            }
            LDS_BARRIER();
            rotate();
        }

        // ---- the sums of the scoring role meet in LDS (the exchange area is free now) ----
        float *lsum = reinterpret_cast<float *>(&sm.x[0]);            // [16-head block][head]
        float ls = xor16_sum(l_priv);
        ls = xor32_sum(ls);
        if (g == 0) lsum[hq * 16 + n] = ls;
        LDS_BARRIER();
    } else {
        f32x4 oacc[NHQ][8];                               // [16-head block][dim block]: dims 128 cw + 16 j + 4 g + i, head n
#pragma unroll
        for (int h = 0; h < NHQ; h++)
#pragma unroll
            for (int j = 0; j < 8; j++) oacc[h][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        int e_run = E_NONE;                               // 2^e_run is above every scale of this wave's block seen so far
        uint32_t thr_bits = 0u;                           // bits of 2^e_run: a scale whose bits reach them does not fit
        float wfac = 0.0f;                                // 2^(WEXP - e_run)
        __builtin_amdgcn_s_setprio(3);
        // transpose-read addressing for V^T: lane i of 16-lane group g supplies key 8 g + (i >> 1),
        // bytes 8 (i & 1) .. +7 of the sixteen-byte column
        const uint32_t tr_off = (uint32_t)((8 * cw) * (TK * 16) + (8 * g + (n >> 1)) * 16 + 8 * (n & 1));
        // the two scales this lane turns into a pair of factors (see the loop)
        const uint32_t sv_off = SC_OFF + (uint32_t)(cw * (TK * 4) + (32 * ((n & 7) >> 2) + 8 * g + 2 * (n & 3)) * 4);
        // the probabilities of this lane's slots: [16-head block][key half][g][n][4 dwords]
        const uint32_t pw_off = (uint32_t)((g * 16 + n) * 16);
        const uint32_t xcl_off = XC_OFF + (uint32_t)(n * 4);
        asm volatile("" ::: "memory");
#pragma clang loop unroll(disable)
        for (int t = -1; t < n_tiles; t++) {
            if (t >= 0 && t + 2 < n_tiles) share_v(t + 2, st_cp);     // the stage tile t-1 left at the last barrier
            if (t >= 0) {
                // ---- values O^T[dim][head] += V^T W^T for dims 128 cw.., all 64 heads, tile t ----
                const uint32_t tb = st_val;
                const uint32_t xb = lds0 + X_OFF + (uint32_t)(t & 1) * XCH_B;
                // The sixteen lanes of a row share their contraction slots (keys 8 g .. 8 g + 7 of each
                // half), so a row needs eight fp16 pairs of scale factors per tile: lane (g, n) reads
                // the two scales of pair n & 7 (half (n & 7) >> 2, keys 8 g + 2 (n & 3) and the next),
                // forms that one pair, and every lane takes the eight pairs out of the row by DPP.
                const f32x2 sv = LDS_AT(lds_f32x2, tb + sv_off);
                const u32x4 fl = LDS_AT(lds_u32x4, xb + XF_OFF);
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
                const uint32_t any_moved = fl[0] | fl[1] | fl[2] | fl[3];
                if (__builtin_amdgcn_readfirstlane(any_moved) != 0u || ecorr != 1.0f) {
                    // a scoring wave moved a reference in this tile (or the weights' normaliser
                    // grew): the accumulators so far shrink to the new units
#pragma unroll
                    for (int h = 0; h < NHQ; h++) {
                        float c = ecorr;
                        if (__builtin_amdgcn_readfirstlane(fl[h]) != 0u) c *= LDS_AT(lds_f32, xb + xcl_off + (uint32_t)(h * 64));
#pragma unroll
                        for (int j = 0; j < 8; j++) oacc[h][j] *= c;
                    }
                }
                const uint32_t va0 = tb + tr_off;
#pragma unroll
                for (int kh = 0; kh < 2; kh++) {
                    u32x4 pw[NHQ];                        // the tile's weights of this key half, per 16-head block
#pragma unroll
                    for (int h = 0; h < NHQ; h++) {
                        pw[h] = LDS_AT(lds_u32x4, xb + pw_off + (uint32_t)((h * 2 + kh) * 1024));
#pragma unroll
                        for (int d = 0; d < 4; d++) pw[h][d] = mul_f16x2(pw[h][d], sw[kh][d]);
                    }
#pragma unroll
                    for (int j0 = 0; j0 < 8; j0 += 4) {
                        i32x2 vt[4];
#pragma unroll
                        for (int j = 0; j < 4; j++)
                            vt[j] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2 *)(size_t)(va0 + (uint32_t)((j0 + j) * (TK * 16) + kh * (32 * 16))));
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            u32x4 vh;
                            vh[0] = e4m3x2_to_f16x2<false>((uint32_t)vt[j][0]);
                            vh[1] = e4m3x2_to_f16x2<true>((uint32_t)vt[j][0]);
                            vh[2] = e4m3x2_to_f16x2<false>((uint32_t)vt[j][1]);
                            vh[3] = e4m3x2_to_f16x2<true>((uint32_t)vt[j][1]);
                            const f16x8 va = __builtin_bit_cast(f16x8, vh);
#pragma unroll
                            for (int h = 0; h < NHQ; h++)
                                oacc[h][j0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(f16x8, pw[h]), oacc[h][j0 + j], 0, 0, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);   // the next block's fragments are not fetched across this point (registers)
                    }
                }
            }
            // tile t+2, copied by the value waves during this step, is scored in the next one
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            LDS_BARRIER();
            rotate();
        }

        const float *lsum = reinterpret_cast<const float *>(&sm.x[0]);
        LDS_BARRIER();
        // ---- every value wave owns its dims: write the result directly ----
        const float unit_f = e_run == E_NONE ? 0.0f : pow2i(e_run - WEXP);   // the accumulators are in units of 2^(e_run - WEXP)
#pragma unroll
        for (int h = 0; h < NHQ; h++) {
            const float L = lsum[h * 16 + n];
            const int head = hb * HW + 16 * h + n;
            if (head >= p.nh) continue;
            const float fin = L > 0.0f ? unit_f / L : 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                // accumulator register i <-> dim 16 db + 4 g + i
                const f32x4 v = oacc[h][j] * fin;
                *(f32x4 *)(p.out + ((size_t)y * p.nh + head) * VDIM + 16 * (8 * cw + j) + 4 * g) = v;
            }
        }
    }
}

}  // namespace

// chunked prefill with 64 heads per workgroup; the caller has checked the operands
int launch_mla_prefill_wide(const uint8_t *rows, const float *scales, int64_t pos0, int64_t n, const uint16_t *q,
                            int n_heads, float scale, float *out, hipStream_t s) {
    static std::once_flag attr_once;
    static hipError_t attr_err = hipSuccess;
    const size_t smem = sizeof(Smem);
    std::call_once(attr_once, [&] {
        attr_err = hipFuncSetAttribute((const void *)mla_prefill64_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    });
    CWICK_HIP_CALL(attr_err);
    WideParams p{};
    p.rows = rows; p.scales = scales; p.pos0 = pos0; p.q = q; p.nh = n_heads; p.nq = (int)n; p.scale = scale; p.out = out;
    const int n_hb = (n_heads + HW - 1) / HW;
    const int64_t total = (int64_t)n_hb * n;
    CWICK_REQUIRE(total <= 0x7FFFFFFF, "mla_prefill: grid of %lld workgroups is too large", (long long)total);
    {
        ProfKernel pk(CWICK_HIP_PROF_MLA_PREFILL, s);
        pk.launch(mla_prefill64_kernel, dim3((unsigned)total), dim3(THREADS), smem, p);
    }
    CWICK_HIP_CALL(hipGetLastError());
    return 1;
}

}  // namespace cwick
