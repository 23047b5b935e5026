/* cwick_hip.h -- C ABI of libcwick_hip.so, the MI355X (gfx950) attention backend.
 *
 * The engine keeps its attention entry points (src/attention.c, src/ds_ops.c,
 * src/q35_model.c, src/ds_model.c) and guards each hot loop with one of the
 * calls below, the way src/h3.c:562-564 guards its CPU loop with
 * h3_gpu_attention().  Conventions are the reference's own GPU-hook
 * conventions (src/h3_gpu.h:19-27, src/cwick.h:480-529):
 *
 *   - every compute call returns 1 when the GPU produced the result and 0 when
 *     it declined; on 0 the outputs are untouched and the caller runs its CPU
 *     path.  A call declines on an unsupported shape, a bad argument, a
 *     missing device or a HIP error; it never aborts and never approximates.
 *   - cwick_hip_last_error() says why the last call on this thread declined.
 *   - called from the request thread, one generation at a time
 *     (src/attention.c:353-354); calls on one handle must not overlap.  Every
 *     cache handle owns a HIP stream and a staging buffer for the operands of
 *     its host-pointer calls, so calls on different handles may run on different
 *     threads (the per-slot model of src/metal.c:306-319).  The two host-pointer
 *     calls that take no handle (cwick_hip_topk, cwick_hip_e4m3_table) take
 *     turns under a lock.  The *_dev calls use the caller's stream and a
 *     split-K workspace per stream: one thread per stream.
 *
 * MI355X has its own memory, so caches live in device memory behind opaque
 * handles that the engine fills at the sites where it writes its host caches
 * (src/attention.c:699-709, src/q35_model.c:1649-1651, src/ds_model.c:1061-1070).
 * Queries, index lists and outputs are host pointers, copied per call.
 *
 * The *_dev entry points are the same operations on memory that is already in
 * HBM (device pointers, caller's HIP stream, no copies, no synchronisation);
 * the host-pointer calls are thin wrappers over them.
 *
 * Data formats
 *   bf16           uint16_t, the top half of an fp32 (src/util.h:55-60)
 *   FP8            E4M3fn bytes, bias 7, no inf, 0x7F/0xFF NaN (src/tensor.c:344-368)
 *   latent row     576 FP8 bytes = 512 "nope" dims followed by 64 rope dims;
 *                  5 fp32 scales per row, one per 128-element block (the last
 *                  block is the 64 rope dims); value = e4m3(byte) * scale[d/128]
 *   indexer key    128 FP8 bytes + one fp32 scale per token
 */
#ifndef CWICK_HIP_H
#define CWICK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CWICK_HIP_LATENT_KDIM 576   /* score width: nope + rope */
#define CWICK_HIP_LATENT_VDIM 512   /* value width: nope only */
#define CWICK_HIP_LATENT_BLOCK 128  /* elements per fp32 scale */
#define CWICK_HIP_LATENT_NBLK 5
#define CWICK_HIP_INDEX_DIM 128

/* ---- lifecycle ------------------------------------------------------- */

/* Replaces h3_gpu_ready (src/h3_gpu.h:9) / cwick_metal_backend_active
 * (src/metal.c:120-123).  Brings device 0 up on first use.  State machine of
 * src/h3_gpu.c:35-40: untried -> ready | unavailable (permanent).  Honours
 * cwick_hip_force() first, then the CWICK_HIP environment variable
 * (src/metal.c:98-105 pattern; default: on when a gfx950 device exists). */
int cwick_hip_ready(void);

/* Replaces cwick_metal_force (src/metal.c:60-79): 1 = select this backend
 * (returns 0 on success, -1 if the device cannot be brought up), 0 = explicit
 * CPU, every compute call declines from then on. */
int cwick_hip_force(int on);

/* Replaces h3_gpu_shutdown (src/h3_gpu.h:10): frees internal workspaces. */
void cwick_hip_shutdown(void);

/* Why the last call on this thread returned 0 / NULL ("" if it did not).
 * Plays the part of cwick_error.message (src/cwick.h:39-59). */
const char *cwick_hip_last_error(void);

/* "gfx950 ... CUs ... GiB" into buf; returns 1, or 0 when no device is up. */
int cwick_hip_device_info(char *buf, size_t cap);

/* ---- GQA K/V cache: bf16 rows [capacity][n_kv_heads*head_dim] --------- */
/* Device mirror of q35_model.kcache/vcache (src/q35.h:257-261), kept in the
 * bf16 form the reference snapshots them in (src/q35_model.c:1558-1575). */
typedef struct cwick_hip_kv cwick_hip_kv;
cwick_hip_kv *cwick_hip_kv_create(int64_t capacity, int n_kv_heads, int head_dim);
void cwick_hip_kv_free(cwick_hip_kv *c);
/* Store rows pos0..pos0+n-1 (the memcpy pair of src/q35_model.c:1649-1651). */
int cwick_hip_kv_write(cwick_hip_kv *c, int64_t pos0, int64_t n,
                       const uint16_t *k_rows, const uint16_t *v_rows);
/* Same from fp32 rows, narrowed on the device with round-to-nearest-even
 * (q35_narrow_rows, src/q35_model.c:1558-1575). */
int cwick_hip_kv_write_f32(cwick_hip_kv *c, int64_t pos0, int64_t n,
                           const float *k_rows, const float *v_rows);
/* Read rows back as stored (bf16), or widened to fp32 on the device
 * (q35_widen_rows, src/q35_model.c:1543-1556): what a prefix snapshot of the
 * caches takes (src/pfx.h:42-73, src/engine.c:3630-3660). */
int cwick_hip_kv_read(cwick_hip_kv *c, int64_t pos0, int64_t n, uint16_t *k_rows, uint16_t *v_rows);
int cwick_hip_kv_read_f32(cwick_hip_kv *c, int64_t pos0, int64_t n, float *k_rows, float *v_rows);
uint16_t *cwick_hip_kv_k_dev(cwick_hip_kv *c);   /* device addresses, for */
uint16_t *cwick_hip_kv_v_dev(cwick_hip_kv *c);   /* callers that fill in HBM */

/* ---- MLA latent cache: FP8 rows + block scales ------------------------ */
/* Device mirror of the latent cache `keys[layer][capacity][kv_lora]`
 * (src/attention.c:78-92, src/engine.c:2894-2900) in BASELINE's FP8 format.
 * `slots` independent sequences of `capacity` rows each (the reference's
 * [slots][capacity][kv_lora] layout). */
typedef struct cwick_hip_latent cwick_hip_latent;
cwick_hip_latent *cwick_hip_latent_create(int slots, int64_t capacity);
void cwick_hip_latent_free(cwick_hip_latent *c);
/* Store already-quantised rows: rows [n][576] bytes, scales [n][5] fp32. */
int cwick_hip_latent_write(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                           const uint8_t *rows, const float *scales);
/* Store fp32 latent rows [n][576] (what src/attention.c:699-709 writes),
 * quantised on the device: scale = amax(block)/448 (1 when the block is all
 * zero), byte = RNE e4m3 of value/scale (src/ds_quant.c:102-128). */
int cwick_hip_latent_write_f32(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                               const float *rows);
/* Read rows back (for prefix snapshots, src/pfx.h:42-73). */
int cwick_hip_latent_read(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                          uint8_t *rows, float *scales);
uint8_t *cwick_hip_latent_rows_dev(cwick_hip_latent *c, int slot);
float *cwick_hip_latent_scales_dev(cwick_hip_latent *c, int slot);

/* ---- indexer key cache: FP8 rows [capacity][128] + scale per token ---- */
/* Device mirror of the indexer key store (src/ds_model.c:1054-1063 idx_k,
 * src/cwick.h:832-856 pool) in BASELINE's FP8 format. */
typedef struct cwick_hip_ikeys cwick_hip_ikeys;
cwick_hip_ikeys *cwick_hip_ikeys_create(int slots, int64_t capacity);
void cwick_hip_ikeys_free(cwick_hip_ikeys *c);
int cwick_hip_ikeys_write(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n,
                          const uint8_t *rows, const float *scales);
int cwick_hip_ikeys_write_f32(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n,
                              const float *rows);
/* Read rows back (the indexer pools of a prefix snapshot, src/pfx.h:42-73). */
int cwick_hip_ikeys_read(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n, uint8_t *rows,
                         float *scales);
uint8_t *cwick_hip_ikeys_rows_dev(cwick_hip_ikeys *c, int slot);
float *cwick_hip_ikeys_scales_dev(cwick_hip_ikeys *c, int slot);

/* ---- GQA attention ---------------------------------------------------- */

/* Replaces the decode branch of mixer_attn: dec_scores / dec_softmax /
 * dec_out_slices (src/q35_model.c:1656-1701).  One query position, every
 * head: out[h] = softmax_t(scale * q[h].K[t][h/group]) . V[.][h/group] over
 * t in [0, n_keys).  q [n_heads][head_dim] bf16, out [n_heads][head_dim] fp32.
 * Supported: head_dim 256 or 128, group = n_heads/n_kv_heads in {1,2,4,8,16},
 * 1 <= n_keys <= capacity. */
int cwick_hip_gqa_decode(cwick_hip_kv *c, int64_t n_keys, const uint16_t *q,
                         int n_heads, float scale, float *out);

/* Replaces the prefill branch of mixer_attn (src/q35_model.c:1713-1746):
 * causal attention of n new queries at positions pos0..pos0+n-1 over cache
 * rows 0..pos0+n-1 (which the caller has already written); query i sees keys
 * 0..pos0+i.  q [n][n_heads][head_dim] bf16, out [n][n_heads][head_dim] fp32.
 * Supported: head_dim 256, group = n_heads/n_kv_heads in {1,2,4,8}. */
int cwick_hip_gqa_prefill(cwick_hip_kv *c, int64_t pos0, int64_t n, const uint16_t *q,
                          int n_heads, float scale, float *out);

/* ---- absorbed-latent MLA ---------------------------------------------- */

/* Replaces the two reductions of mla_latent_decode (src/attention.c:749-811):
 * scores over the latent, cwick_softmax per head, c_acc accumulation.  q is
 * the absorbed query q_abs (after src/attention.c:741-744) as bf16
 * [n_heads][576]; out is c_acc [n_heads][512] fp32 (before :812-815).
 * sel == NULL: every position 0..n_list-1 (:759).  sel != NULL: n_list
 * entries, each a row of the slot (any order, as indexer_select emits them);
 * entries < 0 are skipped (the -1 padding of src/ds_model.c:929).
 * Supported: 1 <= n_heads <= 128, 1 <= n_list, rows < capacity. */
int cwick_hip_mla_decode(cwick_hip_latent *c, int slot, const int32_t *sel, int64_t n_list,
                         const uint16_t *q, int n_heads, float scale, float *out);

/* The same with the attention sink of ds_sparse_attn_heads (src/ds_model.c:917-966,
 * the sink term at :946): sink [n_heads] fp32, in the units of the scaled scores;
 * exp(sink[h] - max) joins the softmax denominator of head h and carries no
 * value.  sink == NULL is cwick_hip_mla_decode.  The reference's index list
 * addresses two stores -- t < W the window ring, else compressed row t - W
 * (:930-931) -- which here is one slot whose first W rows hold the ring. */
int cwick_hip_mla_decode_sink(cwick_hip_latent *c, int slot, const int32_t *sel, int64_t n_list,
                              const uint16_t *q, int n_heads, float scale, const float *sink,
                              float *out);

/* Replaces the per-token loop of cwick_attention_mla_prefill_chunk
 * (src/attention.c:1010-1019): n queries at positions pos0..pos0+n-1, query t
 * attends rows 0..pos0+t of the slot (npos = pos+1, :662), all of which are
 * already written (:988-1007).  q [n][n_heads][576] bf16, out
 * [n][n_heads][512] fp32. */
int cwick_hip_mla_prefill_chunk(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                                const uint16_t *q, int n_heads, float scale, float *out);

/* ---- DSA: lightning indexer, top-k, sparse MLA ------------------------- */

/* Replaces the score loop of indexer_select (src/attention.c:573-582) and of
 * ds_indexer (src/ds_model.c:1108-1121): scores[t] = sum_h relu(q_h.k_t) * w[h]
 * for t in [0, n_keys).  q_idx [n_idx_heads][128] bf16, w [n_idx_heads] fp32
 * (already folded with 1/sqrt(hd*ih), :564-565).  The summation order is
 * fixed and documented beside the kernel, so the result is bit-identical to
 * the CPU oracle that follows the same order.  n_idx_heads <= 64. */
int cwick_hip_indexer_scores(cwick_hip_ikeys *c, int slot, int64_t n_keys,
                             const uint16_t *q_idx, const float *w, int n_idx_heads,
                             float *scores);

/* The two CPU score loops differ in their roundings; `mode` picks whose bits
 * the scores reproduce:
 *   CWICK_HIP_INDEXER_GLM  indexer_select (src/attention.c:573-582): four-lane
 *                          dot_f32 order, ReLU, times w[h]; what
 *                          cwick_hip_indexer_scores computes.
 *   CWICK_HIP_INDEXER_DS   ds_indexer (src/ds_model.c:1099-1121): serial dot over
 *                          the dequantised key, the dot rounded to bf16
 *                          (ds_bf16_round) before the ReLU, w[h] rounded to
 *                          bf16 (the kernel rounds what it is given). */
enum { CWICK_HIP_INDEXER_GLM = 0, CWICK_HIP_INDEXER_DS = 1 };
int cwick_hip_indexer_scores_mode(cwick_hip_ikeys *c, int slot, int64_t n_keys,
                                  const uint16_t *q_idx, const float *w, int n_idx_heads,
                                  int mode, float *scores);

/* No counterpart in the reference: the first stage of the fused select
 * (cwick_hip_dsa_decode), on its own, for checking it.  scores[t] approximates
 * the score above on the matrix cores; *bound is one number for the row with
 * |scores[t] - exact score[t]| <= *bound for every t (see indexer_band.hip for
 * the derivation).  The fused call scores exactly only the keys whose
 * approximate score lies within 2 * bound of the selection threshold. */
int cwick_hip_indexer_scores_approx(cwick_hip_ikeys *c, int slot, int64_t n_keys,
                                    const uint16_t *q_idx, const float *w, int n_idx_heads,
                                    float *scores, float *bound);

/* Replaces ds_topk_scores (src/ds_ops.c:310-338, contract src/ds_ops.h:110-112)
 * and the threshold selector of src/attention.c:585-598: the k best of n
 * scores by (score descending, index ascending), written in ascending index
 * order.  -0.0 == +0.0; NaN ranks below -inf.  *n_out = min(k, n).
 * n <= 2^24, k <= 65536. */
int cwick_hip_topk(const float *scores, int64_t n, int64_t k, int32_t *out_idx,
                   int64_t *n_out);

/* Replaces the indexer -> top-k -> sparse attention chain of a DSA decode
 * step (src/ds_model.c:1081-1164 + :968-995; src/attention.c:716-811) for a
 * batch of independent queries: query b reads slot slot0 + b*slot_step of
 * both caches (slot_step 0 = one shared context).
 * q_idx [batch][n_idx_heads][128] bf16, w [batch][n_idx_heads], q
 * [batch][n_heads][576] bf16, out [batch][n_heads][512] fp32; sel_out, when
 * not NULL, receives the selected rows [batch][topk] (ascending, -1 padded
 * when n_keys < topk). */
int cwick_hip_dsa_decode(cwick_hip_ikeys *ik, cwick_hip_latent *lat, int slot0, int slot_step,
                         int batch, int64_t n_keys, const uint16_t *q_idx, const float *w,
                         int n_idx_heads, int64_t topk, const uint16_t *q, int n_heads,
                         float scale, float *out, int32_t *sel_out);

/* ---- the same operations on HBM-resident operands ---------------------- */
/* All pointers are device pointers; `stream` is a hipStream_t (NULL = the
 * null stream).  Kernels are enqueued, nothing is copied or waited for.
 * Scratch (split-K partials, select state) comes from a grow-only workspace
 * that the library keeps per stream.  A call whose shape needs more than the
 * stream's workspace holds allocates a larger buffer (hipMalloc) and keeps the
 * old one until cwick_hip_stream_release() or cwick_hip_shutdown(): kernels
 * already enqueued and HIP graphs captured earlier stay valid, and no *_dev
 * call ever waits for the stream or frees memory.  While the stream is being
 * captured into a graph a call that would have to allocate declines instead
 * (the capture stays intact): run each shape once before capturing, or size
 * the workspace up front with cwick_hip_reserve_dev().  The split-K partials and the
 * ticket counters of cwick_hip_gqa_prefill_dev belong to the stream: two calls
 * that use one stream's workspace at the same time (a graph replayed on another stream
 * while eager calls run on the capture stream) race. */

/* No counterpart in the reference (its GPU hooks allocate on demand,
 * src/metal.c:306-319): sizes the workspace of `stream` to at least `bytes`,
 * together with the small fixed-size state the select and prefill kernels keep
 * per stream, so that later *_dev calls whose scratch fits allocate nothing.
 * cwick_hip_workspace_bytes_dev() reports what the stream holds now: run the
 * largest shapes once and reserve that figure in the next process. */
int cwick_hip_reserve_dev(void *stream, int64_t bytes);
int64_t cwick_hip_workspace_bytes_dev(void *stream);
/* Waits for `stream`, then frees everything the library keeps for it
 * (workspace, retired buffers, ticket counters).  For callers about to destroy
 * a stream they passed to *_dev calls: a later stream may reuse the handle
 * value.  Graphs captured from this stream's calls must not be replayed
 * afterwards. */
int cwick_hip_stream_release(void *stream);

int cwick_hip_gqa_decode_dev(const uint16_t *k, const uint16_t *v, int64_t n_keys,
                             int n_kv_heads, int head_dim, const uint16_t *q, int n_heads,
                             float scale, float *out, void *stream);

int cwick_hip_gqa_prefill_dev(const uint16_t *k, const uint16_t *v, int64_t pos0, int64_t n,
                              int n_kv_heads, int head_dim, const uint16_t *q, int n_heads,
                              float scale, float *out, void *stream);

/* batch queries; query b uses rows + b*row_batch_stride (bytes) and
 * scales + b*scale_batch_stride (floats), each holding n_rows valid rows;
 * sel [batch][n_list] or NULL.  sel entries outside [0, n_rows) are skipped. */
int cwick_hip_mla_decode_dev(const uint8_t *rows, const float *scales,
                             int64_t row_batch_stride, int64_t scale_batch_stride,
                             int64_t n_rows, int batch, const int32_t *sel, int64_t n_list,
                             const uint16_t *q, int n_heads, float scale, float *out,
                             void *stream);

/* No counterpart in the reference: cwick_hip_mla_decode_dev for callers that
 * cannot allocate device memory (code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc).  Same operands, same kernels, same
 * result; the split-K partials go to a fixed 16 MiB area inside the library's
 * device image instead of the grow-only workspace, and no call of this entry
 * point allocates or frees anything (no phase-timer events either: launches
 * made here are not timed).  It declines when the partials of the call would
 * not fit (they take about 34 KB per workgroup: every shape whose one round
 * of workgroups -- at most one per compute unit -- is 256 or fewer fits, the
 * five benchmark configurations included).  All calls of this entry point on
 * a GPU share that area: calls that overlap in time on one GPU, on whatever
 * streams, race. */
int cwick_hip_mla_decode_static_dev(const uint8_t *rows, const float *scales,
                                    int64_t row_batch_stride, int64_t scale_batch_stride,
                                    int64_t n_rows, int batch, const int32_t *sel, int64_t n_list,
                                    const uint16_t *q, int n_heads, float scale, float *out,
                                    void *stream);

int cwick_hip_mla_decode_sink_dev(const uint8_t *rows, const float *scales,
                                  int64_t row_batch_stride, int64_t scale_batch_stride,
                                  int64_t n_rows, int batch, const int32_t *sel, int64_t n_list,
                                  const uint16_t *q, int n_heads, float scale, const float *sink,
                                  float *out, void *stream);

int cwick_hip_mla_prefill_chunk_dev(const uint8_t *rows, const float *scales, int64_t pos0,
                                    int64_t n, const uint16_t *q, int n_heads, float scale,
                                    float *out, void *stream);

int cwick_hip_indexer_scores_dev(const uint8_t *keys, const float *kscale,
                                 int64_t key_batch_stride, int64_t kscale_batch_stride,
                                 int batch, int64_t n_keys, const uint16_t *q_idx,
                                 const float *w, int n_idx_heads, float *scores,
                                 void *stream);

int cwick_hip_indexer_scores_mode_dev(const uint8_t *keys, const float *kscale,
                                      int64_t key_batch_stride, int64_t kscale_batch_stride,
                                      int batch, int64_t n_keys, const uint16_t *q_idx,
                                      const float *w, int n_idx_heads, int mode, float *scores,
                                      void *stream);

/* scores [batch][n], out_idx [batch][k] (rows padded with -1 past min(k,n)). */
int cwick_hip_topk_dev(const float *scores, int batch, int64_t n, int64_t k,
                       int32_t *out_idx, void *stream);

/* The fused step of cwick_hip_dsa_decode on device operands.  scores_tmp
 * [batch][n_keys] floats is scratch: what it holds afterwards are not the
 * indexer's scores (the fused select overwrites most of them with +inf / -inf
 * marks); cwick_hip_indexer_scores_dev returns scores.  sel_out [batch][topk]
 * receives the selected rows and is required. */
int cwick_hip_dsa_decode_dev(const uint8_t *ikeys, const float *ikscale,
                             int64_t key_batch_stride, int64_t kscale_batch_stride,
                             const uint8_t *rows, const float *scales,
                             int64_t row_batch_stride, int64_t scale_batch_stride,
                             int batch, int64_t n_keys, const uint16_t *q_idx, const float *w,
                             int n_idx_heads, int64_t topk, const uint16_t *q, int n_heads,
                             float scale, float *scores_tmp, int32_t *sel_out, float *out,
                             void *stream);

/* ---- the steps around the attention kernels, on HBM-resident operands ---- */
/* With these the queries and the attention outputs never cross the host link:
 * the projections' outputs go in, what the attention kernels take comes out. */

/* Replaces the absorb loop of mla_latent_decode (src/attention.c:741-744,
 * gemv_bf16_t :145-177): q_abs[h][c] = sum_i q[h][i] * W_k[h][i][c] for the
 * `nope` leading dims of every head's query, W_k[h] = rows h*kv_dim ..
 * h*kv_dim+nope of kv_b_proj (bf16, row-major [n_heads*kv_dim][kv_lora]);
 * the `rope` dims that follow in q pass through to q_abs[h][512 .. 512+rope)
 * (zero-filled to 576).  q fp32 [batch][n_heads][q_dim] (batch stride in
 * floats), q_abs bf16 [batch][n_heads][576], rounded to nearest even: the
 * query operand of cwick_hip_mla_decode_dev.  kv_lora must be 512. */
int cwick_hip_mla_absorb_dev(const uint16_t *kv_b_proj, const float *q, int64_t q_batch_stride,
                             int batch, int n_heads, int q_dim, int nope, int rope, int kv_dim,
                             int kv_lora, uint16_t *q_abs, void *stream);

/* Replaces the expansion after the accumulation (src/attention.c:812-815,
 * gemv_bf16_n :184-224): attn_out[h][r] = W_v[h][r] . c_acc[h], W_v[h] = rows
 * h*kv_dim+nope .. +vdim of kv_b_proj.  c_acc fp32 [batch][n_heads][512] (the
 * output of the MLA kernels), attn_out fp32 [batch][n_heads][vdim]. */
int cwick_hip_mla_expand_dev(const uint16_t *kv_b_proj, const float *c_acc, int batch, int n_heads,
                             int nope, int vdim, int kv_dim, int kv_lora, float *attn_out,
                             void *stream);

/* Replaces the per-token loop of mixer_attn between the projections and the
 * attention (src/q35_model.c:1627-1652): for each of n tokens at positions
 * pos0.., every query head and every key head is RMS-normalised with (1 + w)
 * weights (rms_norm_w, :111-121; a NULL weight means no weight) and its first
 * rotary_dim dims are rotated, rotate-half form (rope_apply, :144-153), with
 * the cos/sin tables of build_rope (:459-476), [position][rotary_dim/2] fp32.
 * q_proj fp32 [n][n_heads] heads q_head_stride floats apart (2*head_dim when
 * the projection carries a gate per head, :1634-1637), k_proj and v_proj fp32
 * [n][n_kv_heads*head_dim].  q_out bf16 [n][n_heads][head_dim] is the query
 * operand of cwick_hip_gqa_decode_dev / _prefill_dev; the K and V rows are
 * narrowed to bf16 and stored into rows pos0.. of `cache` (the memcpy pair of
 * :1649-1651).  head_dim <= 256. */
int cwick_hip_gqa_prepare_dev(const float *q_proj, int64_t q_head_stride, const float *k_proj,
                              const float *v_proj, int64_t n, int64_t pos0, int n_heads,
                              int n_kv_heads, int head_dim, const float *q_norm,
                              const float *k_norm, float eps, const float *rope_cos,
                              const float *rope_sin, int rotary_dim, uint16_t *q_out,
                              cwick_hip_kv *cache, void *stream);

/* Replaces the attention of the block-sparse GQA decode (src/mm_model.c:
 * 1962-2047: per head, scores over the selected positions selpos[] with the
 * kv head h / group, max, exp, sum, normalise, weighted sum of the V rows).
 * sel[i] is a cache row; cwick_hip_mm_select_dev below writes the list on
 * the device.  Query heads per kv head: 1, 2, 4, 8 or 16.  Entries that are negative or not below the number of rows
 * carry no weight; a list without a valid entry gives zeros.  Softmax is a sum:
 * the order of the list does not matter beyond rounding. */
int cwick_hip_gqa_decode_sel(cwick_hip_kv *c, const int32_t *sel, int64_t n_list, const uint16_t *q,
                             int n_heads, float scale, float *out);
int cwick_hip_gqa_decode_sel_dev(const uint16_t *k, const uint16_t *v, int64_t n_rows, int n_kv_heads,
                                 int head_dim, const int32_t *sel, int64_t n_list,
                                 const uint16_t *q, int n_heads, float scale, float *out,
                                 void *stream);

/* Replaces what selects those positions: mm_index_scores (src/mm_model.c:
 * 1764-1780: per position, the dot of each index head's fp32 query with the
 * position's bf16 index key, one fused multiply-add per dimension in order
 * from zero, ReLU, the heads added in head order, no head weights),
 * mm_select_blocks (:1733-1761: a block scores its largest position score, the
 * keep_blocks best blocks are kept -- mm_topk, :777-814, whose choice on
 * tie-free input is the one made here: lowest index first among equal maxima
 * -- and block limit / block is added when it is not among them, which for a
 * limit that is a multiple of the block size is a block with nothing written
 * yet) and the loop that writes the kept blocks out as positions (:1969-1976).
 * Query t of the batch stands at position limit0 - 1 + t and sees limit0 + t
 * positions, as the queries of a prefill chunk do (:1962-1967); a decode step
 * is batch 1.  idx_keys bf16 [limit0 + batch - 1][index_dim] (one layer's slice
 * of the reference's idxcache), iq fp32 [batch][index_heads][index_dim],
 * scores fp32 [batch][score_stride] (out; row t is filled up to its limit),
 * blk_out int32 [batch][keep_blocks + 1] (out, may be NULL; ascending, -1
 * padded), sel int32 [batch][max_sel] (out; the positions in the reference's
 * order, cut at max_sel as the reference cuts at 4096, then -1: what
 * cwick_hip_gqa_decode_sel_dev takes with n_list = max_sel), n_sel int32
 * [batch] (out, may be NULL).  1..8 index heads, index_dim a multiple of 8 up
 * to 512, at most 16383 blocks. */
/* The same for one query of an engine whose state is in host memory: the index
 * keys are the K side of a cwick_hip_kv created with one head per position
 * (cwick_hip_kv_create(capacity, 1, index_dim); rows appended with
 * cwick_hip_kv_write, the V side unused), iq, blk_out (may be NULL), sel and
 * n_sel (may be NULL) are host pointers.  sel then feeds
 * cwick_hip_gqa_decode_sel with n_list = *n_sel. */
int cwick_hip_mm_select(cwick_hip_kv *idx, int64_t limit, const float *iq, int index_heads,
                        int block, int keep_blocks, int32_t *blk_out, int32_t *sel,
                        int64_t max_sel, int64_t *n_sel);
int cwick_hip_mm_select_dev(const uint16_t *idx_keys, const float *iq, int batch, int64_t limit0,
                            int index_heads, int index_dim, int block, int keep_blocks,
                            float *scores, int64_t score_stride, int32_t *blk_out,
                            int32_t *sel, int64_t max_sel, int32_t *n_sel, void *stream);

/* Replaces the closing of an indexer pool (indexer_absorb, src/attention.c:
 * 486-525; the two projections in front of it, :481-482, stay the caller's
 * GEMVs).  For each of n closed pools: layer-norm statistics of each of the
 * kpool raw key rows (mean and variance over the 128 dims, in double), a
 * softmax over the pool's slots, per dimension, of gate + position bias
 * (`ape`, bf16 [kpool][128]), the affine k_norm (weight and bias fp32 [128])
 * on the normalised rows, and their softmax-weighted mean as the pool's key.
 * raw_k and raw_gate fp32 [n][kpool][128] (tail_k / tail_g of the reference,
 * one pool after the other), kpool 1..8 (:492).  The key is quantised like
 * every row of the index-key store (one fp32 scale per row, amax / 448) and
 * stored as rows pos0 .. pos0+n of `slot`; rows_f32, if not NULL, also
 * receives the unquantised keys, fp32 [n][128] (st->pool of the reference). */
int cwick_hip_ikeys_pool_append_dev(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n,
                                    const float *raw_k, const float *raw_gate,
                                    const uint16_t *ape, const float *k_norm_w,
                                    const float *k_norm_b, float eps, int kpool,
                                    float *rows_f32, void *stream);

/* Replaces the rest of indexer_select behind the pool scores (src/attention.c:
 * 585-620), so that a chain indexer scores -> selection -> sparse attention
 * with index_kpool > 1 stays on the device.  scores fp32 [batch][n_comp], one
 * per closed pool of `kpool` positions (what cwick_hip_indexer_scores_dev
 * leaves); every query of the batch stands at position npos - 1, with
 * n_comp = npos / kpool.  want = ceil(topk / kpool) pools are kept: the best
 * by (score descending, pool index ascending), i.e. the reference's
 * `> thr` then `== thr` passes with thr the want-th largest score (its
 * quickselect can leave a larger threshold and then takes fewer pools,
 * src/attention.c:529-543 and :590; this call always takes `want`).  The
 * list sel[batch][max_sel] is in the reference's order: the pools above the
 * threshold ascending, then the pools at it, each as positions c*kpool + r
 * (:592-598); the npos % kpool positions behind the last closed pool
 * (:603-604); and, unless `strict` (CWICK_INDEXER_STRICT), npos - 1 when the
 * list does not already END with it (:618-620 tests the last entry only, so a
 * selected last pool that is not the threshold pool is followed by a second
 * copy of npos - 1, as in the reference).  Entries behind the list are -1;
 * n_sel[batch] (may be NULL) receives the count.  When n_comp <= want the
 * reference attends to the whole prefix (:558-559): the list is then
 * 0 .. npos-1 and n_sel is -1.  max_sel >= (want + 1) * kpool; pass sel with
 * n_list = max_sel to cwick_hip_mla_decode_dev, which skips the -1 entries. */
int cwick_hip_glm_select_dev(const float *scores, int batch, int64_t n_comp, int64_t npos,
                             int kpool, int64_t topk, int strict, int32_t *sel, int64_t max_sel,
                             int32_t *n_sel, void *stream);

/* Replaces level one of the two-level selection on the layer that is the
 * candidate source (src/ds_model.c:1125-1144): the maximum score of every
 * block of `block` positions, the last (partly filled) block forced in with
 * +inf (:1134-1135), the keep_blocks best blocks (ds_topk_scores, src/ds_ops.c:
 * 294-338; blocks of equal maximum are taken lowest index first, which is that
 * routine's choice on tie-free input), and a byte mask cand[batch][n], 1 inside
 * a kept block and 0 elsewhere.  scores fp32 [batch][n]; at most 16383 blocks
 * per row. */
int cwick_hip_candidate_select_dev(const float *scores, int batch, int64_t n, int block,
                                   int64_t keep_blocks, uint8_t *cand, void *stream);

/* Replaces the masking on the layers that use the candidates (src/ds_model.c:
 * 1145-1148): scores outside the kept blocks become -inf, in place, before
 * cwick_hip_topk_dev picks the positions. */
int cwick_hip_candidate_apply_dev(float *scores, const uint8_t *cand, int batch, int64_t n,
                                  void *stream);

/* Replace the fp32 copies of a prefix snapshot (cwick_engine_capture_prefix,
 * src/engine.c:3626-3641 for the latent rows, :3664-3666 for the indexer pool;
 * the layout is cwick_prefix_state's, src/pfx.h:63-67): rows pos0 .. pos0+n of
 * `slot` dequantised (byte value x the scale of its block) into host fp32,
 * [n][576] and [n][128].  Restoring is cwick_hip_latent_write_f32 /
 * cwick_hip_ikeys_write_f32; a read followed by a write reproduces the stored
 * bytes, and each scale to within one unit in its last place (448 s / 448
 * need not round back to s). */
int cwick_hip_latent_read_f32(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                              float *rows);
int cwick_hip_ikeys_read_f32(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n, float *rows);

/* ---- phase timers ------------------------------------------------------- */
/* Replace the reference's attention sub-timers (g_attn_*_ns, src/attention.c:1169-1174,
 * read out by src/prof.c:184-196 under CWICK_PROFILE; CWICK_Q35_PROF's
 * qk/softmax/av split, src/q35_model.c:72-99).  While enabled, an entry that
 * names one kernel is timed by a start and a stop event bound to that kernel's
 * dispatch (hipExtLaunchKernel): the kernel's own duration, as a kernel trace
 * reports it.  An entry that names several kernels is bracketed by a pair of
 * events recorded on the stream around the launches, which also counts the
 * dispatch latency between them.  cwick_hip_prof_read() waits for the
 * recorded events and returns the summed GPU time and the number of timed
 * sections since the last reset.  Off by default (no events are recorded). */
enum {
    CWICK_HIP_PROF_GQA_DECODE = 0,      /* gqa_decode_split_kernel */
    CWICK_HIP_PROF_GQA_DECODE_MERGE,    /* splitk_merge_wide_kernel<256|128> after it */
    CWICK_HIP_PROF_GQA_PREFILL,         /* gqa_prefill_kernel */
    CWICK_HIP_PROF_MLA,                 /* mla_roles_kernel (decode, sparse, prefill of at most 32 heads) */
    CWICK_HIP_PROF_MLA_MERGE,           /* mla_merge_frag16_kernel after it */
    CWICK_HIP_PROF_INDEXER,             /* indexer_scores_kernel, or in a fused select indexer_approx_kernel + topk_mw_hist_kernel + topk_mw_classify_kernel + indexer_rescore_kernel + the exact kernel's fallback pass */
    CWICK_HIP_PROF_TOPK,                /* every kernel of one top-k call: topk_mw_hist_kernel x4 + topk_mw_emit_kernel, or topk_radix[_reg]_kernel; in a fused select topk_band_finish_kernel */
    CWICK_HIP_PROF_MLA_PREFILL,         /* mla_prefill64_kernel (chunked prefill of more than 32 heads) */
    CWICK_HIP_PROF_MM_SELECT,           /* mm_index_scores[_long]_kernel + mm_pick_kernel; for block sizes that are not a multiple of 64 mm_blockmax_kernel and mm_expand_kernel, with the block top-k between them under CWICK_HIP_PROF_TOPK */
    CWICK_HIP_PROF_INDEXER_APPROX,      /* indexer_approx_kernel alone (also counted inside CWICK_HIP_PROF_INDEXER) */
    CWICK_HIP_PROF_COUNT
};
void cwick_hip_prof_enable(int on);
void cwick_hip_prof_reset(void);
int cwick_hip_prof_read(int which, double *total_ms, int64_t *launches);
const char *cwick_hip_prof_name(int which);

/* ---- measured ceilings -------------------------------------------------- */
/* The reference measures what a machine can do before judging a kernel against
 * it (tools/membwbench.c, tools/gpubw.m; docs/PERF.md:997-1042).  The same two
 * probes for this device: a 128-bit grid-stride read of `bytes` bytes (take
 * them well beyond the 256 MB of on-package cache), best of `reps` launches,
 * in GB/s; and a loop of nothing but matrix instructions on every SIMD, in
 * TFLOP/s -- kind 0: bf16 32x32x16, kind 1: FP8 (E4M3) 16x16x128, the form
 * the MLA score stage uses.  Both allocate and free their own buffers and use
 * the null stream; they are bench.py's, not the engine's. */
int cwick_hip_probe_hbm_read(size_t bytes, int reps, double *gbps);
int cwick_hip_probe_mfma(int kind, int reps, double *tflops);

/* Device-side codec check used by the parity tests: decodes all 256 E4M3
 * bytes with the conversion instruction the kernels use into out256 (host). */
int cwick_hip_e4m3_table(float *out256);

/* Device-side check of the lane exchanges the kernels are built on (sums, maxima and prefix sums
 * over a wave through DPP and lane swaps instead of LDS): one wave applies each of them to the 64
 * words of in64 (host); out832 (host) receives thirteen results of 64 words: sum, maximum, minimum
 * and inclusive prefix sum of the words as unsigned integers; then, on the floats
 * 1.m (m = the low 23 bits of a word), the maximum over the wave, the maximum and the sum over
 * lanes l and l ^ 16, over l and l ^ 32, and the sums over aligned groups of 2, 4, 8 and 16
 * lanes.  No counterpart in the reference (its reductions are NEON lanes and pthread slices);
 * used by the parity tests. */
int cwick_hip_lane_ops(const uint32_t *in64, uint32_t *out832);

#ifdef __cplusplus
}
#endif
#endif /* CWICK_HIP_H */
