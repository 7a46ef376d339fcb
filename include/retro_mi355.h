/*
 * retro_mi355.h — C ABI of libretro_mi355.so: MI355X (gfx950) kernels and host
 * services for RetroInfer's wave-index attention path.
 *
 * Conventions
 *  - Every pointer is a raw address: device memory unless the comment says "host".
 *    The library never allocates, frees or keeps tensor memory; buffers are borrowed
 *    for the duration of the call.  The only exception is the host wave buffer
 *    (ri_wavebuf_*), which — like the reference's WaveBufferCPU — remembers the pinned
 *    host arrays registered with set_indices/set_kv, so the caller keeps them alive.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Kernels
 *    are only enqueued; nothing synchronises unless stated.
 *  - Element type of K/V/centroid/query data is bfloat16 (uint16 bit patterns); every entry point whose
 *    arithmetic depends on the element type has a twin with the suffix _f16 for IEEE half (the copy and
 *    permutation entry points move 16-bit elements of either type).
 *    head_dim must be 128 (the reference hard-codes it: gather_copy.cu:196-199).
 *  - Return value: RI_OK (0) or a negative RI_ERR_* code; ri_status_string() names it
 *    and ri_last_hip_error() returns the HIP error behind RI_ERR_LAUNCH.
 *  - "group" g = batch * kv_heads + kv_head, BG groups in total; gs = query heads per
 *    KV head (<= 16).
 *
 * Each entry point cites the reference interface (file:line under the reference tree)
 * it stands in for.
 */
#ifndef RETRO_MI355_H
#define RETRO_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ri_stream_t;

enum {
  RI_OK = 0,
  RI_ERR_ARG = -1,       /* bad shape / null pointer / unsupported size */
  RI_ERR_LAUNCH = -2,    /* HIP reported an error at launch: see ri_last_hip_error() */
  RI_ERR_WORKSPACE = -3, /* workspace too small */
  RI_ERR_STATE = -4      /* host object used out of order */
};

const char* ri_status_string(int status);
int ri_last_hip_error(void);
/* ABI version: bumped when a signature changes. */
int ri_abi_version(void);   /* 6 */
/* Launches an empty kernel on `stream`: lets a caller measure the per-dispatch overhead that
 * event timings of back-to-back launches include.  No counterpart in the reference. */
int ri_null_launch(ri_stream_t stream);
/* Read-only streaming probe: `workgroups` workgroups of 256 threads read `bytes` bytes of `buf` once with
 * `loads_in_flight` (4, 8 or 16) 16-byte loads outstanding per thread and reduce them; `sink` (4 bytes of
 * device memory, or NULL) is written only if the reduction hits a magic value.  Lets a caller measure the
 * read bandwidth a kernel can reach on the part, the ceiling of the streaming kernels.  No counterpart in
 * the reference. */
int ri_probe_stream_read(const void* buf, size_t bytes, int workgroups, int loads_in_flight, void* sink,
                         ri_stream_t stream);

/* ------------------------------------------------------------------------------------
 * (2) Centroid scoring
 * ---------------------------------------------------------------------------------- */

/* Replaces retroinfer_kernels.batch_gemm_softmax
 * (library/retroinfer/retroinfer_kernels/src/batch_gemm_softmax.cu:171-198, pybind :201-209).
 *   A [batch, m, k] queries, B [batch, n, k] centroids (both bf16, k == 128, m <= 16,
 *   n % 8 == 0), D [batch, m, n] bf16 = bf16(alpha * A·Bᵀ), Softmax [batch, m, n] bf16 =
 *   bf16(exp(float(D) - rowmax) / rowsum) with rowmax/rowsum taken from the fp32 logits.
 *   Norm/Sum [batch, ceil(n/256), m] fp32: per-256-column partials; on return slot
 *   [batch, 0, :] holds the final row max and 1/rowsum (as the reference leaves them).
 *   beta must be 0. */
int ri_batch_gemm_softmax(const void* A, const void* B, void* D, float* Norm, float* Sum,
                          void* Softmax, int batch_count, int m, int n, int k, float alpha,
                          float beta, ri_stream_t stream);
/* The same operator on IEEE half inputs and outputs (batch_gemm_softmax.cu:185-197 accepts Half as
 * well as BFloat16): A, B, D and Softmax hold fp16, everything else as above. */
int ri_batch_gemm_softmax_f16(const void* A, const void* B, void* D, float* Norm, float* Sum,
                              void* Softmax, int batch_count, int m, int n, int k, float alpha,
                              float beta, ri_stream_t stream);

/* Fused scoring + selection: replaces the sequence batch_gemm_softmax → torch.sum →
 * masked_fill_ → torch.topk → cluster_ids.copy_ (cache_hub/retroinfer_cache.py:569-575).
 *   q          [BG, gs, 128] bf16
 *   centroids  [BG, nc, 128] bf16
 *   mask       [BG, nc] uint8 (1 = empty cluster, scored as finfo(bf16).min) or NULL
 *   cluster_size_i32 [BG, nc] int32 token count per cluster, or NULL (then no token layout)
 *   cluster_start    [BG, nc] int32 first row of the cluster in the cluster-contiguous
 *                    K/V store, or NULL
 * Outputs
 *   logits     [BG, gs, nc] fp32  = scale * q·c  (kept for the estimation zone)
 *   dist       [BG, nc] bf16 score or NULL
 *   cI         [BG, np+es] int64 or NULL: retrieval ids in rank order (score descending,
 *              ties by ascending id) followed by estimation ids in ascending id order
 *   ret_ids    [BG, np] int32, est_ids [BG, es] int32 (same content as cI)
 *   (np: 1..4096 clusters in the retrieval zone; nc <= 65536, a multiple of 8)
 *   ret_tok_off[BG, np+1] int32: exclusive token prefix of the retrieval clusters after
 *              the reference's buffer cut-off (stop before the first cluster whose pages
 *              push the running total over max_pages; wave_buffer_cpu.cpp:207-216)
 *              (entries from the last kept rank on hold the retrieved token count)
 *   ret_start  [BG, np] int32 or NULL: first store row of the cluster of every rank
 *   row_src    [BG, row_src_stride] int32: store row of every retrieved token, or NULL (the
 *              attention can work from ret_tok_off + ret_start instead, which is cheaper to write)
 *   meta       [BG, 4] int32: {clusters kept, retrieved tokens, pages used, 0}
 * workspace: ri_score_select_workspace_bytes(BG, gs, nc) bytes of device memory. */
size_t ri_score_select_workspace_bytes(int BG, int gs, int nc);
int ri_score_select(const void* q, const void* centroids, const uint8_t* mask,
                    const int32_t* cluster_size_i32, const int32_t* cluster_start,
                    float* logits, void* dist, int64_t* cI, int32_t* ret_ids,
                    int32_t* est_ids, int32_t* ret_tok_off, int32_t* ret_start, int32_t* row_src,
                    int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np, int es,
                    int page, int max_pages, float scale, void* workspace,
                    size_t workspace_bytes, ri_stream_t stream);
/* ri_score_select on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_score_select_f16(const void* q, const void* centroids, const uint8_t* mask,
                        const int32_t* cluster_size_i32, const int32_t* cluster_start,
                        float* logits, void* dist, int64_t* cI, int32_t* ret_ids,
                        int32_t* est_ids, int32_t* ret_tok_off, int32_t* ret_start, int32_t* row_src,
                        int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np, int es,
                        int page, int max_pages, float scale, void* workspace,
                        size_t workspace_bytes, ri_stream_t stream);

/* Scores only: logits[g, j, c] = scale * <q[g,j,:], centroids[g,c,:]> in fp32, no selection.
 * Used when the zones of a layer were chosen ahead of time from a predicted query
 * (use_cluster_estimation, cache_hub/retroinfer_cache.py:582-595) and the estimation zone must be
 * scored with the layer's true query (the reference does that by gathering the zone's centroids
 * and running weighted_flash_decoding over them, :598-617).
 * workspace: ri_score_select_workspace_bytes(BG, gs, nc). */
int ri_score_logits(const void* q, const void* centroids, float* logits, int BG, int gs, int nc,
                    float scale, void* workspace, size_t workspace_bytes, ri_stream_t stream);
/* ri_score_logits on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_score_logits_f16(const void* q, const void* centroids, float* logits, int BG, int gs, int nc,
                        float scale, void* workspace, size_t workspace_bytes, ri_stream_t stream);

/* ------------------------------------------------------------------------------------
 * (4) Weighted flash decoding
 * ---------------------------------------------------------------------------------- */

/* Replaces weighted_flash_decoding(q, k, v[, weight], previous_out=, previous_lse=,
 * cache_seqlens=, return_softmax_lse=) as called at cache_hub/retroinfer_cache.py:611-617
 * and :666-674 (the callee is an external fork that is not part of the reference tree).
 *   q [BG, gs, 128], k/v [BG, kv_stride rows, 128] bf16 (row r of group g at
 *   (g*kv_stride + r)*128), weight [BG, S] bf16 or NULL (multiplies each key's term in the
 *   softmax denominator only), cache_seqlens [BG] int32 or NULL (then every group has S
 *   rows), prev_out [BG, gs, 128] bf16 + prev_lse [BG, gs] fp32 or both NULL,
 *   out [BG, gs, 128] bf16, lse_out [BG, gs] fp32 or NULL.
 *   out = (e^{prev_lse}·prev_out + Σ_r e^{s_r} v_r) / (e^{prev_lse} + Σ_r w_r e^{s_r}),
 *   s_r = scale·q·k_r;  lse_out = log of that denominator.
 *   workspace: ri_flash_decoding_workspace_bytes(BG, gs) bytes of device memory that the
 *   caller zeroes once after allocating it (its head holds per-group arrival counters which
 *   every call leaves at zero again); calls sharing a workspace must not overlap in time.
 *   BG <= 4096. */
size_t ri_flash_decoding_workspace_bytes(int BG, int gs);
/* Clears the arrival counters at the head of an attention workspace (of ri_weighted_flash_decoding,
 * ri_wave_attention, ri_wave_attention_part or ri_buffer_attention) with a small kernel on `stream`; no
 * memset, so the call can be captured.  Every attention call leaves the counters at zero; this is for the
 * case that a launch did not run to its end (device fault or reset): counters left non-zero would make
 * every later call on that workspace write no output.  No counterpart in the reference. */
int ri_attention_workspace_reset(void* workspace, size_t workspace_bytes, ri_stream_t stream);
int ri_weighted_flash_decoding(const void* q, const void* k, const void* v, const void* weight,
                               const int32_t* cache_seqlens, const void* prev_out,
                               const float* prev_lse, void* out, float* lse_out, int BG,
                               int gs, int S, int64_t kv_stride, float scale, void* workspace,
                               size_t workspace_bytes, ri_stream_t stream);
/* ri_weighted_flash_decoding on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_weighted_flash_decoding_f16(const void* q, const void* k, const void* v, const void* weight,
                                   const int32_t* cache_seqlens, const void* prev_out,
                                   const float* prev_lse, void* out, float* lse_out, int BG,
                                   int gs, int S, int64_t kv_stride, float scale, void* workspace,
                                   size_t workspace_bytes, ri_stream_t stream);

/* Fused wave-index attention over a device-resident cluster store: replaces steps 4-8 of
 * retroinfer_cache.compute (gather_copy_vectors → weighted_flash_decoding →
 * gather_copy_and_concat → weighted_flash_decoding, cache_hub/retroinfer_cache.py:598-674)
 * when every cluster's K/V already sits in device memory, reading K/V in place (located through
 * the rank tables or a row table) instead of staging them in an execution buffer.
 *   steady_k/v [BG, steady_stride, 128]: first static_len rows attended; with static_len_dev (one
 *   int32 in device memory, or NULL) the count is read there when the kernel runs (clamped to
 *   [0, steady_stride]) and static_len only sizes the split: a captured launch then stays valid while
 *   the steady zone grows token by token
 *   store_k/v  [BG, store_stride, 128]: cluster-contiguous K/V
 *   row_src [BG, row_src_stride]: store row of every retrieved token; or NULL with ret_tok_off
 *   [BG, np+1] and ret_start [BG, np]: rank r's tokens are the store rows ret_start[r] + i
 *   meta, est_ids, logits: as written by ri_score_select (or meta by ri_lru_access_update)
 *   est_centroids [BG, nc, 128] bf16: given instead of logits (exactly one of the two is NULL when
 *   es > 0) when the zones were chosen from another query than q (next-layer cluster estimation,
 *   cache_hub/retroinfer_cache.py:582-617): the estimation zone's scores are then computed inside
 *   the launch from the centroid rows of est_ids
 *   np: 1..4096 probes with the rank tables (their 2 np + 1 words are staged in LDS); any number with
 *   a row table
 *   value_sum [BG, nc, 128] bf16, cluster_size_bf16 [BG, nc] bf16 (estimation weights)
 *   es may be 0 (no estimation zone).  out [BG, gs, 128] bf16; valid_lengths [BG] int32 or
 *   NULL receives static_len + retrieved tokens (what gather_copy_and_concat reports).
 *   workspace: same rules as ri_weighted_flash_decoding (zeroed once by the caller). */
size_t ri_wave_attention_workspace_bytes(int BG, int gs);
int ri_wave_attention(const void* q, const void* steady_k, const void* steady_v,
                      int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                      const void* store_k,
                      const void* store_v, int64_t store_stride, const int32_t* row_src,
                      int row_src_stride, const int32_t* ret_tok_off, const int32_t* ret_start, int np,
                      const int32_t* meta, const int32_t* est_ids,
                      const float* logits, const void* est_centroids, const void* value_sum,
                      const void* cluster_size_bf16, void* out, int32_t* valid_lengths,
                      int BG, int gs, int nc, int es, float scale, void* workspace,
                      size_t workspace_bytes, ri_stream_t stream);
/* ri_wave_attention on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_wave_attention_f16(const void* q, const void* steady_k, const void* steady_v,
                          int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                          const void* store_k,
                          const void* store_v, int64_t store_stride, const int32_t* row_src,
                          int row_src_stride, const int32_t* ret_tok_off, const int32_t* ret_start, int np,
                          const int32_t* meta, const int32_t* est_ids,
                          const float* logits, const void* est_centroids, const void* value_sum,
                          const void* cluster_size_bf16, void* out, int32_t* valid_lengths,
                          int BG, int gs, int nc, int es, float scale, void* workspace,
                          size_t workspace_bytes, ri_stream_t stream);

/* One part of a wave attention over a row table (host-resident store, block cache managed on the device;
 * cache_hub/retroinfer_cache.py:629-674, where the reference overlaps the transfer of missed blocks with
 * other work on its copy stream): as ri_wave_attention with row_src, but of the table's rows only those
 * whose source row lies in [src_row_lo, src_row_hi) are attended (the window may be empty: a block cache of
 * zero blocks has no cached rows).  (prev_out [BG, gs, 128] bf16, prev_lse
 * [BG, gs] fp32), both or neither, is an earlier part's result that is merged in (log-sum-exp rule);
 * lse_out [BG, gs] fp32 or NULL receives this part's log-sum-exp.  static_len = 0 leaves the steady zone
 * out, es = 0 the estimation zone.  Two calls over complementary windows, the second with the first's
 * (out, lse_out) as its previous result, equal one ri_wave_attention up to the bf16 rounding of the
 * intermediate output.  static_len_dev only counts for a part that attends the steady zone: with
 * static_len = 0 it is ignored (a caller that hands the same device length to both parts would otherwise
 * attend the steady zone twice).  A part that attends nothing (no steady zone, no estimation zone, no row inside the
 * window) writes zeros and a log-sum-exp of -inf, and such a previous result is ignored by the part that
 * merges it.  Workspace as for ri_wave_attention. */
int ri_wave_attention_part(const void* q, const void* steady_k, const void* steady_v,
                           int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                           const void* store_k, const void* store_v, int64_t store_stride,
                           const int32_t* row_src, int row_src_stride, int src_row_lo, int src_row_hi,
                           const int32_t* meta, const int32_t* est_ids, const float* logits,
                           const void* value_sum, const void* cluster_size_bf16, const void* prev_out,
                           const float* prev_lse, void* out, float* lse_out, int32_t* valid_lengths,
                           int BG, int gs, int nc, int es, float scale, void* workspace,
                           size_t workspace_bytes, ri_stream_t stream);
/* ri_wave_attention_part on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_wave_attention_part_f16(const void* q, const void* steady_k, const void* steady_v,
                               int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                               const void* store_k, const void* store_v, int64_t store_stride,
                               const int32_t* row_src, int row_src_stride, int src_row_lo, int src_row_hi,
                               const int32_t* meta, const int32_t* est_ids, const float* logits,
                               const void* value_sum, const void* cluster_size_bf16, const void* prev_out,
                               const float* prev_lse, void* out, float* lse_out, int32_t* valid_lengths,
                               int BG, int gs, int nc, int es, float scale, void* workspace,
                               size_t workspace_bytes, ri_stream_t stream);

/* ri_wave_attention for callers that cannot allocate device memory: code running under HIP stream
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * Same arguments and result as ri_wave_attention without the workspace: the arrival counters and the
 * split partials live in a static device array of ri_wave_attention_static_scratch_bytes() (8 MiB) that
 * each GPU holds from the moment the library is loaded until the process ends.  The call allocates and
 * frees nothing (no hipMalloc/hipFree, no allocating library routine); it enqueues one small kernel that
 * clears the counters and the attention kernel on `stream`.
 * Limit: RI_MAX_GROUPS counters plus BG * splits * pad(gs) * 520 bytes of partials must fit the array
 * (splits <= 64 per group, about 512-768 workgroups in total; pad(gs) = 4, 8 or 16) — every benchmark
 * shape needs under 4 MiB; larger shapes return RI_ERR_WORKSPACE.
 * Every call on one GPU shares that GPU's array: calls that overlap in time on one GPU (different
 * streams or threads) race and must be serialised by the caller. */
size_t ri_wave_attention_static_scratch_bytes(void);
int ri_wave_attention_static(const void* q, const void* steady_k, const void* steady_v,
                             int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                             const void* store_k, const void* store_v, int64_t store_stride,
                             const int32_t* row_src, int row_src_stride, const int32_t* ret_tok_off,
                             const int32_t* ret_start, int np, const int32_t* meta, const int32_t* est_ids,
                             const float* logits, const void* est_centroids, const void* value_sum,
                             const void* cluster_size_bf16, void* out, int32_t* valid_lengths, int BG,
                             int gs, int nc, int es, float scale, ri_stream_t stream);
/* ri_wave_attention_static on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_wave_attention_static_f16(const void* q, const void* steady_k, const void* steady_v,
                                 int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                 const void* store_k, const void* store_v, int64_t store_stride,
                                 const int32_t* row_src, int row_src_stride, const int32_t* ret_tok_off,
                                 const int32_t* ret_start, int np, const int32_t* meta, const int32_t* est_ids,
                                 const float* logits, const void* est_centroids, const void* value_sum,
                                 const void* cluster_size_bf16, void* out, int32_t* valid_lengths, int BG,
                                 int gs, int nc, int es, float scale, ri_stream_t stream);

/* Attention over an execution buffer with the estimation zone fused in: replaces
 * gather_copy_vectors → weighted_flash_decoding (estimation) and the final
 * weighted_flash_decoding with previous_out/previous_lse
 * (cache_hub/retroinfer_cache.py:598-617 and :666-674) when the retrieved K/V were staged by
 * gather_copy_and_concat (host-resident cluster store).
 *   buf_k/v [BG, buf_stride, 128]: rows [0, cache_seqlens[g]) attended, cache_seqlens [BG] int32
 *   as written by ri_gather_copy_and_concat; max_len: upper bound of the lengths (<= buf_stride);
 *   est_ids, logits: as written by ri_score_select for the same query; value_sum, cluster_size_bf16
 *   as for ri_wave_attention.  Workspace: ri_wave_attention_workspace_bytes, same rules. */
int ri_buffer_attention(const void* q, const void* buf_k, const void* buf_v, int64_t buf_stride,
                        const int32_t* cache_seqlens, int max_len, const int32_t* est_ids,
                        const float* logits, const void* value_sum, const void* cluster_size_bf16,
                        void* out, int BG, int gs, int nc, int es, float scale, void* workspace,
                        size_t workspace_bytes, ri_stream_t stream);
/* ri_buffer_attention on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_buffer_attention_f16(const void* q, const void* buf_k, const void* buf_v, int64_t buf_stride,
                            const int32_t* cache_seqlens, int max_len, const int32_t* est_ids,
                            const float* logits, const void* value_sum, const void* cluster_size_bf16,
                            void* out, int BG, int gs, int nc, int es, float scale, void* workspace,
                            size_t workspace_bytes, ri_stream_t stream);

/* ------------------------------------------------------------------------------------
 * (3) Wave-buffer copies
 * ---------------------------------------------------------------------------------- */

/* Replaces gather_copy_vectors (gather_copy.cu:25-96, kernel copy_kernel.cuh:43-88):
 * dst_keys[g, i] = src_keys[g, idx[g, copy_start+i]] for i < copy_num, same for values and
 * the 2-byte metadata.  idx [groups, index_size] int64. */
int ri_gather_copy_vectors(const void* src_keys, void* dst_keys, const void* src_values,
                           void* dst_values, const void* src_meta, void* dst_meta,
                           const int64_t* idx, int groups, int data_length, int buffer_length,
                           int index_size, int copy_start, int copy_num, ri_stream_t stream);

/* Replaces gather_copy_and_concat (gather_copy.cu:100-212, kernel copy_kernel.cuh:215-329).
 * Per group: dst = [src1[0:copy_vectors1] | src2 blocks | src3 blocks]; src2 (cluster store,
 * may be pinned host memory mapped into the device) is indexed by start vector, src3 (block
 * cache [groups, data_length3, 8, 128]) by block id; each block copies sizes[] (<= 8)
 * vectors to dst offset copy_vectors1 (+ all src2 vectors for src3) + dst_off[].  Index
 * arrays [groups, offset_length] int32 and counts [groups] int32 may live in pinned host
 * memory.  valid_lengths[g] = total vectors written. */
int ri_gather_copy_and_concat(const void* k1, const void* k2, const void* k3, void* kdst,
                              const void* v1, const void* v2, const void* v3, void* vdst,
                              const int32_t* off2, const int32_t* sizes2, const int32_t* dst2,
                              const int32_t* num2, const int32_t* off3, const int32_t* sizes3,
                              const int32_t* dst3, const int32_t* num3, int32_t* valid_lengths,
                              int groups, int data_length1, int data_length2, int data_length3,
                              int buffer_length, int offset_length, int copy_vectors1,
                              ri_stream_t stream);

/* Replaces gather_copy_and_scatter (gather_copy.cu:216-283, kernel copy_kernel.cuh:379-420):
 * cache[g, dst_block[g,j], 0:sizes[g,j]] = src[g, s_copy_start + src_off[g,j] : +sizes]. */
int ri_gather_copy_and_scatter(const void* ksrc, void* kcache, const void* vsrc, void* vcache,
                               const int32_t* src_off, const int32_t* sizes,
                               const int32_t* dst_block, const int32_t* num, int groups,
                               int data_length, int buffer_length, int offset_length,
                               int s_copy_start, ri_stream_t stream);

/* ------------------------------------------------------------------------------------
 * (1) Prefill k-means
 * ---------------------------------------------------------------------------------- */

/* Assignment step of _triton_k_means_train (cache_hub/kmeans.py:6-49, launch :101-111):
 * assign[p, n] = argmax_c <data[p,n,:], centroids[p,c,:]> with fp32 accumulation and the
 * smallest c on ties.  centroids [P, nc, 128] bf16 (nc % 32 == 0, kmeans.py:99), assign
 * [P, N] int32.  Problem p reads N data rows starting at row
 * (p / seg) * head_rows + (p % seg) * N of `data` (bf16, 128 wide): seg consecutive
 * segments per head, heads head_rows apart — the reshape of kmeans.py:242 without a copy;
 * seg = 1, head_rows = N for one problem per head.  (The reference's atomic sum/count side
 * effects are produced by ri_kmeans_update instead, in a fixed summation order.) */
int ri_kmeans_assign(const void* data, const void* centroids, int32_t* assign, int P, int N,
                     int nc, int seg, int64_t head_rows, ri_stream_t stream);
/* ri_kmeans_assign on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_kmeans_assign_f16(const void* data, const void* centroids, int32_t* assign, int P, int N,
                         int nc, int seg, int64_t head_rows, ri_stream_t stream);

/* Inverted lists: replaces triton_reverse_index (cache_hub/kmeans.py:128-173) in CSR form.
 * counts [P, nc] int32, offsets [P, nc+1] int32 (exclusive prefix), members [P, N] int32 =
 * token ids grouped by cluster, ascending inside each cluster.
 * workspace: ri_kmeans_workspace_bytes(P, N, nc). */
size_t ri_kmeans_workspace_bytes(int P, int N, int nc);
int ri_kmeans_build_lists(const int32_t* assign, int32_t* counts, int32_t* offsets,
                          int32_t* members, int P, int N, int nc, void* workspace,
                          size_t workspace_bytes, ri_stream_t stream);

/* Centroid update: replaces the atomic accumulation of _triton_assign_kernel
 * (kmeans.py:48-49) plus _triton_update_kernel (kmeans.py:52-80).  For every cluster with
 * counts > 0: mean = (Σ member rows) / count; if normalize, mean /= ||mean||₂;
 * centroids[p,c,:] = bf16(mean).  Empty clusters keep their centroid.
 * Σ is a fixed-order fp32 sum (the reference's atomics leave the order open): the list, in
 * ascending token order, is cut into blocks of 256 rows; each block is summed one row at a time
 * from +0, and the block sums are added in block order starting from the first block's.
 * workspace: ri_kmeans_reduce_workspace_bytes(P, N, nc), no initialisation needed. */
size_t ri_kmeans_reduce_workspace_bytes(int P, int N, int nc);
int ri_kmeans_update(const void* data, const int32_t* counts, const int32_t* offsets,
                     const int32_t* members, void* centroids, int P, int N, int nc, int seg,
                     int64_t head_rows, int normalize, void* workspace, size_t workspace_bytes,
                     ri_stream_t stream);
/* ri_kmeans_update on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_kmeans_update_f16(const void* data, const int32_t* counts, const int32_t* offsets,
                         const int32_t* members, void* centroids, int P, int N, int nc, int seg,
                         int64_t head_rows, int normalize, void* workspace, size_t workspace_bytes,
                         ri_stream_t stream);

/* Per-cluster value sums: replaces triton_index_add (cache_hub/kmeans.py:176-221).
 * value_sum[p,c,:] = bf16(Σ member value rows), Σ in the same fixed order as above. */
int ri_kmeans_value_sum(const void* values, const int32_t* counts, const int32_t* offsets,
                        const int32_t* members, void* value_sum, int P, int N, int nc,
                        void* workspace, size_t workspace_bytes, ri_stream_t stream);
/* ri_kmeans_value_sum on IEEE half instead of bfloat16 (every 16-bit tensor of the call; fp32 and integer
 * arguments as above; the reference's operators and cache take either type: batch_gemm_softmax.cu:185-197,
 * gather_copy.cu:63-67, and its harnesses default to fp16: simple_test.py:29). */
int ri_kmeans_value_sum_f16(const void* values, const int32_t* counts, const int32_t* offsets,
                            const int32_t* members, void* value_sum, int P, int N, int nc,
                            void* workspace, size_t workspace_bytes, ri_stream_t stream);

/* Device-side block cache manager: BufferManager::batch_access followed by
 * BufferManager::batch_update (wave_buffer_cpu.cpp:190-257 and :102-188) in one launch, one
 * workgroup per group, with no host round trip, for a host-resident cluster store.
 *   ret_ids [BG, np] int32: retrieved cluster ids in rank order (from ri_score_select)
 *   sizes, starts [BG, meta_stride] int32: tokens and first host-store row of every cluster
 *   blk_off [BG, blk_off_stride] int32: exclusive prefix of ceil(size / block), ncl + 1 entries
 * State, all device memory owned by the caller and only touched by this call:
 *   stamp [BG, stamp_stride] int32 (zero-initialised: nothing resident; else the step that last touched the
 *   cluster), order [BG, stamp_stride] int32 (the cluster's position inside that step, any initial content), blk_ids
 *   [BG, blk_ids_stride] int32 (cache block ids of resident clusters at blk_off),
 *   free_list [BG, capacity] int32 (initialised 0..capacity-1), free_count [BG] (= capacity),
 *   epoch [BG] (= 0).
 * Output lists [BG, buffer_size] int32 and counts [BG], in the layout ri_gather_copy_and_concat
 * and ri_gather_copy_and_scatter read: hit (cache block id, size, token offset), miss (host row,
 * size, token offset), update (execution-buffer token offset, size, cache block id).
 * Policy: the walk over the ranks stops at the first cluster whose blocks do not fit
 * buffer_size; the longest prefix of the misses that fits `capacity` is admitted; victims are
 * whole clusters from the least recently used end of the reference's list until the admission is covered
 * (wave_buffer_cpu.cpp:140-142).  The list is kept as (step, order inside the step) per cluster: the hits of a
 * call are touched in reverse rank order and the admitted misses pushed in rank order behind them
 * (:106-114, :170-176), so the hit / miss / admission lists and the evictions are those of the reference's
 * manager; block id values are the manager's own (the reference's come from an unordered_set).  np <= 4096, ncl <= 65536.  capacity may be 0 (no block cache, as
 * throughput_eval/test.py:77 runs the reference): every kept cluster is then a miss at every call and
 * nothing is admitted (wave_buffer_cpu.cpp:119-130 with a capacity of 0); free_list may then be NULL.
 * With row_src [BG, row_src_stride] and meta [BG, 4] (both or neither): for attention in place over
 * one tensor that holds the `capacity` cache blocks first and the staging rows of the misses from row
 * stage_row0 on, row_src receives the row of every retrieved token (hits: block id * block + i;
 * misses: stage_row0 + their offset in the miss list), meta {clusters kept, tokens, blocks, 0} as
 * ri_score_select writes it, and the hit count is reported as 0 (nothing to copy). */
int ri_lru_access_update(const int32_t* ret_ids, const int32_t* sizes, const int32_t* starts,
                         int meta_stride, const int32_t* blk_off, int blk_off_stride, int32_t* stamp,
                         int32_t* order, int stamp_stride, int32_t* blk_ids, int blk_ids_stride, int32_t* free_list,
                         int32_t* free_count, int32_t* epoch, int32_t* hit_ids, int32_t* hit_sizes,
                         int32_t* hit_cumsum, int32_t* hit_num, int32_t* miss_ids,
                         int32_t* miss_sizes, int32_t* miss_cumsum, int32_t* miss_num,
                         int32_t* upd_buf, int32_t* upd_sizes, int32_t* upd_cache, int32_t* upd_num,
                         int32_t* row_src, int row_src_stride, int stage_row0, int32_t* meta,
                         int BG, int np, int ncl, int buffer_size, int capacity, int block,
                         ri_stream_t stream);

/* Device-side replacement of WaveBufferCPU::organize_kv (wave_buffer_cpu.cpp:545-567):
 * out[p, i, :] = in[p, members[p, i], :] — K/V rows permuted into cluster-contiguous order. */
int ri_permute_rows(const void* in, const int32_t* members, void* out, int P, int N,
                    int64_t in_stride_rows, int64_t out_stride_rows, ri_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Host wave buffer (LRU block cache manager + K/V re-organisation) and its thread pool
 * ---------------------------------------------------------------------------------- */

typedef struct ri_threadpool ri_threadpool;
typedef struct ri_wavebuf ri_wavebuf;

/* Replaces ThreadPool / MyThreadPool (wave_buffer_cpu.cpp:17-35, thread_pool.hpp:27-141). */
ri_threadpool* ri_threadpool_create(int num_threads);
/* The same pool with worker i bound to core first_core + i, as set_affinity does for core i
 * (thread_pool.hpp:18-23, 65-66).  A worker whose core the process may not use stays unbound;
 * ri_threadpool_pinned_workers tells how many were bound.  NULL for first_core < 0. */
ri_threadpool* ri_threadpool_create_pinned(int num_threads, int first_core);
int ri_threadpool_pinned_workers(const ri_threadpool* pool);
void ri_threadpool_destroy(ri_threadpool* pool);

/* Replaces WaveBufferCPU (wave_buffer_cpu.cpp:328-383 ctor; pybind surface :822-849). */
ri_wavebuf* ri_wavebuf_create(int batch_size, int group_num, int dim, int nprobe,
                              int block_size, int n_centroids, int final_n_centroids,
                              int buffer_size, int capacity, int threads, ri_threadpool* pool);
void ri_wavebuf_destroy(ri_wavebuf* wb);
/* set_indices (wave_buffer_cpu.cpp:442-486): 12 host int32 arrays + searched ids (int64). */
int ri_wavebuf_set_indices(ri_wavebuf* wb, int32_t* hit_ids, int32_t* hit_sizes,
                           int32_t* hit_cumsum, int32_t* hit_nums, int32_t* miss_ids,
                           int32_t* miss_sizes, int32_t* miss_cumsum, int32_t* miss_nums,
                           int32_t* update_buffer_indices, int32_t* update_sizes,
                           int32_t* update_cache_indices, int32_t* update_nums,
                           int64_t* searched_clusters);
/* set_kv (wave_buffer_cpu.cpp:488-507): host arrays, 2-byte elements. */
int ri_wavebuf_set_kv(ri_wavebuf* wb, void* ivf_keys, void* ivf_values,
                      int64_t output_seq_length, void* input_keys, void* input_values,
                      int64_t input_seq_length);
/* async_construction / construction_sync (wave_buffer_cpu.cpp:592-630). */
int ri_wavebuf_async_construction(ri_wavebuf* wb, const int32_t* clusters,
                                  const int32_t* cluster_size, int64_t max_cluster_size,
                                  int batch_idx);
int ri_wavebuf_construction_sync(ri_wavebuf* wb);
/* update_kv (wave_buffer_cpu.cpp:688-720). */
int ri_wavebuf_update_kv(ri_wavebuf* wb, void* update_keys, void* update_values,
                         int64_t update_seq_length, const int32_t* clusters,
                         const int32_t* cluster_size, int update_n_centroids,
                         int64_t max_cluster_size);
/* batch_access = para_batch_access (wave_buffer_cpu.cpp:789-809); sync (:811-814). */
int ri_wavebuf_batch_access(ri_wavebuf* wb);
int ri_wavebuf_sync(ri_wavebuf* wb);
/* Number of clusters skipped so far because a group's pages exceeded buffer_size (the
 * reference prints a warning per event, wave_buffer_cpu.cpp:212-216). */
int64_t ri_wavebuf_overflow_events(const ri_wavebuf* wb);

#ifdef __cplusplus
}
#endif
#endif /* RETRO_MI355_H */
