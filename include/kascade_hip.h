/*
 * kascade_hip.h -- C ABI of libkascade_hip.so (gfx950 / MI355X).
 *
 * One shared library replaces the per-kernel shared objects the reference
 * builds with tilelang's LibraryGenerator and loads through
 * JITKernel.from_database (reference src/kernels/kernel_utils.py:15-81).  Each
 * of those objects exports `int init()`, `int call(<device pointers>, <dims>,
 * stream)` and `const char* get_last_error()`; this header keeps that
 * convention: every entry point takes raw device pointers owned by the
 * caller, plain integer sizes and a stream handle, allocates nothing, returns
 * 0 on success and -1 on failure, and leaves a message retrievable through
 * kascade_get_last_error().
 *
 * Conventions
 *   H = 32 query heads, G = 8 KV heads, D = 128, fp16 data, fp32 accumulate,
 *   prefill tile = 32 queries (the shapes the reference kernels are specialised
 *   to: EfficientKascadeStrategy.py:19-21).  `stream` is a hipStream_t passed
 *   as void* (NULL = the default stream).  Index tensors hold logical token ids.
 *   All softmax arithmetic is in the exp2 domain with
 *   scale = D^-0.5 * log2(e); log-sum values are log2(sum) + max*scale.
 *
 * Paged KV cache (extension of the reference's padded [B, maxL, G, D] cache)
 *   K/V pages are [num_pages, page_size, G, D] fp16; logical token i of
 *   sequence b lives in page block_table[b*max_pages + i/page_size], slot
 *   i % page_size.  page_size must be a power of two.  Passing
 *   block_table == NULL selects the reference's contiguous layout: K/V are
 *   [B, kv_stride_tokens, G, D] and token i of sequence b is row
 *   b*kv_stride_tokens + i.
 */
#ifndef KASCADE_HIP_H
#define KASCADE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t kascade_half; /* IEEE binary16 bit pattern */

/* Strides are in elements; the innermost (D) dimension is contiguous.  A tensor
 * laid out [B,L,H,D] has (s_b, s_l, s_h) = (L*H*D, H*D, D); HF's [B,H,L,D]
 * seen as [B,L,H,D] has (H*L*D, D, L*D). */
typedef struct {
    int64_t b, l, h;
} kascade_strides;

/* Tensor shape of a call.  The reference kernels exist for one shape only (32 query heads, 8 KV
 * heads, head dimension 128, fp16: EfficientKascadeStrategy.py:19-21, README.md:74-75), and the
 * entry points named after them take no shape.  Their `*_shaped_call` twins take this descriptor
 * as first argument and the argument list of the plain entry after it; every size that the
 * comments give as 32 / 8 / 128 reads group_size*kv_heads / kv_heads / head_dim there, and
 * kascade_half means an element of `dtype`.  Pooled scores stay fp16 for both element types.
 * No counterpart in the reference. */
enum { KASCADE_F16 = 0, KASCADE_BF16 = 1 };
typedef struct {
    int32_t kv_heads;   /* >= 1 */
    int32_t head_dim;   /* 64 or 128 */
    int32_t dtype;      /* KASCADE_F16 or KASCADE_BF16 */
    int32_t group_size; /* query heads per KV head: 1 to 16; 0 means 4 */
} kascade_shape;

/* Replaces `init()` of every reference kernel object (e.g. decode reuse .cu:253-258):
 * one-time device query and kernel attribute set-up for the current device. */
int kascade_init(void);

/* Replaces `get_last_error()` (e.g. decode reuse .cu:249-251).  Thread-local buffer. */
const char* kascade_get_last_error(void);

/* ABI version of this header (bumped on any signature change). */
int kascade_abi_version(void);

/* Number of compute units of the current device (0 before kascade_init). */
int kascade_device_cu_count(void);

/* ------------------------------------------------------------------ decode */

/* Every decode call splits each (sequence, KV head) row list over num_split workgroups that
 * write partial results (glse, Output_partial) and then merges them.  sync_counters selects
 * how (no counterpart in the reference, which always launches a second kernel):
 *   NULL      a second (combine) launch merges the splits;
 *   non-NULL  [batch*8] i32 in device memory, zero before the first call: the last split
 *             workgroup of each (sequence, KV head) to finish merges that pair's splits inside
 *             the same launch and sets its counter back to zero, so the array can be handed
 *             to the next call as it is.  One launch fewer per layer, which matters at short
 *             contexts.  Calls that overlap in time on one device must not share an array. */

/* Reuse-layer decode, contiguous cache.  Same argument list as the reference's
 * `call` of dynamic_alllen_reuse_cp_async_dim128_gsize4_heads32_groups8.cu:260
 * (DSL: reuse_kascade_gqa_decode.py:180-191) plus the split count that the
 * reference fixes at 8 through the shape of its scratch tensors.
 *   Q [B,H,D]  K,V [B,kv_seqlen,G,D]  topk_indices [B,G,topk] i32
 *   head_mapping [G] i32  glse [B,H,num_split] f32
 *   Output_partial [B,H,num_split,D] f32  Output [B,H,D] f16 */
int kascade_decode_reuse_call(const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                              const int32_t* topk_indices, const int32_t* head_mapping,
                              float* glse, float* Output_partial, kascade_half* Output,
                              int batch, int kv_seqlen, int topk, int num_split,
                              int32_t* sync_counters, void* stream);

/* Reuse-layer decode over a padded or paged cache with per-sequence lengths.
 * Argument order follows the reference's kvcache `call`
 * (dynamic_alllen_reuse_cp_async_dim128_gsize4_heads32_groups8_with_kvcache.cu:249;
 * DSL reuse_kascade_gqa_decode_with_kvcache.py:160-173) with the block table
 * added.  Sequence b consumes the first n(b) entries of its index rows,
 *   n(b) = 128*ceil(floor(topk_percent*cache_seqlens[b]/100)/128)  if topk_percent > 0
 *   n(b) = topk                                                   otherwise,
 * clamped to `topk` (the row width of topk_indices).
 *   block_table [B,max_pages] i32 or NULL (then K,V are [B,kv_stride_tokens,G,D]).
 *   kv_strides  NULL, or (only without a block table) the element strides (b, l, h) of K and V
 *               seen as [B,tokens,G,D]: multiples of 8, D contiguous.  Lets the kernels read a
 *               head-major [B,G,tokens,D] cache (Hugging Face's layout) in place, where the
 *               reference copies the whole cache to [B,tokens,G,D] on every decode step
 *               (EfficientKascadeStrategy.py:149-150).
 *   k_new,v_new NULL, or [B,G,D] f16: the K and V rows of each sequence's newest token, i.e. of
 *               position cache_seqlens[b]-1 (kv_stride_tokens-1 without cache_seqlens).  The
 *               launch writes them into that slot of the cache (through K and V) and attends
 *               to them, so a decode step needs no separate kascade_paged_kv_append_call.
 *   log_sum     NULL, or [B,H] f32: log2 of the sum of 2^(q.k*scale) over the rows each head
 *               attended to (the merged log-sum of the splits, which the reference's combine
 *               step forms and drops, reuse_kascade_gqa_decode.py:160-177).  Next to the dense
 *               log-sum of the same layer it says how much attention mass an index list covers,
 *               which is what the layer / head calibration measures. */
int kascade_decode_reuse_paged_call(const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    const int32_t* topk_indices, const int32_t* head_mapping,
                                    float topk_percent, float* glse, float* Output_partial,
                                    kascade_half* Output, int batch, int kv_stride_tokens,
                                    int topk, int num_split, const int32_t* block_table,
                                    int max_pages, int page_size, const kascade_strides* kv_strides,
                                    const kascade_half* k_new, const kascade_half* v_new,
                                    int32_t* sync_counters, float* log_sum, void* stream);
/* kascade_decode_reuse_paged_call for any kascade_shape. */
int kascade_decode_reuse_paged_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    const int32_t* topk_indices, const int32_t* head_mapping,
                                    float topk_percent, float* glse, float* Output_partial,
                                    kascade_half* Output, int batch, int kv_stride_tokens,
                                    int topk, int num_split, const int32_t* block_table,
                                    int max_pages, int page_size, const kascade_strides* kv_strides,
                                    const kascade_half* k_new, const kascade_half* v_new,
                                    int32_t* sync_counters, float* log_sum, void* stream);

/* Reuse-layer decode over a paged cache whose index lists were translated to cache rows once, at
 * the anchor (kascade_translate_indices_call): cache_rows [B,G,topk] holds page * page_size + slot
 * of every selected token, so the path from a list entry to its K/V row has one dependent load
 * instead of two (list -> block table -> row).  An anchor's selection serves every reuse layer up
 * to the next anchor, all over the same block table, so the translation is paid once per anchor.
 * No counterpart in the reference (its caches are contiguous).  Otherwise as
 * kascade_decode_reuse_paged_call: sequence b consumes the first n(b) entries of its rows (n(b)
 * from topk_percent and cache_seqlens, or topk).  cache_seqlens may be NULL when topk_percent
 * <= 0 and nothing is appended.  The block table is used by the fused append only.  Entries are
 * clamped to [0, num_pages * page_size). */
int kascade_decode_reuse_rows_call(const kascade_half* Q, const kascade_half* K_pages,
                                   const kascade_half* V_pages, const int32_t* cache_seqlens,
                                   const int32_t* cache_rows, const int32_t* head_mapping,
                                   float topk_percent, float* glse, float* Output_partial,
                                   kascade_half* Output, int batch, int topk, int num_split,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int num_pages, const kascade_half* k_new,
                                   const kascade_half* v_new, int32_t* sync_counters, float* log_sum, void* stream);
/* kascade_decode_reuse_rows_call for any kascade_shape. */
int kascade_decode_reuse_rows_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                   const kascade_half* V_pages, const int32_t* cache_seqlens,
                                   const int32_t* cache_rows, const int32_t* head_mapping,
                                   float topk_percent, float* glse, float* Output_partial,
                                   kascade_half* Output, int batch, int topk, int num_split,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int num_pages, const kascade_half* k_new,
                                   const kascade_half* v_new, int32_t* sync_counters, float* log_sum, void* stream);

/* kascade_decode_reuse_paged_call for callers that cannot allocate device memory and have no
 * scratch of their own to pass: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference.  The partial results of the splits
 * (glse, Output_partial) live in a buffer built into the library instead of in caller memory; the
 * splits are merged by the combine launch.  Everything else is the argument list above.
 *   Limit: batch * num_split <= 1024 (a 16.9 MB buffer per device, held until the process ends);
 *   larger launches are rejected with an error.  The call allocates and frees nothing.
 *   Every call on a device uses that device's one buffer, on whatever stream: calls that overlap
 *   in time on one device race.  Nothing in the buffer has to be cleared between calls (every
 *   entry a launch reads it has written itself).  kascade_init() on the device prepares the
 *   buffer's address; without it the first call does. */
int kascade_decode_reuse_paged_noalloc_call(const kascade_half* Q, const kascade_half* K,
                                            const kascade_half* V, const int32_t* cache_seqlens,
                                            const int32_t* topk_indices, const int32_t* head_mapping,
                                            float topk_percent, kascade_half* Output, int batch,
                                            int kv_stride_tokens, int topk, int num_split,
                                            const int32_t* block_table, int max_pages, int page_size,
                                            const kascade_strides* kv_strides,
                                            const kascade_half* k_new, const kascade_half* v_new,
                                            void* stream);

/* Dense split-K decode (the reference's TileLang dense baseline, gqa_decode.py:117-254 and
 * gqa_decode_with_kvcache.py:118-257), same cache conventions as above.
 * cache_seqlens may be NULL (all sequences have kv_stride_tokens tokens).  With a block
 * table kv_stride_tokens is an upper bound on the sequence lengths (0: max_pages*page_size);
 * it sizes the splits. */
int kascade_decode_dense_paged_call(const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    float* glse, float* Output_partial, kascade_half* Output,
                                    int batch, int kv_stride_tokens, int num_split,
                                    const int32_t* block_table, int max_pages, int page_size,
                                    const kascade_strides* kv_strides, const kascade_half* k_new,
                                    const kascade_half* v_new, int32_t* sync_counters,
                                    void* stream);
/* kascade_decode_dense_paged_call for any kascade_shape. */
int kascade_decode_dense_paged_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    float* glse, float* Output_partial, kascade_half* Output,
                                    int batch, int kv_stride_tokens, int num_split,
                                    const int32_t* block_table, int max_pages, int page_size,
                                    const kascade_strides* kv_strides, const kascade_half* k_new,
                                    const kascade_half* v_new, int32_t* sync_counters,
                                    void* stream);

/* Anchor-layer decode: split QK^T (+PV when with_output != 0), log-sum merge and
 * pooled post-softmax scores.  Replaces the three launches of the reference's
 * flashattn_gqa_decode_split_{0,1} (recompute_kascade_gqa_decode.py:318-348;
 * kvcache form recompute_kascade_gqa_decode_with_kvcache.py:302-333).
 *   scores            B*H*scores_stride floats of scratch, scores_stride a multiple of 8, that
 *                     carry the raw q.k from the streaming launch to the pooling launch; the
 *                     contents are private to the library (per head 16-bit codes in steps of
 *                     2^-11 of the exponent below a per-64-token fp32 reference: a third of an
 *                     fp16 step on the pooled value, where the reference's fp16 raw scores
 *                     (recompute_kascade_gqa_decode.py:102) lose up to two)
 *   row_sums          [B,H] f32: global log2-domain log-sum per head
 *   aggregated_scores [B,G,scores_stride] f16: sum over the 4 heads of a KV head
 *                     of softmax probabilities; 0 at positions >= cache_seqlens[b]
 *   Output            [B,H,D] f16, written only when with_output != 0. */
int kascade_decode_recompute_paged_call(const kascade_half* Q, const kascade_half* K,
                                        const kascade_half* V, const int32_t* cache_seqlens,
                                        float* glse, float* Output_partial, float* row_sums,
                                        float* scores, kascade_half* Output,
                                        kascade_half* aggregated_scores, int batch,
                                        int kv_stride_tokens, int scores_stride, int num_split,
                                        int with_output, const int32_t* block_table,
                                        int max_pages, int page_size,
                                        const kascade_strides* kv_strides,
                                        const kascade_half* k_new, const kascade_half* v_new,
                                        int32_t* sync_counters, void* stream);
/* kascade_decode_recompute_paged_call for any kascade_shape. */
int kascade_decode_recompute_paged_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                        const kascade_half* V, const int32_t* cache_seqlens,
                                        float* glse, float* Output_partial, float* row_sums,
                                        float* scores, kascade_half* Output,
                                        kascade_half* aggregated_scores, int batch,
                                        int kv_stride_tokens, int scores_stride, int num_split,
                                        int with_output, const int32_t* block_table,
                                        int max_pages, int page_size,
                                        const kascade_strides* kv_strides,
                                        const kascade_half* k_new, const kascade_half* v_new,
                                        int32_t* sync_counters, void* stream);

/* ------------------------------------------------------------------- top-k */

/* Exact per-row top-n selection over non-negative-or--inf fp16 scores; replaces
 * the ATen torch.topk call sites (EfficientKascadeStrategy.py:82, 90, 111).
 *   scores  [rows, row_stride] f16
 *   out_idx [rows, k] i32
 * Row r looks at its first valid_len[r % period] entries (valid_len == NULL:
 * uniform_len) and must select n_sel[r % period] of them (n_sel == NULL: k).
 * Slots [0, n) receive exactly the n largest entries (ties broken towards the
 * lower index), ordered by ascending index; when fewer than n entries are valid
 * all valid ones are emitted followed by the first invalid positions, as
 * torch.topk does for -inf padding.  Slots [n, k) are set to fill_value.
 * uniform_len is also the upper bound of every valid_len entry (longer entries are clamped).
 *   workspace: NULL, or device scratch of kascade_topk_workspace_bytes(rows, uniform_len)
 *   bytes.  With a workspace, long rows (that function returns > 0) are selected by several
 *   workgroups per row -- coarse histograms merged with atomics, per-chunk counts, ordered
 *   compaction -- with identical results; without one, one workgroup handles each row. */
int64_t kascade_topk_workspace_bytes(int rows, int64_t row_len);
int kascade_topk_call(const kascade_half* scores, int32_t* out_idx, int rows, int64_t row_stride,
                      int uniform_len, const int32_t* valid_len, const int32_t* n_sel, int period,
                      int k, int fill_value, void* workspace, void* stream);

/* kascade_topk_call with a second output: every selected position also as a row of a paged
 * cache, out_rows[r, i] = block_table[r / rows_per_sequence, t / page_size] * page_size +
 * t % page_size for t = out_idx[r, i] (fill slots included), which is what
 * kascade_decode_reuse_rows_call and kascade_prefill_chunk_reuse_call gather from -- the
 * translation of kascade_translate_indices_call without its launch.  out_rows [rows, k] i32 or
 * NULL (then the block-table arguments are ignored); rows_per_sequence consecutive score rows
 * belong to one sequence (8 for decode rows, 8 * tiles for prefill rows). */
int kascade_topk_rows_call(const kascade_half* scores, int32_t* out_idx, int rows, int64_t row_stride,
                           int uniform_len, const int32_t* valid_len, const int32_t* n_sel, int period,
                           int k, int fill_value, void* workspace, int32_t* out_rows,
                           const int32_t* block_table, int max_pages, int page_size,
                           int rows_per_sequence, void* stream);

/* The selection in the form torch.topk(scores[..., :uniform_len], k).indices has
 * (EfficientKascadeStrategy.py:82, 90, 111): full-width rows ordered by descending score, for a
 * consumer that slices its own prefix of a row.
 *   out_idx [rows, k] i32: the k largest entries among the first valid_len[r % period] of row r
 *   (valid_len == NULL: uniform_len), largest first, equal scores by ascending position.  A row
 *   with fewer than k valid entries lists all of them in that order, then the positions
 *   valid_len, valid_len + 1, ... (where the reference's tensor holds -inf; torch.topk leaves
 *   the choice among those open).  0 < k <= uniform_len.
 *   workspace: device scratch of kascade_topk_sorted_workspace_bytes(rows, uniform_len, k) bytes
 *   (NULL when that is 0: lists of up to 4096 entries over rows short enough for one workgroup).
 * Runs kascade_topk_call and then a stable two-pass radix sort of each row's list. */
int64_t kascade_topk_sorted_workspace_bytes(int rows, int64_t row_len, int k);
int kascade_topk_sorted_call(const kascade_half* scores, int32_t* out_idx, int rows, int64_t row_stride,
                             int uniform_len, const int32_t* valid_len, int period, int k,
                             void* workspace, void* stream);

/* ----------------------------------------------------------------- prefill */

/* Anchor layer 0: dense causal GQA flash attention that also emits the log2
 * log-sum per (token, head).  Replaces `prefill`
 * (recompute_kascade_gqa_prefill.py:225-274).  with_output == 0 gives
 * `compute_scores` (same file :277-312): log_sum only, V and Output unused.
 *   Q [B,L,H,D]  K,V [B,L,G,D]  log_sum [B,L,H] f32  Output [B,L,H,D] f16 (contiguous) */
int kascade_prefill_dense_call(const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               float* log_sum, kascade_half* Output, int batch, int seq_len,
                               kascade_strides q_strides, kascade_strides kv_strides,
                               int with_output, void* stream);
/* kascade_prefill_dense_call for any kascade_shape. */
int kascade_prefill_dense_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               float* log_sum, kascade_half* Output, int batch, int seq_len,
                               kascade_strides q_strides, kascade_strides kv_strides,
                               int with_output, void* stream);

/* Pooled tile scores.  Same argument list as the reference's aggregate `call`
 * (dynamic_alllen_aggregate_cp_async_ts32_dim128_gsize4_heads32_groups8.cu:138;
 * DSL recompute_kascade_gqa_prefill.py:192-222) plus strides and fill_invalid:
 *   aggregate_scores [B,G,ceil(L/32),L] f16; entry (t, j) for j < 32 t is
 *   sum over the 32 queries of tile t and the 4 heads of the KV head of
 *   exp2(q.k*scale - log_sum).  With fill_invalid != 0 the entries j >= 32 t are
 *   written as -inf (the reference pre-fills the tensor on the host instead). */
int kascade_prefill_aggregate_call(const kascade_half* Q, const kascade_half* K,
                                   const float* log_sum, kascade_half* aggregate_scores, int batch,
                                   int seq_len, kascade_strides q_strides,
                                   kascade_strides kv_strides, int fill_invalid, void* stream);
/* kascade_prefill_aggregate_call for any kascade_shape. */
int kascade_prefill_aggregate_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                   const float* log_sum, kascade_half* aggregate_scores, int batch,
                                   int seq_len, kascade_strides q_strides,
                                   kascade_strides kv_strides, int fill_invalid, void* stream);

/* kascade_prefill_aggregate_call for a range of query tiles of a long prompt, so that the pooled
 * scores of a prompt never have to exist all at once (they take L^2/4 bytes per sequence: 8 GiB at
 * 131072 tokens).  The reference chunks only its torch.topk call, by rows, above 131072 tokens
 * (EfficientKascadeStrategy.py:83-90) and keeps the whole score tensor.
 *   Q        the q_len query rows at positions q_start .. q_start+q_len-1 (q_start a multiple of
 *            32): a view into the prompt's Q, [B,q_len,H,D] through q_strides
 *   K        the prompt's keys [B,>=q_start+q_len,G,D] through kv_strides
 *   log_sum  [B,q_len,H] f32, the rows of the log-sum pass that belong to these queries
 *   aggregate_scores [B,G,ceil(q_len/32),q_start+q_len] f16; row t is valid for keys < q_start+32t */
int kascade_prefill_aggregate_range_call(const kascade_half* Q, const kascade_half* K,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, kascade_strides kv_strides,
                                         int fill_invalid, void* stream);
/* kascade_prefill_aggregate_range_call for any kascade_shape. */
int kascade_prefill_aggregate_range_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, kascade_strides kv_strides,
                                         int fill_invalid, void* stream);

/* Reuse-layer prefill.  Same argument list as the reference's reuse `call`s
 * (…reuse_cp_async_ts32…groups8_rolling.cu:268 and …groups8.cu:260; DSL
 * reuse_kascade_gqa_prefill.py:147-198) plus strides and the rolling switch that
 * the reference bakes into two separate objects.
 *   topk_indices [B,G,ceil(L/32),max_topk_num] i32, head_mapping [G] i32.
 *   rolling != 0 and seq_len > 128: tile t uses its first
 *   128*ceil(max(floor(topk_percent*32t/100),128)/128) indices, else max_topk_num.
 *   log_sum NULL, or [B,L,H] f32: per (token, head) log2 of the sum of 2^(q.k*scale) over the keys
 *   the row attended to (its tile's list and its own tile up to itself); see
 *   kascade_decode_reuse_paged_call. */
int kascade_prefill_reuse_call(const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               const int32_t* topk_indices, const int32_t* head_mapping,
                               float topk_percent, kascade_half* Output, int batch, int seq_len,
                               int max_topk_num, int rolling, kascade_strides q_strides,
                               kascade_strides kv_strides, float* log_sum, void* stream);
/* kascade_prefill_reuse_call for any kascade_shape. */
int kascade_prefill_reuse_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               const int32_t* topk_indices, const int32_t* head_mapping,
                               float topk_percent, kascade_half* Output, int batch, int seq_len,
                               int max_topk_num, int rolling, kascade_strides q_strides,
                               kascade_strides kv_strides, float* log_sum, void* stream);

/* --------------------------------------------------------------- KV append */

/* Writes n_new tokens per sequence into the paged cache at logical positions
 * start_pos[b] .. start_pos[b]+n_new-1.  The reference has no counterpart (it
 * re-materialises the whole cache every step: EfficientKascadeStrategy.py:149-150);
 * this is the step right before the decode path.
 *   k_new, v_new [B,n_new,G,D] with strides new_strides (b, l, h=g).
 *   n_new_rows   NULL, or [B] i32: sequence b brings only its first n_new_rows[b] (<= n_new) rows.
 *   Positions beyond what the block table covers are skipped. */
int kascade_paged_kv_append_call(kascade_half* K_pages, kascade_half* V_pages,
                                 const kascade_half* k_new, const kascade_half* v_new,
                                 const int32_t* start_pos, const int32_t* block_table, int batch,
                                 int n_new, int max_pages, int page_size,
                                 kascade_strides new_strides, const int32_t* n_new_rows, void* stream);
/* kascade_paged_kv_append_call for any kascade_shape. */
int kascade_paged_kv_append_shaped_call(const kascade_shape* shape, kascade_half* K_pages, kascade_half* V_pages,
                                 const kascade_half* k_new, const kascade_half* v_new,
                                 const int32_t* start_pos, const int32_t* block_table, int batch,
                                 int n_new, int max_pages, int page_size,
                                 kascade_strides new_strides, const int32_t* n_new_rows, void* stream);

/* The hand-off from a decoder layer's projections to the attention path in one launch: RMS
 * normalisation of every query and key head (optional), rotary position embedding of queries
 * and keys, queries written as [B,n_new,H,D], keys and values written into their page slots.
 * No kernel of the reference does this: its transformers dependency runs these steps as
 * separate tensor operations inside the attention module before the registered attention
 * function is called, and the strategy then transposes (and, when decoding, copies) the
 * results (EfficientKascadeStrategy.py:144-150).
 *   q_in [B,n_new,H,D], k_in / v_in [B,n_new,G,D] through element strides (b, l, h), multiples
 *        of 8 with D contiguous (e.g. views of one packed projection output); NULL strides =
 *        contiguous.
 *   cos_sin [max_pos, D] f32: row p holds cos(p*f_i), i < D/2, then sin(p*f_i); element i of a
 *        head pairs with element i + D/2 ("rotate half").
 *   q_norm_weight, k_norm_weight [D] f16 or NULL (no normalisation); the normalised value is
 *        rounded to f16 before and after the weight, as the library's module does.
 *   Token t of sequence b sits at position start_pos[b] + pos_offset + t; negative positions
 *   and positions beyond the block table are skipped, angles beyond max_pos use the last row. */
int kascade_rope_append_paged_call(const kascade_half* q_in, const kascade_strides* q_strides,
                                   const kascade_half* k_in, const kascade_half* v_in,
                                   const kascade_strides* kv_strides, const float* cos_sin,
                                   int max_pos, const kascade_half* q_norm_weight,
                                   const kascade_half* k_norm_weight, float norm_eps,
                                   const int32_t* start_pos, int pos_offset, kascade_half* q_out,
                                   kascade_half* K_pages, kascade_half* V_pages,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int batch, int n_new, void* stream);
int kascade_rope_append_paged_shaped_call(const kascade_shape* shape, const kascade_half* q_in, const kascade_strides* q_strides,
                                   const kascade_half* k_in, const kascade_half* v_in,
                                   const kascade_strides* kv_strides, const float* cos_sin,
                                   int max_pos, const kascade_half* q_norm_weight,
                                   const kascade_half* k_norm_weight, float norm_eps,
                                   const int32_t* start_pos, int pos_offset, kascade_half* q_out,
                                   kascade_half* K_pages, kascade_half* V_pages,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int batch, int n_new, void* stream);

/* Bookkeeping of a ragged decode step in one small launch (no reference counterpart; the
 * reference's benchmark computes these on the host, recompute_kascade_gqa_decode_with_kvcache.py:
 * 368-377).  Adds `advance` to every cache_seqlens[b] in place (1 when the step's new token is
 * appended by the decode calls themselves, 0 to leave the lengths alone) and writes, per
 * (sequence, KV head) row r = b*8+g (b*kv_heads+g for the shaped twin) of the pooled scores, what kascade_topk_call takes as
 * valid_len / n_sel:  valid_len_rows[r] = len_b,
 *                     n_sel_rows[r]     = 128*ceil(floor(topk_percent*len_b/100)/128),
 * with len_b the length after the advance.  Either output may be NULL.  A sequence of length 0
 * is an empty slot of the batch: it is not advanced (and the decode calls append nothing to it). */
int kascade_decode_budgets_call(int32_t* cache_seqlens, int advance, float topk_percent, int batch,
                                int32_t* valid_len_rows, int32_t* n_sel_rows, void* stream);
int kascade_decode_budgets_shaped_call(const kascade_shape* shape, int32_t* cache_seqlens, int advance,
                                       float topk_percent, int batch, int32_t* valid_len_rows,
                                       int32_t* n_sel_rows, void* stream);

/* ------------------------------------------- chunked prefill over the paged cache */

/* The reference prefills a prompt in one call over contiguous K/V
 * (EfficientKascadeStrategy.py:110-147).  A serving engine prefills in chunks: the chunk's K/V
 * are appended to the paged cache first, then its queries attend to everything cached so far.
 * These three calls are the three prefill kernels above with
 *   - queries Q [B,q_len,H,D] (strides q_strides) at global positions q_start .. q_start+q_len-1,
 *     q_start a multiple of 32 and the same for every sequence of the batch;
 *   - keys = cache positions 0 .. q_start+q_len-1, read from K_pages/V_pages
 *     [num_pages,page_size,G,D] through block_table [B,max_pages];
 *   - outputs indexed by the chunk's own rows: log_sum [B,q_len,H], Output [B,q_len,H,D],
 *     aggregate_scores [B,G,ceil(q_len/32),q_start+q_len].
 * With q_start = 0 and q_len = L they compute what the whole-prompt calls compute; a prompt
 * processed in 32-aligned chunks gives bit-identical rows.  No counterpart in the reference.
 *
 * A batch whose sequences stand at different positions passes two more arrays (both NULL: every
 * sequence starts at q_start and owns all q_len rows):
 *   q_start_rows [B] i32: first global position of sequence b's rows, a multiple of 32 and at most
 *                q_start, which then is the largest of them (it sizes aggregate_scores and is what
 *                the block table must cover);
 *   q_len_rows   [B] i32 or NULL: how many of the q_len rows of Q belong to sequence b (0: none).
 * Rows beyond a sequence's own are left alone: no Output, no log_sum; their tiles' pooled scores
 * are not written (-inf with fill_invalid).  Sequence b then attends to cache positions
 * [0, q_start_rows[b] + q_len_rows[b]) and gets exactly the rows it gets in a call of its own;
 * without the rolling budget a sparse tile uses min(max_topk_num, the row width of a prompt of the
 * sequence's own length) entries of its list. */
int kascade_prefill_chunk_dense_call(const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, float* log_sum,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     kascade_strides q_strides, const int32_t* block_table,
                                     int max_pages, int page_size, int num_pages, int with_output, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows,
                                     void* stream);
int kascade_prefill_chunk_dense_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, float* log_sum,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     kascade_strides q_strides, const int32_t* block_table,
                                     int max_pages, int page_size, int num_pages, int with_output, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows,
                                     void* stream);

int kascade_prefill_chunk_aggregate_call(const kascade_half* Q, const kascade_half* K_pages,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, const int32_t* block_table,
                                         int max_pages, int page_size, int num_pages,
                                         int fill_invalid, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, void* stream);
int kascade_prefill_chunk_aggregate_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, const int32_t* block_table,
                                         int max_pages, int page_size, int num_pages,
                                         int fill_invalid, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, void* stream);

/* physical_rows [B,G,ceil(q_len/32),max_topk_num]: the tile's top-k tokens already translated
 * to rows of the paged cache (kascade_translate_indices_call), so that the gather needs no
 * second dependent load. */
int kascade_prefill_chunk_reuse_call(const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, const int32_t* physical_rows,
                                     const int32_t* head_mapping, float topk_percent,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     int max_topk_num, int rolling, kascade_strides q_strides,
                                     const int32_t* block_table, int max_pages, int page_size,
                                     int num_pages, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, float* log_sum, void* stream);
int kascade_prefill_chunk_reuse_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, const int32_t* physical_rows,
                                     const int32_t* head_mapping, float topk_percent,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     int max_topk_num, int rolling, kascade_strides q_strides,
                                     const int32_t* block_table, int max_pages, int page_size,
                                     int num_pages, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, float* log_sum, void* stream);

/* physical_rows[b,i] = block_table[b, t / page_size] * page_size + t % page_size with
 * t = clamp(token_idx[b,i], 0, kv_len-1), i < per_sequence.  physical_rows may alias token_idx.
 * No counterpart in the reference (its prefill never sees a paged cache). */
int kascade_translate_indices_call(const int32_t* token_idx, int32_t* physical_rows,
                                   const int32_t* block_table, int batch, int64_t per_sequence,
                                   int max_pages, int page_size, int kv_len, void* stream);

/* ------------------------------------ the reference's argument lists, verbatim */

/* The five kernel objects the reference ships as generated sources each export
 * `call(<pointers>, <dims>, stream)`.  The entry points below take exactly those argument lists,
 * in that order and with those types, so a loader that binds the reference's `call` can bind
 * these instead; each forwards to the entry point above that does the work, with what the
 * reference fixes implicitly: contiguous [B,L,heads,128] tensors, 8 splits (the shape of the
 * reference's glse [B,32,8] and Output_partial [B,32,8,128] scratch: attention_utils.py:36-59,
 * EfficientKascadeStrategy.py:103-104, 119-120), a combine launch, no -inf fill by the kernel
 * (the reference pre-fills aggregate_scores on the host, EfficientKascadeStrategy.py:75-76). */

/* `call` of flash_decoding/kascade_decode_cu_kernels/
 * dynamic_alllen_reuse_cp_async_dim128_gsize4_heads32_groups8.cu:260 */
int kascade_ref_decode_reuse_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                  int* topk_indices, int* head_mapping, float* glse,
                                  float* Output_partial, kascade_half* Output, int batch,
                                  int kv_seqlen, int topk, void* stream);

/* `call` of ..._groups8_with_kvcache.cu:249 (K, V [B,max_cache_seqlen,8,128]) */
int kascade_ref_decode_reuse_kvcache_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                          int* cache_seqlens, int* topk_indices, int* head_mapping,
                                          float topk_percent, float* glse, float* Output_partial,
                                          kascade_half* Output, int batch, int max_cache_seqlen,
                                          int topk, void* stream);

/* `call` of flash_attention/kascade_prefill_cu_kernels/
 * dynamic_alllen_aggregate_cp_async_ts32_dim128_gsize4_heads32_groups8.cu:138 */
int kascade_ref_prefill_aggregate_call(kascade_half* Q, kascade_half* K, float* log_sum,
                                       kascade_half* aggregate_scores, int batch, int seq_len,
                                       void* stream);

/* `call` of ...reuse_cp_async_ts32_dim128_gsize4_heads32_groups8_rolling.cu:268 */
int kascade_ref_prefill_reuse_rolling_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                           int* topk_indices, int* head_mapping,
                                           float topk_percent, kascade_half* Output, int batch,
                                           int seq_len, int max_topk_num, void* stream);

/* `call` of ...reuse_cp_async_ts32_dim128_gsize4_heads32_groups8.cu:260 (every tile uses topk_num) */
int kascade_ref_prefill_reuse_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                   int* topk_indices, int* head_mapping, float topk_percent,
                                   kascade_half* Output, int batch, int seq_len, int topk_num,
                                   void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KASCADE_HIP_H */
