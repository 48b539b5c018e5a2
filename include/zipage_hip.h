/* C ABI of libzipage_hip.so: hand-written gfx950 (MI355X) kernels for the KV-cache
 * compression path of compressed PagedAttention.
 *
 * The reference (microsoft/Zipage) has no FFI on this path: its boundary is the set of
 * Python functions under zipage/kernel/.  Each entry point below replaces the device
 * work of one of them and is what a Python (ctypes) or C++ host binds; the citation on
 * each declaration names the reference interface it stands in for.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is retained;
 *   - dims are int32, strides are int64 and counted in ELEMENTS; the innermost
 *     (head_dim / slot) axis of every tensor has stride 1;
 *   - `dtype` tags the element type of caches and scores (zp_dtype);
 *   - `stream` is a hipStream_t passed as void*; calls only enqueue work on it, never
 *     synchronise the device and never allocate;
 *   - functions return ZP_OK or an error code; zp_last_error() gives the thread-local
 *     message of the last failure on the calling thread;
 *   - block tables are contiguous int32 (B, NB): id >= 0 full page, -1 padding,
 *     x < -1 the sequence's last page with id = -x-2
 *     (zipage/engine/model_runner.py:437-463);
 *   - a page id outside [0, num_pages) is treated as padding instead of being
 *     dereferenced.
 */
#ifndef ZIPAGE_HIP_H
#define ZIPAGE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { ZP_BF16 = 0, ZP_F16 = 1, ZP_F32 = 2 } zp_dtype;

enum { ZP_OK = 0, ZP_EINVAL = 1, ZP_EHIP = 2, ZP_EUNSUPPORTED = 3 };

enum { ZP_REDUCE_MEAN = 0, ZP_REDUCE_MAX = 1 };    /* attention_score `reduced` */
enum { ZP_ACTIVATE_MAX = 0, ZP_ACTIVATE_SUM = 1 }; /* global_score `activate_method` */
enum { ZP_POOL_MAX = 0, ZP_POOL_AVG = 1 };

/* ABI version of this header; bumped on any signature change. */
int zp_abi_version(void);
/* Message of the last error raised on the calling thread ("" if none). */
const char* zp_last_error(void);

/* store_query_cache(query, query_cache, slot_mapping)
 * zipage/kernel/store_query_cache.py:35-68 (kernel :7-32).
 * For each of the n int32 triples (pos, seq_id, slot):
 *   query_cache[seq_id, slot, :] = query[pos, :]   (row_elems = Hq*D elements). */
int zp_store_query(const void* query, void* query_cache, const int32_t* slot_mapping,
                   int32_t n, int32_t row_elems, int32_t num_tokens, int32_t max_seqs,
                   int32_t window, int64_t q_stride_tok, int64_t c_stride_seq,
                   int64_t c_stride_slot, int64_t sm_stride_row, int64_t sm_stride_col,
                   int32_t dtype, void* stream);

/* attention_score(k_cache, query_cache, seq_idx, block_table, softmax_scale, reduced,
 *                 return_logits)
 * zipage/kernel/attention_score.py:133-250 (kernel :8-130).
 * k_cache (L, num_pages, BS, Hkv, D), query_cache (L, max_seqs, W, Hq, D), both
 * contiguous in their last two axes; scores_out (L, B, Hkv, NB, BS) contiguous, in the
 * cache dtype; logits_out NULL or (L, B, Hq, W, NB, BS) contiguous.
 * workspace: zp_attention_score_workspace_for(..., dtype) bytes of device scratch
 * (zp_attention_score_workspace(): the upper bound over the dtypes).  With no logits_out, a
 * positive scale and at most 2560 tokens per sequence that scratch lets the library keep the
 * logits in registers and sweep K once (fp32 window partials per block of 32 query rows -- 16
 * for fp32 caches -- go through the scratch); with less scratch (NULL is fine up to 128 window x
 * group rows) the same entry point sweeps K three times (twice for fp32 caches).  The kernels
 * round at the same points and differ only in the fp32 order of the row sums (fp32 caches: also
 * in the last bit of the probabilities, e / sum against 2^(x log2 e - log2 sum)). */
int zp_attention_score(const void* k_cache, const void* query_cache, const int32_t* seq_idx,
                       const int32_t* block_table, void* scores_out, void* logits_out,
                       int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                       int32_t Hq, int32_t D, int32_t W, int32_t num_pages,
                       int32_t max_seqs, int64_t k_stride_layer, int64_t k_stride_page,
                       int64_t q_stride_layer, int64_t q_stride_seq, float softmax_scale,
                       int32_t reduced, int32_t dtype, void* workspace,
                       int64_t workspace_bytes, void* stream);
int64_t zp_attention_score_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                     int32_t Hkv, int32_t Hq, int32_t W);
int64_t zp_attention_score_workspace_for(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                         int32_t Hkv, int32_t Hq, int32_t W, int32_t dtype);

/* global_score(reduced_scores, score_cache, block_table, compressed, decay_factor,
 *              activate_method)
 * zipage/kernel/global_score.py:77-120 (kernel :8-74).
 * scores (L, B, Hkv, NB, BS) contiguous, updated in place; score_cache
 * (L, num_pages, BS, Hkv) with the given layer/page strides, slot stride Hkv, head
 * stride 1; compressed: B bytes (bool).
 * write_cache != 0 is the reference: every sequence's result is also stored to its pages of
 * the score cache (global_score.py:73-74).  When several sequences of the batch share a page
 * (prefix cache) those stores race, and compress_score would read back whichever landed last;
 * with write_cache == 0 the cache is only read, and zp_compress_score(scores_src = scores)
 * takes the carried values from `scores` instead, which is deterministic and equal to the
 * reference whenever no page is shared. */
int zp_global_score(void* scores, void* score_cache, const int32_t* block_table,
                    const uint8_t* compressed, int32_t L, int32_t B, int32_t NB,
                    int32_t BS, int32_t Hkv, int32_t num_pages, int64_t c_stride_layer,
                    int64_t c_stride_page, float decay_factor, int32_t activate_method,
                    int32_t write_cache, int32_t dtype, void* stream);

/* Sequence-axis pooling done inline by the runner:
 * zipage/engine/model_runner.py:499-530  (F.max_pool1d, stride 1, pad kernel//2, then
 * torch.where(compressed, raw, pooled) unless continues_pooling).
 * in/out (L, B, Hkv, T) contiguous, distinct buffers.  ZP_POOL_AVG is an extension
 * with no counterpart in the reference. */
int zp_pool_scores(const void* scores_in, void* scores_out, const uint8_t* compressed,
                   int32_t L, int32_t B, int32_t Hkv, int32_t T, int32_t kernel_size,
                   int32_t continues_pooling, int32_t mode, int32_t dtype, void* stream);

/* key_norm(key_cache, block_table, norm_epsilon)
 * zipage/kernel/key_norm.py:72-113 (kernel :8-69).  norm_out (L,B,Hkv,NB,BS). */
int zp_key_norm(const void* k_cache, const int32_t* block_table, void* norm_out, int32_t L,
                int32_t B, int32_t NB, int32_t BS, int32_t Hkv, int32_t D,
                int32_t num_pages, int64_t k_stride_layer, int64_t k_stride_page,
                float norm_epsilon, int32_t dtype, void* stream);

/* lightning_redudancy_score / raw_redudancy_score(key_cache, block_table, threshold,
 *                                                 temperature, return_logits)
 * zipage/kernel/lightning_redudancy_score.py:172-261 (kernel :10-169)
 * zipage/kernel/raw_redudancy_score.py:158-238 (kernel :10-155).
 * red_out (L,B,Hkv,NB,BS) softmax-normalised redundancy; logits_out NULL or the same
 * shape with the pre-softmax row sums (pad pages -inf). */
int zp_redundancy_lightning(const void* k_cache, const int32_t* block_table, void* red_out,
                            void* logits_out, int32_t L, int32_t B, int32_t NB, int32_t BS,
                            int32_t Hkv, int32_t D, int32_t num_pages,
                            int64_t k_stride_layer, int64_t k_stride_page, float threshold,
                            double temperature, int32_t dtype, void* stream);
int zp_redundancy_raw(const void* k_cache, const int32_t* block_table, void* red_out,
                      void* logits_out, int32_t L, int32_t B, int32_t NB, int32_t BS,
                      int32_t Hkv, int32_t D, int32_t num_pages, int64_t k_stride_layer,
                      int64_t k_stride_page, float threshold, double temperature,
                      int32_t dtype, void* workspace, int64_t workspace_bytes,
                      void* stream);
int64_t zp_redundancy_raw_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS,
                                    int32_t Hkv);

/* Score post-processing done inline by the runner, fused into one pass over
 * (L, B, Hkv, NB*BS), in place on `scores`:
 *   zipage/engine/model_runner.py:482-487  scores /= max_T            (max_norm_scores)
 *   zipage/engine/model_runner.py:551-559  red /= max_T (max_norm_red);
 *                                          scores*lambda - red*(1-lambda)  (red != NULL)
 *   zipage/engine/model_runner.py:565-578  first sink_len tokens -> +inf   (sink_len>0)
 *   zipage/kernel/window_mask.py:47-72     last `window` slots of the last page -> +inf
 *                                          (window > 0)
 *   zipage/engine/model_runner.py:592-593  pad pages -> -inf               (mask_pad)
 * Any subset can be selected; window_mask() alone is window>0 with everything else off.
 */
int zp_score_epilogue(void* scores, const void* redundancy, const int32_t* block_table,
                      int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                      int32_t max_norm_scores, int32_t max_norm_red, double redudancy_lambda,
                      int32_t sink_len, int32_t window, int32_t mask_pad, int32_t dtype,
                      void* stream);

/* topk_mask(scores, k)   zipage/kernel/utils.py:21-36.
 * scores (rows, T) contiguous; flag_out (rows, T) bytes, exactly min(k,T) ones per row.
 * Ties are broken towards the lowest index (torch.topk leaves them unspecified). */
int zp_topk_mask(const void* scores, uint8_t* flag_out, int32_t rows, int32_t T, int32_t k,
                 int32_t dtype, void* stream);

/* The selection stages of one layer chunk in one pass per score row (no counterpart as a
 * single function in the reference, which runs them inline in the runner):
 *   zipage/engine/model_runner.py:499-530  pooling (pool_kernel_size > 1; see zp_pool_scores)
 *   zipage/engine/model_runner.py:551-559  red /= max_T (max_norm_red);
 *                                          scores*lambda - red*(1-lambda)  (redundancy != NULL)
 *   zipage/engine/model_runner.py:565-578  first sink_len tokens -> +inf
 *   zipage/kernel/window_mask.py:47-72     last `window` slots of the last page -> +inf
 *   zipage/engine/model_runner.py:592-593  pad pages -> -inf               (mask_pad)
 *   zipage/engine/model_runner.py:594-600, zipage/kernel/utils.py:21-36    top-k keep flag
 * Results are bit-identical to zp_pool_scores + zp_score_epilogue + zp_topk_mask run one
 * after the other.  scores (L, B, Hkv, NB*BS) is read only unless scores_out == scores;
 * scores_out (same shape, may be NULL) receives the post-processed scores;
 * flag_out (L, B, Hkv, NB*BS) bytes, exactly k ones per row, ties to the lowest index. */
int zp_select_topk(const void* scores, void* scores_out, const void* redundancy,
                   uint8_t* flag_out, const int32_t* block_table, const uint8_t* compressed,
                   int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                   int32_t pool_kernel_size, int32_t continues_pooling, int32_t pool_mode,
                   int32_t max_norm_red, double redudancy_lambda, int32_t sink_len,
                   int32_t window, int32_t mask_pad, int32_t k, int32_t dtype, void* stream);

/* compress_kv(key, value, flag, block_table, target_block_table)
 * zipage/kernel/compress_kv.py:103-141 (kernel :8-100).
 * key/value (L, num_pages, BS, Hkv, D) with the given element strides (head_dim stride
 * 1); flag (L, B, Hkv, NB, BS) bytes contiguous; target (B, target_width) int32.
 * Stable in-place compaction.  A target page may be one of the sequence's own source pages
 * only if that source page sits at the same or a LATER position of block_table than the
 * position the page has in target_block_table (source index >= target index: survivors only
 * ever move towards the front), which is what BlockManager.may_compress produces
 * (zipage/engine/block_manager.py:129-169). */
int zp_compress_kv(void* key, void* value, const uint8_t* flag, const int32_t* block_table,
                   const int32_t* target_block_table, int32_t L, int32_t B, int32_t NB,
                   int32_t BS, int32_t Hkv, int32_t D, int32_t num_pages,
                   int32_t target_width, int64_t k_stride_layer, int64_t k_stride_page,
                   int64_t k_stride_slot, int64_t k_stride_head, int64_t v_stride_layer,
                   int64_t v_stride_page, int64_t v_stride_slot, int64_t v_stride_head,
                   int32_t dtype, void* stream);

/* compress_score(score_cache, flag, block_table, target_block_table)
 * zipage/kernel/compress_score.py:66-99 (kernel :8-63).
 * scores_src NULL: the reference (each kept token's value is read from its source page of the
 * score cache).  scores_src = the (L, B, Hkv, NB, BS) scores zp_global_score left: the value
 * of a kept token is read from there (see zp_global_score, write_cache). */
int zp_compress_score(void* score_cache, const void* scores_src, const uint8_t* flag,
                      const int32_t* block_table,
                      const int32_t* target_block_table, int32_t L, int32_t B, int32_t NB,
                      int32_t BS, int32_t Hkv, int32_t num_pages, int32_t target_width,
                      int64_t c_stride_layer, int64_t c_stride_page, int64_t c_stride_slot,
                      int64_t c_stride_head, int32_t dtype, void* stream);

/* ---- one layer chunk of the compression step as one call ----
 * The body of ModelRunner.compress for one chunk of layers
 * (zipage/engine/model_runner.py:466-622): attention_score -> [max-norm, global_score] ->
 * [redundancy] -> pooling / combine / sink / window mask / pad mask / top-k -> compress_kv ->
 * [compress_score], enqueued on `stream` in that order, so every result is bit-identical to
 * calling the entry points above one after the other (the carried scores of the survivors move
 * inside the compress_kv launch, by the same survivor list).  The switches are the fields of
 * zipage/config.py:22-46 that the runner reads. */
typedef struct {
  int32_t budget_blocks;          /* max_cache_blocks_per_seq: k = BS * budget_blocks survive */
  int32_t query_cache_len;        /* window W (also the window mask) */
  float softmax_scale;            /* <= 0: head_dim^-1/2 */
  int32_t reduced;                /* ZP_REDUCE_* */
  int32_t use_global_score;
  float decay_factor;
  int32_t activate_method;        /* ZP_ACTIVATE_* */
  int32_t max_norm;
  int32_t use_redundancy;
  int32_t lightning;              /* 1: per page, 0: all pairs */
  double redundancy_lambda;
  double redundancy_temperature;
  float redundancy_threshold;
  int32_t pooling_size;           /* <= 1: no pooling */
  int32_t continues_pooling;
  int32_t pooling_mode;           /* ZP_POOL_* */
  int32_t sink_len;               /* 0: no attention sink */
  int32_t deterministic_carry;    /* see zp_global_score: 1 = carried scores come from the
                                     scores, no shared page is written; 0 = the reference */
} zp_compress_config;

/* Stage names of the reference's timers (zipage/engine/model_runner.py:424-429,624-630);
 * ZP_STAGE_SELECT is pooling + window_mask + topk_mask as the one launch this library uses
 * when a row fits in LDS. */
enum {
  ZP_STAGE_ATTENTION_SCORE = 0, ZP_STAGE_GLOBAL_SCORE, ZP_STAGE_POOLING, ZP_STAGE_REDUNDANCY,
  ZP_STAGE_WINDOW_MASK, ZP_STAGE_TOPK_MASK, ZP_STAGE_SELECT, ZP_STAGE_COMPRESS_KV,
  ZP_STAGE_COMPRESS_SCORE, ZP_NUM_STAGES
};

/* Bytes of device workspace zp_compress_layers needs for these dims (scores, redundancy, the
 * stages' own scratch, and the keep flags when flag_in_workspace != 0); -1 on bad arguments. */
int64_t zp_compress_layers_workspace(int32_t L, int32_t B, int32_t NB, int32_t BS, int32_t Hkv,
                                     int32_t Hq, int32_t W, int32_t dtype,
                                     const zp_compress_config* cfg, int32_t flag_in_workspace);

/* k_cache / v_cache (L, num_pages, BS, Hkv, D), compacted in place; query_cache
 * (L, max_seqs, W, Hq, D); score_cache (L, num_pages, BS, Hkv) or NULL (required with
 * use_global_score), updated in place; seq_idx (B,) rows of the query cache; block_table
 * (B, NB); compressed (B,) bytes; target_block_table (B, target_width); flag_out NULL or
 * (L, B, Hkv, NB, BS) bytes receiving the keep flags.
 * strides: 14 int64 element strides: key layer, page, slot, head; value layer, page, slot,
 * head; query layer, sequence; score cache layer, page, slot, head (the last four ignored
 * without a score cache).  workspace: 256-byte aligned, zp_compress_layers_workspace() bytes;
 * its contents before the call do not matter and nothing in it is needed afterwards.
 * stage_events: NULL, or a HOST array of 2 * ZP_NUM_STAGES hipEvent_t (start, stop per stage,
 * NULL entries skipped) recorded on `stream` around the stages that run. */
int zp_compress_layers(void* k_cache, void* v_cache, const void* query_cache, void* score_cache,
                       const int32_t* seq_idx, const int32_t* block_table,
                       const uint8_t* compressed, const int32_t* target_block_table,
                       uint8_t* flag_out, int32_t L, int32_t B, int32_t NB, int32_t BS,
                       int32_t Hkv, int32_t Hq, int32_t D, int32_t W, int32_t num_pages,
                       int32_t max_seqs, int32_t target_width, const int64_t* strides,
                       int32_t dtype, const zp_compress_config* cfg, void* workspace,
                       int64_t workspace_bytes, void* const* stage_events, void* stream);

/* The same call for callers that cannot allocate device memory -- code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * The workspace is a fixed array of ZP_STATIC_SCRATCH_BYTES in device memory that the library
 * owns (one per GPU, held until the process ends), so the call takes no workspace and calls no
 * hipMalloc / hipFree or allocating routine; flag_out may be NULL (the flags then live in the
 * array too).  A chunk whose zp_compress_layers_workspace() exceeds the array is refused with
 * ZP_EINVAL: 32 MiB covers one layer of 256 sequences x 10 pages at 8 kv heads in a 16-bit
 * dtype with the lightning redundancy on.  The array is too small for the scorer's window
 * partials beyond ~90 such sequences per layer; larger chunks that still fit run the scorer's
 * three-sweep kernel (same rounding points, see zp_attention_score).  Every call on a GPU uses
 * that GPU's one array: calls that overlap in time on one GPU (two streams, two threads) race
 * and must be serialised by the caller.  Nothing in the array has to be cleared between calls.
 * zp_static_scratch_init() looks the array's address up for the current device (once per
 * device; the entry point does it on its first call otherwise): a caller that captures the
 * entry point into a HIP graph calls it beforehand, outside the capture. */
#define ZP_STATIC_SCRATCH_BYTES (32u << 20)
int zp_static_scratch_init(void);
int zp_compress_layers_static(void* k_cache, void* v_cache, const void* query_cache,
                              void* score_cache, const int32_t* seq_idx,
                              const int32_t* block_table, const uint8_t* compressed,
                              const int32_t* target_block_table, uint8_t* flag_out, int32_t L,
                              int32_t B, int32_t NB, int32_t BS, int32_t Hkv, int32_t Hq,
                              int32_t D, int32_t W, int32_t num_pages, int32_t max_seqs,
                              int32_t target_width, const int64_t* strides, int32_t dtype,
                              const zp_compress_config* cfg, void* stream);

/* ---- decode-step neighbours of the compression path (the callers either side of it) ---- */

/* store_kvcache(key, value, k_cache, v_cache, slot_mapping)
 * zipage/layers/attention.py:12-50 (kernel :12-30): token i of key/value (row_elems = Hkv*D
 * elements, row stride key_stride/value_stride elements) is copied to slot slot_mapping[i] of
 * the flat caches (num_slots x row_elems); a slot of -1 skips the token. */
int zp_store_kvcache(const void* key, const void* value, void* k_cache, void* v_cache,
                     const int32_t* slot_mapping, int32_t n, int32_t row_elems,
                     int64_t key_stride, int64_t value_stride, int64_t num_slots,
                     int32_t dtype, void* stream);

/* Single-query attention over a paged cache, the decode branch of Attention.forward:
 * zipage/layers/attention.py:95-103 (flash_attn_with_kvcache(q.unsqueeze(1), k_cache, v_cache,
 * cache_seqlens=context_lens, block_table=block_tables, softmax_scale, causal=True)).
 * q, out: (B, Hq, D); caches (num_pages, BS, Hkv, D) of one layer with page strides in
 * elements; block_tables (B, NB) plain page ids (-1 pad); context_lens (B,) tokens attended.
 * 16-bit caches, D <= 128, GQA group in {1,2,4,8}. */
int zp_paged_decode_attention(const void* q, const void* k_cache, const void* v_cache,
                              const int32_t* block_tables, const int32_t* context_lens,
                              void* out, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                              int32_t BS, int32_t NB, int32_t num_pages,
                              int64_t k_stride_page, int64_t v_stride_page,
                              float softmax_scale, int32_t dtype, void* stream);

/* ---- fused elementwise pieces of the decoder layer (between the GEMMs and the cache kernels).
 * The reference takes RMSNorm and SiluAndMul from its nanovllm dependency (imports at
 * zipage/models/qwen3.py:6-7) and applies per-head q/k norm, rotary embedding, store_kvcache and
 * store_query_cache as separate modules (zipage/models/qwen3.py:72-88,
 * zipage/layers/rotary_embedding.py:9-18, zipage/layers/attention.py:69-92). ---- */

/* out = rmsnorm(x [+ residual]) * weight; with a residual pointer the rounded sum is written
 * back to it (RMSNorm.forward(x, residual) of the dependency).  Strides in elements. */
int zp_add_rms_norm(const void* x, void* residual, const void* weight, void* out,
                    int32_t n, int32_t hidden, int64_t x_stride, int64_t r_stride,
                    int64_t out_stride, float eps, int32_t dtype, void* stream);

/* out = silu(gate_up[:, :I]) * gate_up[:, I:]  (SiluAndMul, zipage/models/qwen3.py:108-111). */
int zp_silu_and_mul(const void* gate_up, void* out, int32_t n, int32_t intermediate,
                    int64_t gu_stride, int64_t out_stride, int32_t dtype, void* stream);

/* For every token row of the fused qkv projection: q and k heads are RMS-normalised over the
 * head (weights q_norm_weight / k_norm_weight), rotated (NeoX halves, cos/sin tables of
 * (max_position, D/2) fp32 indexed by positions); q goes to q_out (n, Hq, D) and, when
 * query_triples[i] = (i, query row, ring slot) names the token, into the window ring; k and v go
 * to slot_mapping[i] of the flat caches (-1 skips); k_out (n, Hkv, D), when given, also receives
 * the rotated keys (prefill attention reads them).  k_out, query_cache, slot_mapping and
 * query_triples may be null. */
int zp_qk_norm_rope_store(const void* qkv, void* q_out, void* k_out, void* k_cache, void* v_cache,
                          void* query_cache, const void* q_norm_weight,
                          const void* k_norm_weight, const float* cos, const float* sin,
                          const int32_t* positions, const int32_t* slot_mapping,
                          const int32_t* query_triples, int32_t n, int32_t Hq,
                          int32_t Hkv, int32_t D, int32_t max_position,
                          int64_t qkv_stride, int64_t num_slots, int32_t max_seqs,
                          int32_t window, int64_t qc_stride_seq, int64_t qc_stride_slot,
                          float eps, int32_t dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ZIPAGE_HIP_H */
