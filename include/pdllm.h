/*
 * pdllm.h -- C ABI of the MI355X (gfx950) hot path of Prefilling-dLLM.
 *
 * Every entry point takes plain device pointers, sizes and strides, launches on
 * the given HIP stream and returns an int status (PDLLM_OK or a negative
 * PDLLM_ERR_* code).  Nothing here allocates, frees or synchronises; scratch
 * memory is a caller-provided workspace whose size a *_workspace_bytes query
 * returns.  No entry point throws across the boundary.
 *
 * Each declaration cites the reference interface it replaces.  Paths are
 * relative to prefilling_dllm_engine/prefilling_dllm/ of the reference:
 *   OPS = layers/attention/ops,  ENG = fastdllm_engine.py
 */
#ifndef PDLLM_H
#define PDLLM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pdllm_stream_t; /* a hipStream_t (0 = the null stream) */

enum {
  PDLLM_OK = 0,
  PDLLM_ERR_NULL = -1,        /* a required pointer is NULL                       */
  PDLLM_ERR_SHAPE = -2,       /* a size is negative / inconsistent / unsupported  */
  PDLLM_ERR_STRIDE = -3,      /* a stride or alignment the kernels rely on fails  */
  PDLLM_ERR_DTYPE = -4,       /* unknown dtype / mode enumerator                  */
  PDLLM_ERR_WORKSPACE = -5,   /* workspace missing or too small                   */
  PDLLM_ERR_LAUNCH = -6,      /* hipLaunch reported an error                      */
  PDLLM_ERR_UNSUPPORTED = -7, /* valid request the kernels do not cover           */
  PDLLM_ERR_SCRATCH_LIMIT = -8 /* input too large for the static device scratch of a *_static entry point */
};

enum { PDLLM_KV_BF16 = 0, PDLLM_KV_FP8_E4M3 = 1 };
/* visibility of the in-flight (active) keys; cached prefix keys are always visible */
enum { PDLLM_MASK_FULL = 0, PDLLM_MASK_CAUSAL = 1, PDLLM_MASK_DENSE = 2 };

const char* pdllm_status_string(int status);
/* version of this ABI; bumped when a struct layout changes */
int pdllm_abi_version(void);

/* ------------------------------------------------------------------------- *
 * Paged KV store                                                             *
 * ------------------------------------------------------------------------- */

/* Replaces store_kvcache_unified_layout + store_kvcache_kernel_diffusion_lm
 * (OPS/kv_cache_kernels.py:150-172, 34-55).
 * key/value: [n_tokens, Hkv*d] rows of row_elems 16-bit elements, row strides
 * key_stride / value_stride (elements).  k_cache/v_cache viewed as
 * [n_slots, row_elems].  slot_mapping[n_tokens] int32; slot < 0 = skip the
 * token; slot >= n_slots is skipped as well (never written out of bounds). */
int pdllm_kv_store(const void* key, const void* value, void* k_cache, void* v_cache,
                   const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                   int64_t key_stride, int64_t value_stride, int64_t n_slots,
                   pdllm_stream_t stream);

/* fp8 variant of the store (no reference counterpart beyond the scalar-scale
 * branch of OPS/prefix_prefill.py:118-121): quantises bf16 rows to e4m3 with
 * the scale of the destination page and KV head,
 *   x_q = e4m3(x / scale[page * scale_page_stride + head * scale_head_stride]),  head = element / head_dim,
 * the addressing pdllm_attn_desc uses to dequantise (scale_page_stride / scale_head_stride there): strides
 * (0, 0) = one scalar as the reference passes, (1, 0) = scale[n_pages], (Hkv, 1) = scale[n_pages, Hkv].
 * The scales are fp32, already filled by the caller, and cover every page a slot can name. */
int pdllm_kv_store_fp8(const void* key, const void* value, void* k_cache, void* v_cache,
                       const float* k_scale, const float* v_scale,
                       const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                       int64_t key_stride, int64_t value_stride, int64_t n_slots,
                       int32_t page_size, int32_t head_dim, int64_t scale_page_stride,
                       int64_t scale_head_stride, pdllm_stream_t stream);

/* Replaces the slot-mapping builders ENG:331-351, 434-441:
 * slot[i] = page_ids[(start_token+i) / page_size] * page_size + (start_token+i) % page_size.
 * page_ids: device int32 [n_page_ids]; tokens that fall beyond it get -1. */
int pdllm_slot_mapping(const int32_t* page_ids, int64_t n_page_ids, int64_t start_token,
                       int64_t n_tokens, int32_t page_size, int32_t* slots_out,
                       pdllm_stream_t stream);

/* Replaces load_kvcache + load_kvcache_kernel_kv (OPS/kv_cache_kernels.py:278-327,
 * 175-275): per sequence s, k_out[cu_k[s] + t] = cache[block_table[s][t/P]][t%P]
 * for t < ctx_len[s], followed by the sequence's active rows of k_new/v_new.
 * 16-bit elements; all row strides in elements. */
int pdllm_kv_load(const void* k_cache, const void* v_cache, const void* k_new, const void* v_new,
                  void* k_out, void* v_out, const int32_t* block_table, int64_t bt_stride,
                  const int32_t* ctx_lens, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                  int32_t n_seqs, int64_t max_total_len, int64_t row_elems, int32_t page_size,
                  int64_t n_pages, int64_t new_stride, int64_t out_stride, pdllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Attention over non-contiguous chunk KV pages + the active block            *
 * ------------------------------------------------------------------------- */

typedef struct pdllm_attn_desc {
  /* in-flight tensors, bf16, rows of head_dim contiguous elements */
  const void* q;      /* [n_tokens, Hq, d]   token stride q_stride (elements)  */
  const void* k_new;  /* [n_tokens, Hkv, d]  token stride kn_stride            */
  const void* v_new;  /* [n_tokens, Hkv, d]  token stride vn_stride            */
  void* out;          /* [n_tokens, Hq, d]   token stride o_stride             */
  /* paged cache, unified layout [n_pages, page_size, Hkv, d]; NULL = no prefix */
  const void* k_cache;
  const void* v_cache;
  const float* k_scale; /* fp8 only: scale[page*scale_page_stride + kvh*scale_head_stride] */
  const float* v_scale;
  const int32_t* block_table; /* [n_req, bt_stride] page ids.  An entry outside [0, n_pages) (the reference's -1)
                                 names no page: the keys of a visible range that fall on it are left out, as
                                 load_kvcache skips such entries (OPS/kv_cache_kernels.py:208).  (Only a request
                                 whose ranges touch more than 2048 pages has them clamped into the cache instead.) */
  const int32_t* q_start_loc; /* [n_req+1] first active row of each request     */
  /* visible prefix of request r = ranges range_ptr[r] .. range_ptr[r+1]-1, each a
   * run of logical tokens [range_start, range_start+range_len) that is mapped
   * through block_table[r][token / page_size]. */
  const int32_t* range_ptr;   /* [n_req+1] */
  const int32_t* range_start; /* [n_ranges] */
  const int32_t* range_len;   /* [n_ranges] */
  const uint8_t* mask; /* PDLLM_MASK_DENSE: bool[n_tokens, mask_stride], entry
                          (q_start+i, q_start+j) = row i of the request sees active key j */
  void* workspace;     /* split-KV partial results */
  int64_t workspace_bytes;
  int64_t q_stride, kn_stride, vn_stride, o_stride;           /* elements */
  int64_t cache_page_stride, cache_token_stride, cache_head_stride; /* elements of the cache dtype */
  int64_t mask_stride;
  int64_t n_tokens; /* rows of q/k_new/v_new/out                              */
  int64_t n_pages;
  int32_t bt_stride;
  int32_t scale_page_stride, scale_head_stride;
  int32_t n_req;
  int32_t max_q_len;   /* host upper bound of the per-request active length   */
  int32_t max_ctx_len; /* host upper bound of the per-request visible prefix; keys beyond it are not seen */
  int32_t max_ranges;  /* host upper bound of ranges per request (<= 128)     */
  int32_t num_q_heads, num_kv_heads, head_dim; /* head_dim must be 128        */
  int32_t page_size;   /* power of two                                        */
  int32_t kv_dtype;    /* PDLLM_KV_*  (dtype of the cache; in-flight K/V are bf16) */
  int32_t mask_mode;   /* PDLLM_MASK_*                                        */
  int32_t num_splits;  /* 0 = choose; 1..16 = cut every column into this many equal KV splits */
  int32_t rows_per_group; /* 0 = choose; else 32*J, J in {1,2,4,5,6,8} rows per workgroup (8: 512 threads) */
  float sm_scale;      /* softmax scale (1/sqrt(d) when the caller has no own) */
  /* optional: the slot table of the visible prefix, built by pdllm_attn_build_slot_table from
   * block_table and the ranges.  It only depends on those, so one table serves every layer of
   * a step.  NULL = pdllm_sparse_decode_attn builds it in the workspace on every call. */
  const int32_t* slot_table;
  int64_t slot_table_stride; /* int32 entries per request, >= pdllm_attn_slot_table_stride() */
  /* 0 = choose; >0 = every workgroup takes this many consecutive 64-key tiles of the line formed
   * by the tiles of all (request, KV head, row group) columns, so a workgroup may finish one column
   * and start the next; columns cut into pieces are merged from partial rows in the workspace (accumulated in
   * fp32, stored as fp16 with a power-of-two scale per 32 columns: 2^-12 .. 2^-11 of a block's largest element).
   * Overrides num_splits. */
  int32_t tiles_per_workgroup;
  /* optional, pdllm_sparse_decode_attn only: [n_tokens] cache slots (page * page_size + offset) of the active
   * rows.  When not NULL the call also performs store_kvcache_unified_layout of k_new / v_new
   * (attention_v4.py:328-331, OPS/kv_cache_kernels.py:150-172: slot < 0 or beyond the cache skips the row; fp8
   * pages are quantised with the page scales) -- the store and the attention of the reference's decode forward in
   * one call.  The cache must be the contiguous unified layout; the slots must not lie in the visible prefix of
   * this call (they are the block's own pages, behind it). */
  const int32_t* active_slot_mapping;
} pdllm_attn_desc;

/* Bytes of workspace pdllm_sparse_decode_attn needs for this descriptor: split-KV partials
 * and, when desc->slot_table is NULL, the slot table.  Negative = error code. */
int64_t pdllm_attn_workspace_bytes(const pdllm_attn_desc* desc);

/* Replaces the decode branch of Attention.forward (layers/attention/attention_v4.py:368-397),
 * i.e. load_kvcache + flex/SDPA attention (unified layout) or
 * diffusion_lm_parallel_flash_decoding = chunked_prefill_paged_decode ->
 * context_attention_fwd -> _fwd_kernel_d2f (OPS/chunked_prefill_decoding_unified_kernel.py:220-274,
 * OPS/prefix_prefill.py:25-230): out = softmax(Q K^T * sm_scale + mask) V over
 * [selected prefix pages || active block], GQA by head grouping, fp32 softmax
 * and accumulation.  Rows with no visible key produce zeros. */
int pdllm_sparse_decode_attn(const pdllm_attn_desc* desc, pdllm_stream_t stream);

/* Replaces the prefill branch of Attention.forward (attention_v4.py:336-367) for a
 * packed batch of independent chunks (block-diagonal mask, context.py:73-84):
 * per chunk c (rows cu_seqlens[c]..cu_seqlens[c+1]) causal or full
 * self-attention, and (when slot_mapping != NULL) the paged store of K/V of
 * OPS/kv_cache_kernels.py:150-172 for the same rows.  Uses the descriptor's
 * in-flight tensors, q_start_loc (= cu_seqlens), mask_mode and cache fields. */
int pdllm_chunk_prefill_attn(const pdllm_attn_desc* desc, const int32_t* slot_mapping,
                             pdllm_stream_t stream);

/* Replaces the per-forward context arrays of the reference (slot_mapping / block_tables of
 * ContextForDiffusionLM, utils/context.py:58-67, built once per step for all layers; slot
 * formula ENG:331-337): table[r*table_stride + v] = page*page_size + offset of the v-th visible
 * prefix key of request r (the ranges in order, through block_table[r]); entries up to the next
 * multiple of 64 repeat a valid slot; table[r*table_stride + table_stride-1] = number of
 * visible keys = min(sum of range lengths, max_ctx_len).  Uses block_table, bt_stride, range_*,
 * max_ranges, n_req, max_ctx_len, page_size and n_pages of the descriptor. */
int64_t pdllm_attn_slot_table_stride(const pdllm_attn_desc* desc);
int pdllm_attn_build_slot_table(const pdllm_attn_desc* desc, int32_t* table, int64_t table_stride,
                                pdllm_stream_t stream);

/* The plan pdllm_sparse_decode_attn (prefill == 0) or pdllm_chunk_prefill_attn would use:
 * rows per workgroup (32 * row blocks) and number of KV splits.  For tuning and tests. */
int pdllm_attn_plan(const pdllm_attn_desc* desc, int32_t prefill, int32_t* rows_per_group,
                    int32_t* num_splits);

/* The same plan as one line of text ("<kernel> kv=<dtype> row_blocks=J grid=.. span=.. head=.. set=.. tiles=..
 * pieces=.. partial_row_bytes=.."): which kernel runs, how the tiles of the launch are cut over workgroups and how
 * many bytes a partial row of a cut column takes in the workspace.  No counterpart in the
 * reference; it identifies a launch configuration so that measurements (profiles, counters) can be matched to the
 * configuration they were taken on.  text receives at most text_bytes bytes including the terminating 0. */
int pdllm_attn_plan_describe(const pdllm_attn_desc* desc, int32_t prefill, char* text, int32_t text_bytes);

/* ------------------------------------------------------------------------- *
 * Chunk scoring and selection                                                *
 * ------------------------------------------------------------------------- */

/* Replaces F.log_softmax(...).gather(...) of score_chunk_self_information_engine
 * (ENG:1148-1152) for a batch of rows: logp[r] = logits[r, label[r]] - logsumexp(logits[r,:])
 * in fp32 over bf16 logits [n_rows, vocab] (row stride logits_stride elements).
 * A label outside [0, vocab) yields -inf. */
int pdllm_selfinfo_logprob(const void* logits, int64_t logits_stride, const int64_t* labels,
                           int64_t n_rows, int64_t vocab, void* workspace, int64_t workspace_bytes,
                           float* logp_out, pdllm_stream_t stream);

/* Bytes of workspace the two vocabulary scans (pdllm_selfinfo_logprob, pdllm_conf_argmax)
 * need for n_rows rows of `vocab` logits: per-row, per-split (max, sum, argmax) partials. */
int64_t pdllm_vocab_workspace_bytes(int64_t n_rows, int64_t vocab);

/* score[c] = (mean ? 1/rows_per_chunk : 1) * sum_j logp[c*rows_per_chunk + j], summed in
 * index order in fp32 (ENG:1152 takes the mean). */
int pdllm_chunk_score_reduce(const float* logp, int64_t n_chunks, int64_t rows_per_chunk,
                             int32_t mean, float* scores_out, pdllm_stream_t stream);

/* score_chunk_self_information_engine + the ranking of select_chunks_by_engine in one call
 * (ENG:1148-1152 and 1199-1204; the reference runs them back to back for every draft round):
 * pdllm_selfinfo_logprob over [n_chunks * rows_per_chunk, vocab] logits, pdllm_chunk_score_reduce
 * and pdllm_topk_lowest_index of the n_chunks scores, as two launches; same results as the three
 * calls.  logp_out may be NULL.  n_chunks <= 1024, 1 <= k <= n_chunks; workspace as
 * pdllm_vocab_workspace_bytes(n_chunks * rows_per_chunk, vocab). */
int pdllm_chunk_select(const void* logits, int64_t logits_stride, const int64_t* labels,
                       int64_t n_chunks, int64_t rows_per_chunk, int64_t vocab, int32_t mean, int64_t k,
                       int32_t sorted_ascending, void* workspace, int64_t workspace_bytes,
                       float* logp_out, float* scores_out, int64_t* indices_out, pdllm_stream_t stream);

/* Replaces the ranking of select_chunks_by_engine (ENG:1199-1204): per row of
 * scores [n_rows, n] (non-finite -> -inf), the k best indices by (score desc,
 * index asc), returned ascending when sorted_ascending != 0, else in rank order.
 * n <= 65536, k <= n; rank order only for n <= 2048 (PDLLM_ERR_UNSUPPORTED beyond: the
 * reference ranks chunks, of which there are at most a few hundred). */
int pdllm_topk_lowest_index(const float* scores, int64_t n_rows, int64_t n, int64_t scores_stride,
                            int64_t k, int32_t sorted_ascending, int64_t* indices_out,
                            pdllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Intra-chunk token eviction                                                 *
 * ------------------------------------------------------------------------- */

/* Column sums of ready-made attention probabilities: probs [n_chunks, n_heads,
 * n_queries, n_keys] fp32 contiguous -> scores [n_chunks, n_groups, n_keys] with
 * heads_per_group consecutive heads summed (n_groups = n_heads / heads_per_group;
 * heads_per_group = n_heads gives the global score of
 * prefilling_dllm_eval/fastdllm_parallelcomp.py:1607-1637).  The sum runs over
 * (head, query) in index order, so it is reproducible bit for bit.  workspace may be NULL; with
 * pdllm_evict_colsum_workspace_bytes() bytes of it, few chunks are summed by one workgroup per
 * (chunk, head, column range) in two launches (same bits, better use of the memory system). */
int64_t pdllm_evict_colsum_workspace_bytes(int64_t n_chunks, int64_t n_heads, int64_t n_keys);
int pdllm_evict_colsum(const float* probs, int64_t n_chunks, int64_t n_heads, int64_t n_queries,
                       int64_t n_keys, int64_t heads_per_group, void* workspace,
                       int64_t workspace_bytes, float* scores_out, pdllm_stream_t stream);

/* One eviction step from ready-made probabilities in one call: pdllm_evict_colsum followed by
 * pdllm_topb_keep_bos on its scores (fastdllm_engine.py:1230-1322 summed over queries and heads, then :903-927),
 * same scores and same indices bit for bit.  scores_out [n_chunks, n_groups, n_keys] fp32, indices_out
 * [n_chunks * n_groups, keep] int64 ascending with keep = min(max(capacity, 1), n_keys).  With a workspace of
 * pdllm_evict_colsum_workspace_bytes() bytes, few chunks and n_keys <= 2048 the step is two launches (per-head
 * column sums; then the sum over the heads of a group and the selection, one workgroup per row); otherwise it is
 * the launches of the two calls. */
int pdllm_evict_keep_from_probs(const float* probs, int64_t n_chunks, int64_t n_heads, int64_t n_queries,
                                int64_t n_keys, int64_t heads_per_group, int64_t capacity, int32_t keep_high,
                                int32_t force_keep_first, void* workspace, int64_t workspace_bytes,
                                float* scores_out, int64_t* indices_out, pdllm_stream_t stream);

/* Replaces query_to_chunk_attention_scores (OPS/triton_eviction_scorer.py:114-210) and
 * the torch path of _engine_chunk_attention_head_scores (ENG:1279-1310): q [S, Hq, d],
 * k [S, Hkv, d] bf16 contiguous, S = prefix_len + chunk_len + query_len; for every
 * q-head, softmax over the visible keys of the last query_len rows, summed (or averaged)
 * over those rows on the chunk columns -> out [Hq, chunk_len] fp32.
 * causal != 0: key j visible to row i iff j <= i.  workspace: pdllm_evict_score_qk_workspace_bytes() bytes
 * (per-row softmax statistics of the key segments; fp32).  head_dim 128 runs on the matrix cores (QK^T in
 * bf16 with fp32 accumulation, as the reference's tl.dot), other head dims up to 256 on the vector unit. */
int64_t pdllm_evict_score_qk_workspace_bytes(int64_t prefix_len, int64_t chunk_len, int64_t query_len,
                                             int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim);
int pdllm_evict_score_qk(const void* q, const void* k, int64_t prefix_len, int64_t chunk_len,
                         int64_t query_len, int32_t num_q_heads, int32_t num_kv_heads,
                         int32_t head_dim, float scale, int32_t reduce_mean, int32_t causal,
                         float* workspace, int64_t workspace_bytes, float* out, pdllm_stream_t stream);

/* Replaces the pooling + per-KV-head grouping of ENG:1405-1433: optional max/avg pool
 * (kernel, padding kernel/2, stride 1, as F.max_pool1d / F.avg_pool1d with
 * count_include_pad) over [n_heads, n] rows then the mean of each group of
 * heads_per_group rows -> [n_heads/heads_per_group, n].  pool: 0 none, 1 max, 2 avg. */
int pdllm_token_score_pool_group(const float* scores, int64_t n_heads, int64_t n, int32_t pool,
                                 int32_t kernel, int64_t heads_per_group, float* out,
                                 pdllm_stream_t stream);

/* Replaces _select_positions_from_token_scores (ENG:903-927): per row of scores
 * [n_rows, chunk_len]: keep position 0 (BOS) and the keep_count-1 best of positions
 * 1..chunk_len-1 by (score desc, index asc); indices_out [n_rows, keep_count] ascending.
 * keep_count = min(max(1, capacity), chunk_len).  keep_high == 0 ranks by (score asc,
 * index asc).  force_keep_first == 0 ranks all positions. */
int pdllm_topb_keep_bos(const float* scores, int64_t n_rows, int64_t chunk_len,
                        int64_t scores_stride, int64_t capacity, int32_t keep_high,
                        int32_t force_keep_first, int64_t* indices_out, pdllm_stream_t stream);

/* Vote counting of the pre-eviction script (scripts/run_dream_longbench_task_fastdllm_engine_full_
 * bridge_preevict_votetopk.sh:231-239): votes[t] += 1 for every entry t of indices [n] inside
 * [0, length); indices outside are ignored.  votes [length] fp32 must be zeroed by the caller (counts
 * are exact below 2^24); pdllm_topb_keep_bos over the votes of a chunk then gives the script's
 * (-votes, index) order with the chunk's first token forced. */
int pdllm_vote_histogram(const int64_t* indices, int64_t n, int64_t length, float* votes,
                         pdllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * KV compaction / snapshot                                                   *
 * ------------------------------------------------------------------------- */

/* Replaces _snapshot_prompt_cache_per_layer / the gather half of
 * _compact_prompt_cache_per_layer_per_head and _copy_chunk_local_kv_to_prompt_pages
 * (ENG:640-662, 607-638, 525-558).  For token j < n_tokens and head h:
 *   t = token_idx ? token_idx[h*idx_head_stride + j] + src_offset : j + src_offset
 *   dst[j, h, :] = cache[page_ids[t / P], t % P, h, :]
 * dst: dense [n_tokens, Hkv, d].  elem_bytes = bytes of one element (2 or 1). */
int pdllm_kv_gather(const void* cache, const int32_t* page_ids, int64_t n_page_ids,
                    const int64_t* token_idx, int64_t idx_head_stride, int64_t src_offset,
                    int64_t n_tokens, int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                    int64_t n_pages, int32_t elem_bytes, void* dst, pdllm_stream_t stream);

/* Replaces _load_prompt_cache_per_layer / the scatter half of the functions above
 * (ENG:664-698): cache[page_ids[(dst_start+j)/P], (dst_start+j)%P, h, :] = src[j, h, :]. */
int pdllm_kv_scatter(void* cache, const int32_t* page_ids, int64_t n_page_ids, int64_t dst_start,
                     int64_t n_tokens, int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                     int64_t n_pages, int32_t elem_bytes, const void* src, pdllm_stream_t stream);

/* Replaces _compact_prompt_cache_per_layer_per_head (ENG:607-638) for all layers at once: on the unified cache
 * kv_cache [2, n_layers, n_pages, page_size, Hkv, d] (plane stride in bytes), token j of KV head h of layer l becomes
 * token keep[l*keep_layer_stride + h*keep_head_stride + j] of the request's pages (page_ids), j < n_keep, for K and V.
 * The kept rows of a round of layers are gathered into the workspace before the first one is overwritten (the
 * reference clones), two launches per round; the workspace holds at least one layer
 * (pdllm_kv_compact_per_head_workspace_bytes) and as many layers per round as fit. */
int64_t pdllm_kv_compact_per_head_workspace_bytes(int64_t n_keep, int32_t num_kv_heads, int32_t head_dim,
                                                  int32_t elem_bytes);
int pdllm_kv_compact_per_head(void* kv_cache, int64_t plane_stride_bytes, int32_t n_layers,
                              const int32_t* page_ids, int64_t n_page_ids, const int64_t* keep,
                              int64_t keep_layer_stride, int64_t keep_head_stride, int64_t n_keep,
                              int32_t num_kv_heads, int32_t head_dim, int32_t page_size, int64_t n_pages,
                              int32_t elem_bytes, void* workspace, int64_t workspace_bytes, pdllm_stream_t stream);

/* Replaces the per-layer advanced-indexing copies of make_pd_record_from_remote_engine
 * (ENG:845-859) for two unified caches [planes, n_pages, page_size, Hkv, d] (plane = K/V x layer)
 * of the same page geometry: dst[plane][dst_page_ids[i]] = src[plane][src_page_ids[i]] for all
 * planes in one launch, page-granular (the tokens of a last, partly filled page travel with their
 * page).  Strides and page_bytes in bytes, multiples of 16; page ids outside a cache are skipped. */
int pdllm_kv_copy_pages(const void* src_cache, void* dst_cache, const int32_t* src_page_ids,
                        const int32_t* dst_page_ids, int64_t n_copy, int64_t page_bytes, int64_t n_planes,
                        int64_t src_plane_stride_bytes, int64_t dst_plane_stride_bytes,
                        int64_t src_n_pages, int64_t dst_n_pages, pdllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Confidence-threshold unmasking                                             *
 * ------------------------------------------------------------------------- */

/* Replaces _shift_logits + _sample_tokens at temperature 0 (ENG:1647-1681) for
 * n_seqs blocks of block_len rows of bf16 logits [n_seqs*block_len, vocab]:
 * row i of block b reads logits row (b*block_len + i - shift) where shift = 1 uses
 * last_logit[b] (or the block's own row 0 when last_logit == NULL) for i = 0;
 * confidence = max softmax probability in fp32, token = first index of the maximum.
 * Accuracy: the token is exact (integer comparison of the bf16 logits, first index on ties).  The confidence is
 * 1 / sum_j exp(x_j - max) with the sum taken in fp32 over fixed per-lane and per-split partial sums, an order
 * that differs from torch.softmax's; the two agree to within 5e-5 absolute (the bound the parity tests hold, on
 * vocabularies up to 152064).  Everything that compares the confidence with a threshold (pdllm_threshold_unmask,
 * pdllm_denoise_unmask*) therefore decides exactly as the reference whenever the reference's confidence is
 * further than 5e-5 from the threshold; inside that band either decision can come out.  The most confident
 * position of a block is always transferred, so a block never stalls on such a tie.
 * Limit: n_seqs * block_len <= 65535 rows per call (one grid dimension of the scan); more returns
 * PDLLM_ERR_UNSUPPORTED, here and in pdllm_denoise_unmask and pdllm_denoise_unmask_static (where an input
 * of that size also exceeds the static scratch area, whichever check comes first). */
int pdllm_conf_argmax(const void* logits, int64_t logits_stride, const void* last_logit,
                      int64_t last_logit_stride, int64_t n_seqs, int64_t block_len, int64_t vocab,
                      int32_t shift, void* workspace, int64_t workspace_bytes, float* conf_out,
                      int64_t* token_out, pdllm_stream_t stream);

/* Replaces the transfer rule of decode_from_pd_record (ENG:2146-2157) without host
 * syncs: per block b over the positions with block_ids == mask_token_id, transfer the
 * most confident one (lowest index on ties) and every one with conf >= threshold;
 * writes the tokens into block_ids in place, transfer_out[b, i] in {0,1} and
 * n_masked_left[b] = masked positions remaining after the update. */
int pdllm_threshold_unmask(const float* conf, const int64_t* token, int64_t* block_ids,
                           int64_t n_seqs, int64_t block_len, int64_t mask_token_id,
                           float threshold, uint8_t* transfer_out, int32_t* n_masked_left,
                           pdllm_stream_t stream);

/* One denoise step's sampling and transfer (ENG:1647-1681 followed by 2146-2157) in one call:
 * pdllm_conf_argmax and pdllm_threshold_unmask as two launches, same results; conf_out and
 * token_out [n_seqs * block_len] are written as by pdllm_conf_argmax. */
int pdllm_denoise_unmask(const void* logits, int64_t logits_stride, const void* last_logit,
                         int64_t last_logit_stride, int64_t n_seqs, int64_t block_len, int64_t vocab,
                         int32_t shift, int64_t* block_ids, int64_t mask_token_id, float threshold,
                         void* workspace, int64_t workspace_bytes, float* conf_out, int64_t* token_out,
                         uint8_t* transfer_out, int32_t* n_masked_left, pdllm_stream_t stream);

/* pdllm_denoise_unmask for callers that cannot allocate a workspace or have one allocated for them (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  Same arguments and results as pdllm_denoise_unmask without the workspace: the partial
 * results of the vocabulary scan live in a static device array of PDLLM_STATIC_SCRATCH_BYTES that every GPU
 * the library runs on holds until the process ends.  The call allocates and frees nothing.  An input whose
 * partials do not fit, pdllm_vocab_workspace_bytes(n_seqs * block_len, vocab) > PDLLM_STATIC_SCRATCH_BYTES,
 * is refused with PDLLM_ERR_SCRATCH_LIMIT (16384 (row, split) partials of 16 bytes fit: up to 16384 rows, i.e. 512
 * sequences of 32 positions, of any vocabulary).
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams or threads)
 * race; calls on one stream do not.  The first call on a device looks the array's address up; make it
 * outside a stream capture. */
#define PDLLM_STATIC_SCRATCH_BYTES (256 * 1024)
int pdllm_denoise_unmask_static(const void* logits, int64_t logits_stride, const void* last_logit,
                                int64_t last_logit_stride, int64_t n_seqs, int64_t block_len, int64_t vocab,
                                int32_t shift, int64_t* block_ids, int64_t mask_token_id, float threshold,
                                float* conf_out, int64_t* token_out, uint8_t* transfer_out,
                                int32_t* n_masked_left, pdllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Rotary embedding (the step in front of the path)                           *
 * ------------------------------------------------------------------------- */

/* Replaces RotaryEmbedding.forward / apply_rotary_emb (layers/rotary_embedding.py:6-17,
 * 39-65): neox split-half rotation in fp32 with cos_sin_cache[positions] =
 * [cos(d/2) | sin(d/2)] fp32 rows, applied in place to x [n_tokens, n_heads, d] bf16. */
int pdllm_rope_inplace(void* x, int64_t x_stride, const int64_t* positions,
                       const float* cos_sin_cache, int64_t max_positions, int64_t n_tokens,
                       int32_t n_heads, int32_t head_dim, pdllm_stream_t stream);

/* RotaryEmbedding.forward on Q and K (layers/rotary_embedding.py:39-65) and the paged store of the
 * rotated K and of V (OPS/kv_cache_kernels.py:150-172) in one launch, the order the reference's
 * attention layer runs them in (rotary, then Attention.forward stores K/V, attention_v4.py:316-335).
 * q [n_tokens, num_q_heads, d] and k [n_tokens, num_kv_heads, d] bf16 are rotated in place; with
 * slot_mapping != NULL, cache row slot_mapping[t] of the unified bf16 caches receives the rotated K
 * and V of token t (slots < 0 or >= n_slots: not stored).  Same bits as pdllm_rope_inplace on q and
 * k followed by pdllm_kv_store.  head_dim % 16 == 0, strides in elements and multiples of 8. */
int pdllm_rope_qk_store(void* q, int64_t q_stride, int32_t num_q_heads, void* k, int64_t k_stride,
                        const void* v, int64_t v_stride, int32_t num_kv_heads, int32_t head_dim,
                        const int64_t* positions, const float* cos_sin_cache, int64_t max_positions,
                        int64_t n_tokens, void* k_cache, void* v_cache, const int32_t* slot_mapping,
                        int64_t n_slots, pdllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Anchor corrections of the attention output (experimental, default off)     *
 * ------------------------------------------------------------------------- */

enum { PDLLM_ANCHOR_LEFT = 0, PDLLM_ANCHOR_RIGHT = 1, PDLLM_ANCHOR_BOTH = 2 };
enum { PDLLM_ANCHOR_SEL_NONE = 0, PDLLM_ANCHOR_SEL_REPLACE = 1, PDLLM_ANCHOR_SEL_ADD = 2 };

/* Replaces the delta / correction loops of Attention._maybe_apply_decode_delta
 * (layers/attention/attention_v4.py:139-166) and Attention._maybe_prefill_sparse_attention
 * (attention_v4.py:263-293).  Per sequence [q_start_loc[r], q_start_loc[r+1]) of the packed rows the
 * anchors are the local rows anchor_offset, anchor_offset + stride, ...; anchor a spreads
 *   delta[a] = (dense[a] - base[a]) * scale                                           (SEL_NONE)
 *   delta[a] = (sel[a] - base[a]) * scale * valid[a]                                  (SEL_REPLACE)
 *   delta[a] = (dense[a] - base[a]) * scale + (sel[a] - dense[a]) * sel_scale * valid[a]   (SEL_ADD)
 * over the rows [a - left, a] (LEFT), [a, a + right] (RIGHT) or [a - left, a + right] (BOTH), clipped
 * to the sequence, and out[r] = base[r] + sum of the deltas that reach r, anchors ascending.  Every
 * difference, product and sum is rounded to bf16 like the reference's bf16 tensor operations.
 * base, dense, out: bf16 [n_rows, row_elems] (row strides in elements); only the anchor rows of dense
 * are read.  sel: bf16 [n_sel_rows, row_elems] indexed by the local anchor row (rows >= n_sel_rows read
 * as zero and are not valid), valid[a] = sel_counts == NULL || sel_counts[a] > 0; selection modes take
 * one sequence (n_req == 1).  out must not alias base or dense.  row_elems % 8 == 0.  n_rows = rows of base,
 * dense and out: a sequence that does not lie inside them is skipped. */
int pdllm_anchor_delta_add(const void* base, int64_t base_stride, const void* dense, int64_t dense_stride,
                           const void* sel, int64_t sel_stride, int64_t n_sel_rows, const int64_t* sel_counts,
                           void* out, int64_t out_stride, const int32_t* q_start_loc, int64_t n_req,
                           int64_t max_q_len, int64_t n_rows, int64_t row_elems, int32_t stride, int32_t anchor_offset,
                           int32_t left, int32_t right, int32_t direction, float scale, float sel_scale,
                           int32_t sel_mode, pdllm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PDLLM_H */
