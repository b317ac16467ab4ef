// Paged KV cache data movement for gfx950: slot-mapped store (bf16 and fp8), slot-mapping
// construction, dense load (page-table gather + active rows), per-head token gather and
// page scatter.  All of it is HBM-bound byte movement: every lane moves 16 bytes, the lanes
// of a wave cover consecutive bytes of one row, rows are independent.
//
// Reference: layers/attention/ops/kv_cache_kernels.py:34-55,150-327 and
// fastdllm_engine.py:331-351,434-441,525-558,607-698 of the reference engine.

#include "pdllm_common.h"

namespace pdllm {

// ---------------------------------------------------------------------------------------
// store: cache[slot[t], :] = key[t, :]   (slot < 0 or >= n_slots: token skipped)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void kv_store_kernel(const uint4* __restrict__ key,
                                                       const uint4* __restrict__ value,
                                                       uint4* __restrict__ k_cache,
                                                       uint4* __restrict__ v_cache,
                                                       const int* __restrict__ slot_mapping,
                                                       long n_tokens, int chunks_per_row,
                                                       long key_stride16, long value_stride16,
                                                       long n_slots) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long tok = idx / chunks_per_row;
  const int ch = (int)(idx - tok * chunks_per_row);
  if (tok >= n_tokens) return;
  const long slot = slot_mapping[tok];
  if (slot < 0 || slot >= n_slots) return;
  const uint4 kv = key[tok * key_stride16 + ch];
  const uint4 vv = value[tok * value_stride16 + ch];
  k_cache[slot * chunks_per_row + ch] = kv;
  v_cache[slot * chunks_per_row + ch] = vv;
}

__device__ __forceinline__ float clamp448(float x) {
  // e4m3 has no infinity: saturate at the largest finite value
  return fminf(fmaxf(x, -448.f), 448.f);
}

// 8 bf16 -> 8 e4m3 of x / scale
__device__ __forceinline__ uint2 quant_fp8x8(uint4 raw, float scale) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float f[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = clamp448(bf16_bits_to_f32(w[i] & 0xffffu) / scale);
    f[2 * i + 1] = clamp448(bf16_bits_to_f32(w[i] >> 16) / scale);
  }
  uint2 r;
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
  r.x = (uint32_t)lo;
  r.y = (uint32_t)hi;
  return r;
}

__global__ __launch_bounds__(256) void kv_store_fp8_kernel(
    const uint4* __restrict__ key, const uint4* __restrict__ value, uint2* __restrict__ k_cache,
    uint2* __restrict__ v_cache, const float* __restrict__ k_scale, const float* __restrict__ v_scale,
    const int* __restrict__ slot_mapping, long n_tokens, int chunks_per_row, long key_stride16,
    long value_stride16, long n_slots, int page_shift, int chunks_per_head, long scale_page_stride,
    long scale_head_stride) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long tok = idx / chunks_per_row;
  const int ch = (int)(idx - tok * chunks_per_row);
  if (tok >= n_tokens) return;
  const long slot = slot_mapping[tok];
  if (slot < 0 || slot >= n_slots) return;
  // the scale of (page, KV head), addressed like the attention kernel addresses it when it dequantises
  const long so = (slot >> page_shift) * scale_page_stride + (long)(ch / chunks_per_head) * scale_head_stride;
  const uint4 kv = key[tok * key_stride16 + ch];
  const uint4 vv = value[tok * value_stride16 + ch];
  k_cache[slot * chunks_per_row + ch] = quant_fp8x8(kv, k_scale[so]);
  v_cache[slot * chunks_per_row + ch] = quant_fp8x8(vv, v_scale[so]);
}

__global__ __launch_bounds__(256) void slot_mapping_kernel(const int* __restrict__ page_ids,
                                                           long n_page_ids, long start_token,
                                                           long n_tokens, int page_shift,
                                                           int* __restrict__ slots) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_tokens) return;
  const long t = start_token + i;
  const long pi = t >> page_shift;
  int res = -1;
  if (t >= 0 && pi < n_page_ids) {
    const int page = page_ids[pi];
    if (page >= 0) res = (page << page_shift) + (int)(t & ((1L << page_shift) - 1));
  }
  slots[i] = res;
}

// ---------------------------------------------------------------------------------------
// dense load: out[cu_k[s] + t] = t < ctx ? cache[bt[s][t/P]][t%P] : new[cu_q[s] + t - ctx]
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void kv_load_kernel(
    const uint4* __restrict__ k_cache, const uint4* __restrict__ v_cache,
    const uint4* __restrict__ k_new, const uint4* __restrict__ v_new, uint4* __restrict__ k_out,
    uint4* __restrict__ v_out, const int* __restrict__ block_table, long bt_stride,
    const int* __restrict__ ctx_lens, const int* __restrict__ cu_q, const int* __restrict__ cu_k,
    int chunks_per_row, int page_shift, long n_pages, long new_stride16, long out_stride16) {
  const int seq = blockIdx.y;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long t = idx / chunks_per_row;
  const int ch = (int)(idx - t * chunks_per_row);
  const int ctx = ctx_lens[seq];
  const int q0 = cu_q[seq];
  const int active = cu_q[seq + 1] - q0;
  if (ctx < 0 || active < 0 || t >= (long)ctx + active) return;
  const long orow = (long)cu_k[seq] + t;
  uint4 kv = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
  if (t < ctx) {
    const long pi = t >> page_shift;
    if (pi < bt_stride) {
      const long page = block_table[(long)seq * bt_stride + pi];
      if (page >= 0 && page < n_pages) {
        const long slot = (page << page_shift) + (t & ((1L << page_shift) - 1));
        kv = k_cache[slot * chunks_per_row + ch];
        vv = v_cache[slot * chunks_per_row + ch];
      }
    }
  } else {
    const long nrow = (long)q0 + (t - ctx);
    kv = k_new[nrow * new_stride16 + ch];
    vv = v_new[nrow * new_stride16 + ch];
  }
  k_out[orow * out_stride16 + ch] = kv;
  v_out[orow * out_stride16 + ch] = vv;
}

// ---------------------------------------------------------------------------------------
// gather / scatter of [token, head, :] rows between pages and a dense tensor
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void kv_gather_kernel(
    const uint4* __restrict__ cache, const int* __restrict__ page_ids, long n_page_ids,
    const long* __restrict__ token_idx, long idx_head_stride, long src_offset, long n_tokens,
    int n_heads, int chunks_per_head, int page_shift, long n_pages, uint4* __restrict__ dst) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long per_tok = (long)n_heads * chunks_per_head;
  const long j = idx / per_tok;
  if (j >= n_tokens) return;
  const int rem = (int)(idx - j * per_tok);
  const int head = rem / chunks_per_head;
  const long t = (token_idx ? token_idx[(long)head * idx_head_stride + j] : j) + src_offset;
  uint4 v = {0u, 0u, 0u, 0u};
  const long pi = t >> page_shift;
  if (t >= 0 && pi < n_page_ids) {
    const long page = page_ids[pi];
    if (page >= 0 && page < n_pages) {
      const long slot = (page << page_shift) + (t & ((1L << page_shift) - 1));
      v = cache[slot * per_tok + rem];
    }
  }
  dst[idx] = v;
}

__global__ __launch_bounds__(256) void kv_scatter_kernel(
    uint4* __restrict__ cache, const int* __restrict__ page_ids, long n_page_ids, long dst_start,
    long n_tokens, long per_tok, int page_shift, long n_pages, const uint4* __restrict__ src) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long j = idx / per_tok;
  if (j >= n_tokens) return;
  const int rem = (int)(idx - j * per_tok);
  const long t = dst_start + j;
  const long pi = t >> page_shift;
  if (t < 0 || pi >= n_page_ids) return;
  const long page = page_ids[pi];
  if (page < 0 || page >= n_pages) return;
  const long slot = (page << page_shift) + (t & ((1L << page_shift) - 1));
  cache[slot * per_tok + rem] = src[idx];
}

// Per-head compaction of the prompt rows of several planes (K/V x layer) at once: plane y of the launch gathers
// token keep[layer][head][j] of every head into row j of a dense staging plane, a second launch writes the staged
// rows to tokens 0 .. n_keep - 1 of the same pages.  Two launches per round of layers, whatever their number
// (the gather is complete before the first row is overwritten, as in the reference, which clones).
__global__ __launch_bounds__(256) void kv_compact_gather_kernel(
    const uint4* __restrict__ cache, long plane16, const int* __restrict__ page_ids, long n_page_ids,
    const long* __restrict__ keep, long keep_layer_stride, long keep_head_stride, long n_keep, int n_heads,
    int chunks_per_head, int page_shift, long n_pages, int layer0, int layers_round, int n_layers,
    uint4* __restrict__ staged) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long per_tok = (long)n_heads * chunks_per_head;
  const long j = idx / per_tok;
  if (j >= n_keep) return;
  const int rem = (int)(idx - j * per_tok);
  const int head = rem / chunks_per_head;
  const int kv = blockIdx.y / layers_round, li = blockIdx.y - kv * layers_round;
  const long t = keep[(long)(layer0 + li) * keep_layer_stride + (long)head * keep_head_stride + j];
  uint4 v = {0u, 0u, 0u, 0u};
  const long pi = t >> page_shift;
  if (t >= 0 && pi < n_page_ids) {
    const long page = page_ids[pi];
    if (page >= 0 && page < n_pages) {
      const long slot = (page << page_shift) + (t & ((1L << page_shift) - 1));
      v = cache[((long)kv * n_layers + layer0 + li) * plane16 + slot * per_tok + rem];
    }
  }
  staged[(long)blockIdx.y * n_keep * per_tok + idx] = v;
}

__global__ __launch_bounds__(256) void kv_compact_scatter_kernel(
    uint4* __restrict__ cache, long plane16, const int* __restrict__ page_ids, long n_page_ids, long n_keep,
    long per_tok, int page_shift, long n_pages, int layer0, int layers_round, int n_layers,
    const uint4* __restrict__ staged) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long j = idx / per_tok;
  if (j >= n_keep) return;
  const int rem = (int)(idx - j * per_tok);
  const long pi = j >> page_shift;
  if (pi >= n_page_ids) return;
  const long page = page_ids[pi];
  if (page < 0 || page >= n_pages) return;
  const int kv = blockIdx.y / layers_round, li = blockIdx.y - kv * layers_round;
  const long slot = (page << page_shift) + (j & ((1L << page_shift) - 1));
  cache[((long)kv * n_layers + layer0 + li) * plane16 + slot * per_tok + rem] = staged[(long)blockIdx.y * n_keep * per_tok + idx];
}

// whole pages between two caches, all planes (K/V x layer) in one launch:
// dst[plane][dst_page_ids[i]] = src[plane][src_page_ids[i]]; pages outside either cache are skipped
__global__ __launch_bounds__(256) void kv_copy_pages_kernel(
    const uint4* __restrict__ src, uint4* __restrict__ dst, const int* __restrict__ src_page_ids,
    const int* __restrict__ dst_page_ids, long page16, long src_plane16, long dst_plane16, long src_n_pages,
    long dst_n_pages, int parts) {
  const long i = blockIdx.x / parts;
  const int part = blockIdx.x - (int)i * parts;
  const long plane = blockIdx.y;
  const long sp = src_page_ids[i], dp = dst_page_ids[i];
  if (sp < 0 || sp >= src_n_pages || dp < 0 || dp >= dst_n_pages) return;
  const uint4* s = src + plane * src_plane16 + sp * page16;
  uint4* d = dst + plane * dst_plane16 + dp * page16;
  const long seg = (page16 + parts - 1) / parts;
  const long begin = (long)part * seg;
  long end = begin + seg;
  end = end < page16 ? end : page16;
  long c = begin + threadIdx.x;
  for (; c + 3 * 256 < end; c += 4 * 256) {  // four 16-byte loads in flight per lane
    const uint4 a0 = s[c], a1 = s[c + 256], a2 = s[c + 512], a3 = s[c + 768];
    d[c] = a0; d[c + 256] = a1; d[c + 512] = a2; d[c + 768] = a3;
  }
  for (; c < end; c += 256) d[c] = s[c];
}

static int ilog2_exact_l(long v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int s = 0;
  while ((1L << s) < v) ++s;
  return s;
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// shared by the prefill entry point (defined in attn_kernel.hip)
int kv_store_launch(const void* key, const void* value, void* k_cache, void* v_cache,
                    const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                    int64_t key_stride, int64_t value_stride, int64_t n_slots, hipStream_t stream) {
  if (!key || !value || !k_cache || !v_cache || !slot_mapping) return PDLLM_ERR_NULL;
  if (n_tokens < 0 || row_elems <= 0 || n_slots < 0) return PDLLM_ERR_SHAPE;
  if (row_elems % 8 || key_stride % 8 || value_stride % 8) return PDLLM_ERR_STRIDE;
  if (key_stride < row_elems || value_stride < row_elems) return PDLLM_ERR_STRIDE;
  if (!aligned16(key) || !aligned16(value) || !aligned16(k_cache) || !aligned16(v_cache)) return PDLLM_ERR_STRIDE;
  if (n_tokens == 0) return PDLLM_OK;
  const int cpr = (int)(row_elems / 8);
  const long total = n_tokens * cpr;
  hipLaunchKernelGGL(kv_store_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                     static_cast<const uint4*>(key), static_cast<const uint4*>(value),
                     static_cast<uint4*>(k_cache), static_cast<uint4*>(v_cache), slot_mapping,
                     (long)n_tokens, cpr, (long)(key_stride / 8), (long)(value_stride / 8), (long)n_slots);
  return launch_status();
}

}  // namespace pdllm

using namespace pdllm;

extern "C" int pdllm_kv_store(const void* key, const void* value, void* k_cache, void* v_cache,
                              const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                              int64_t key_stride, int64_t value_stride, int64_t n_slots,
                              pdllm_stream_t stream) {
  return kv_store_launch(key, value, k_cache, v_cache, slot_mapping, n_tokens, row_elems, key_stride,
                         value_stride, n_slots, static_cast<hipStream_t>(stream));
}

extern "C" int pdllm_kv_store_fp8(const void* key, const void* value, void* k_cache, void* v_cache,
                                  const float* k_scale, const float* v_scale,
                                  const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                                  int64_t key_stride, int64_t value_stride, int64_t n_slots,
                                  int32_t page_size, int32_t head_dim, int64_t scale_page_stride,
                                  int64_t scale_head_stride, pdllm_stream_t stream) {
  if (!key || !value || !k_cache || !v_cache || !slot_mapping || !k_scale || !v_scale) return PDLLM_ERR_NULL;
  if (n_tokens < 0 || row_elems <= 0 || n_slots < 0) return PDLLM_ERR_SHAPE;
  if (head_dim <= 0 || head_dim % 8 || row_elems % head_dim) return PDLLM_ERR_SHAPE;
  if (scale_page_stride < 0 || scale_head_stride < 0) return PDLLM_ERR_STRIDE;
  const int shift = ilog2_exact_l(page_size);
  if (shift < 0) return PDLLM_ERR_SHAPE;
  if (row_elems % 8 || key_stride % 8 || value_stride % 8) return PDLLM_ERR_STRIDE;
  if (key_stride < row_elems || value_stride < row_elems) return PDLLM_ERR_STRIDE;
  if (!aligned16(key) || !aligned16(value) || ((uintptr_t)k_cache % 8) || ((uintptr_t)v_cache % 8)) return PDLLM_ERR_STRIDE;
  if (n_tokens == 0) return PDLLM_OK;
  const int cpr = (int)(row_elems / 8);
  const long total = n_tokens * cpr;
  hipLaunchKernelGGL(kv_store_fp8_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(key),
                     static_cast<const uint4*>(value), static_cast<uint2*>(k_cache),
                     static_cast<uint2*>(v_cache), k_scale, v_scale, slot_mapping, (long)n_tokens, cpr,
                     (long)(key_stride / 8), (long)(value_stride / 8), (long)n_slots, shift, (int)(head_dim / 8),
                     (long)scale_page_stride, (long)scale_head_stride);
  return launch_status();
}

extern "C" int pdllm_slot_mapping(const int32_t* page_ids, int64_t n_page_ids, int64_t start_token,
                                  int64_t n_tokens, int32_t page_size, int32_t* slots_out,
                                  pdllm_stream_t stream) {
  if (!page_ids || !slots_out) return PDLLM_ERR_NULL;
  const int shift = ilog2_exact_l(page_size);
  if (shift < 0 || n_page_ids < 0 || n_tokens < 0 || start_token < 0) return PDLLM_ERR_SHAPE;
  if (n_tokens == 0) return PDLLM_OK;
  hipLaunchKernelGGL(slot_mapping_kernel, dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), page_ids, (long)n_page_ids, (long)start_token,
                     (long)n_tokens, shift, slots_out);
  return launch_status();
}

extern "C" int pdllm_kv_load(const void* k_cache, const void* v_cache, const void* k_new,
                             const void* v_new, void* k_out, void* v_out, const int32_t* block_table,
                             int64_t bt_stride, const int32_t* ctx_lens, const int32_t* cu_seqlens_q,
                             const int32_t* cu_seqlens_k, int32_t n_seqs, int64_t max_total_len,
                             int64_t row_elems, int32_t page_size, int64_t n_pages, int64_t new_stride,
                             int64_t out_stride, pdllm_stream_t stream) {
  if (!k_cache || !v_cache || !k_new || !v_new || !k_out || !v_out || !block_table || !ctx_lens ||
      !cu_seqlens_q || !cu_seqlens_k)
    return PDLLM_ERR_NULL;
  const int shift = ilog2_exact_l(page_size);
  if (shift < 0 || n_seqs <= 0 || n_seqs > 65535 || max_total_len < 0 || row_elems <= 0 || n_pages <= 0 || bt_stride <= 0)
    return PDLLM_ERR_SHAPE;
  if (row_elems % 8 || new_stride % 8 || out_stride % 8 || new_stride < row_elems || out_stride < row_elems)
    return PDLLM_ERR_STRIDE;
  if (!aligned16(k_cache) || !aligned16(v_cache) || !aligned16(k_new) || !aligned16(v_new) ||
      !aligned16(k_out) || !aligned16(v_out))
    return PDLLM_ERR_STRIDE;
  if (max_total_len == 0) return PDLLM_OK;
  const int cpr = (int)(row_elems / 8);
  const long total = max_total_len * cpr;
  hipLaunchKernelGGL(kv_load_kernel, dim3((unsigned)((total + 255) / 256), (unsigned)n_seqs), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(k_cache),
                     static_cast<const uint4*>(v_cache), static_cast<const uint4*>(k_new),
                     static_cast<const uint4*>(v_new), static_cast<uint4*>(k_out),
                     static_cast<uint4*>(v_out), block_table, (long)bt_stride, ctx_lens, cu_seqlens_q,
                     cu_seqlens_k, cpr, shift, (long)n_pages, (long)(new_stride / 8), (long)(out_stride / 8));
  return launch_status();
}

extern "C" int pdllm_kv_gather(const void* cache, const int32_t* page_ids, int64_t n_page_ids,
                               const int64_t* token_idx, int64_t idx_head_stride, int64_t src_offset,
                               int64_t n_tokens, int32_t num_kv_heads, int32_t head_dim,
                               int32_t page_size, int64_t n_pages, int32_t elem_bytes, void* dst,
                               pdllm_stream_t stream) {
  if (!cache || !page_ids || !dst) return PDLLM_ERR_NULL;
  const int shift = ilog2_exact_l(page_size);
  if (shift < 0 || n_page_ids < 0 || n_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || n_pages <= 0)
    return PDLLM_ERR_SHAPE;
  if (elem_bytes != 1 && elem_bytes != 2) return PDLLM_ERR_DTYPE;
  if (((long)head_dim * elem_bytes) % 16) return PDLLM_ERR_STRIDE;
  if (!aligned16(cache) || !aligned16(dst)) return PDLLM_ERR_STRIDE;
  if (token_idx && idx_head_stride < 0) return PDLLM_ERR_STRIDE;
  if (n_tokens == 0) return PDLLM_OK;
  const int cph = head_dim * elem_bytes / 16;
  const long total = n_tokens * num_kv_heads * cph;
  hipLaunchKernelGGL(kv_gather_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(cache), page_ids,
                     (long)n_page_ids, reinterpret_cast<const long*>(token_idx), (long)idx_head_stride,
                     (long)src_offset, (long)n_tokens, num_kv_heads, cph, shift, (long)n_pages,
                     static_cast<uint4*>(dst));
  return launch_status();
}

extern "C" int pdllm_kv_scatter(void* cache, const int32_t* page_ids, int64_t n_page_ids,
                                int64_t dst_start, int64_t n_tokens, int32_t num_kv_heads,
                                int32_t head_dim, int32_t page_size, int64_t n_pages,
                                int32_t elem_bytes, const void* src, pdllm_stream_t stream) {
  if (!cache || !page_ids || !src) return PDLLM_ERR_NULL;
  const int shift = ilog2_exact_l(page_size);
  if (shift < 0 || n_page_ids < 0 || n_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || n_pages <= 0 || dst_start < 0)
    return PDLLM_ERR_SHAPE;
  if (elem_bytes != 1 && elem_bytes != 2) return PDLLM_ERR_DTYPE;
  if (((long)head_dim * elem_bytes) % 16) return PDLLM_ERR_STRIDE;
  if (!aligned16(cache) || !aligned16(src)) return PDLLM_ERR_STRIDE;
  if (n_tokens == 0) return PDLLM_OK;
  const long per_tok = (long)num_kv_heads * head_dim * elem_bytes / 16;
  const long total = n_tokens * per_tok;
  hipLaunchKernelGGL(kv_scatter_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint4*>(cache), page_ids,
                     (long)n_page_ids, (long)dst_start, (long)n_tokens, per_tok, shift, (long)n_pages,
                     static_cast<const uint4*>(src));
  return launch_status();
}

extern "C" int64_t pdllm_kv_compact_per_head_workspace_bytes(int64_t n_keep, int32_t num_kv_heads, int32_t head_dim,
                                                             int32_t elem_bytes) {
  if (n_keep < 0 || num_kv_heads <= 0 || head_dim <= 0 || (elem_bytes != 1 && elem_bytes != 2)) return PDLLM_ERR_SHAPE;
  return 2 * n_keep * (int64_t)num_kv_heads * head_dim * elem_bytes;  // K and V of one layer
}

extern "C" int pdllm_kv_compact_per_head(void* kv_cache, int64_t plane_stride_bytes, int32_t n_layers,
                                         const int32_t* page_ids, int64_t n_page_ids, const int64_t* keep,
                                         int64_t keep_layer_stride, int64_t keep_head_stride, int64_t n_keep,
                                         int32_t num_kv_heads, int32_t head_dim, int32_t page_size, int64_t n_pages,
                                         int32_t elem_bytes, void* workspace, int64_t workspace_bytes,
                                         pdllm_stream_t stream) {
  if (!kv_cache || !page_ids || !keep || !workspace) return PDLLM_ERR_NULL;
  const int shift = ilog2_exact_l(page_size);
  if (shift < 0 || n_layers <= 0 || n_page_ids < 0 || n_keep < 0 || num_kv_heads <= 0 || head_dim <= 0 || n_pages <= 0)
    return PDLLM_ERR_SHAPE;
  if (elem_bytes != 1 && elem_bytes != 2) return PDLLM_ERR_DTYPE;
  if (((long)head_dim * elem_bytes) % 16 || plane_stride_bytes % 16) return PDLLM_ERR_STRIDE;
  if (plane_stride_bytes < n_pages * (int64_t)page_size * num_kv_heads * head_dim * elem_bytes) return PDLLM_ERR_STRIDE;
  if (!aligned16(kv_cache) || !aligned16(workspace)) return PDLLM_ERR_STRIDE;
  if (n_keep == 0) return PDLLM_OK;
  const int64_t per_layer = pdllm_kv_compact_per_head_workspace_bytes(n_keep, num_kv_heads, head_dim, elem_bytes);
  if (workspace_bytes < per_layer) return PDLLM_ERR_WORKSPACE;
  int64_t round = workspace_bytes / per_layer;   // layers staged at a time
  if (round > n_layers) round = n_layers;
  if (round > 32767) round = 32767;
  const int cph = head_dim * elem_bytes / 16;
  const long per_tok = (long)num_kv_heads * cph;
  const long total = n_keep * per_tok;
  if ((total + 255) / 256 > 0x7fffffffL) return PDLLM_ERR_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  for (int64_t l0 = 0; l0 < n_layers; l0 += round) {
    const int lr = (int)(n_layers - l0 < round ? n_layers - l0 : round);
    const dim3 grid((unsigned)((total + 255) / 256), (unsigned)(2 * lr));
    hipLaunchKernelGGL(kv_compact_gather_kernel, grid, dim3(256), 0, st, static_cast<const uint4*>(kv_cache),
                       (long)(plane_stride_bytes / 16), page_ids, (long)n_page_ids, reinterpret_cast<const long*>(keep),
                       (long)keep_layer_stride, (long)keep_head_stride, (long)n_keep, num_kv_heads, cph, shift,
                       (long)n_pages, (int)l0, lr, n_layers, static_cast<uint4*>(workspace));
    int rc = launch_status();
    if (rc != PDLLM_OK) return rc;
    hipLaunchKernelGGL(kv_compact_scatter_kernel, grid, dim3(256), 0, st, static_cast<uint4*>(kv_cache),
                       (long)(plane_stride_bytes / 16), page_ids, (long)n_page_ids, (long)n_keep, per_tok, shift,
                       (long)n_pages, (int)l0, lr, n_layers, static_cast<const uint4*>(workspace));
    rc = launch_status();
    if (rc != PDLLM_OK) return rc;
  }
  return PDLLM_OK;
}

extern "C" int pdllm_kv_copy_pages(const void* src_cache, void* dst_cache, const int32_t* src_page_ids,
                                   const int32_t* dst_page_ids, int64_t n_copy, int64_t page_bytes,
                                   int64_t n_planes, int64_t src_plane_stride_bytes,
                                   int64_t dst_plane_stride_bytes, int64_t src_n_pages, int64_t dst_n_pages,
                                   pdllm_stream_t stream) {
  if (!src_cache || !dst_cache || !src_page_ids || !dst_page_ids) return PDLLM_ERR_NULL;
  if (n_copy < 0 || page_bytes <= 0 || n_planes <= 0 || n_planes > 65535 || src_n_pages <= 0 || dst_n_pages <= 0)
    return PDLLM_ERR_SHAPE;
  if (page_bytes % 16 || src_plane_stride_bytes % 16 || dst_plane_stride_bytes % 16 ||
      src_plane_stride_bytes < src_n_pages * page_bytes || dst_plane_stride_bytes < dst_n_pages * page_bytes)
    return PDLLM_ERR_STRIDE;
  if (!aligned16(src_cache) || !aligned16(dst_cache)) return PDLLM_ERR_STRIDE;
  if (n_copy == 0) return PDLLM_OK;
  // about 64 KB per workgroup
  int parts = (int)((page_bytes + 65535) / 65536);
  if (n_copy * parts > 0x7fffffffL) return PDLLM_ERR_SHAPE;
  hipLaunchKernelGGL(kv_copy_pages_kernel, dim3((unsigned)(n_copy * parts), (unsigned)n_planes), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(src_cache),
                     static_cast<uint4*>(dst_cache), src_page_ids, dst_page_ids, (long)(page_bytes / 16),
                     (long)(src_plane_stride_bytes / 16), (long)(dst_plane_stride_bytes / 16), (long)src_n_pages,
                     (long)dst_n_pages, parts);
  return launch_status();
}
