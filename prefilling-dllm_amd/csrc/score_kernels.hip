// Vocabulary-wide reductions over bf16 logits for gfx950: draft self-information
// (log-softmax of a label), max-softmax confidence + argmax, and the threshold unmask rule.
// These are single-pass HBM-bound scans: every lane streams 16-byte (8 x bf16) loads, keeps a
// lane-local online (max, sum-of-exp[, argmax]) and the lanes are combined with wavefront
// reductions.  A row is split over several workgroups so that a few hundred rows still fill
// 256 CUs; the per-split partials are combined by a second tiny kernel in split order.
//
// Reference: fastdllm_engine.py:1148-1152 (self-information), :1647-1681 (shift + confidence),
// :2146-2157 (transfer rule) of the reference engine.

#include <mutex>

#include "pdllm_common.h"

namespace pdllm {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct RowStat {
  float m;   // running maximum
  float s;   // sum of exp(x - m)
  long idx;  // first index of the maximum
};

__device__ __forceinline__ void stat_merge(RowStat& a, const RowStat& b) {
  // maximum with lowest-index tie-break, sums rescaled to the common maximum
  const bool b_wins = (b.m > a.m) || (b.m == a.m && b.idx < a.idx);
  const float mm = fmaxf(a.m, b.m);
  const float sa = (a.m == -INFINITY) ? 0.f : a.s * __builtin_amdgcn_exp2f((a.m - mm) * kLog2e);
  const float sb = (b.m == -INFINITY) ? 0.f : b.s * __builtin_amdgcn_exp2f((b.m - mm) * kLog2e);
  a.s = sa + sb;
  a.m = mm;
  if (b_wins) a.idx = b.idx;
}

__device__ __forceinline__ void stat_push(RowStat& st, float x, long i) {
  if (x > st.m) {
    st.s = st.s * __builtin_amdgcn_exp2f((st.m - x) * kLog2e) + 1.f;  // st.m = -inf -> 0
    st.m = x;
    st.idx = i;
  } else {
    st.s += __builtin_amdgcn_exp2f((x - st.m) * kLog2e);
  }
}

// partial[(row * nsplit + split)] = stats of logits[row, split segment]
__global__ __launch_bounds__(256) void vocab_partial_kernel(
    const __bf16* __restrict__ logits, long logits_stride, const __bf16* __restrict__ last_logit,
    long last_stride, long block_len, int shift, long vocab, int nsplit, float* __restrict__ part_m,
    float* __restrict__ part_s, long* __restrict__ part_idx) {
  const long row = blockIdx.y;
  const int split = blockIdx.x;
  // source row after the optional one-position shift inside each block
  const __bf16* src;
  if (shift) {
    const long b = row / block_len, i = row - b * block_len;
    if (i == 0) src = last_logit ? last_logit + b * last_stride : logits + row * logits_stride;
    else src = logits + (row - 1) * logits_stride;
  } else {
    src = logits + row * logits_stride;
  }
  const long seg = (((vocab + nsplit - 1) / nsplit) + 7) & ~7L;  // multiple of 8 elements
  const long begin = (long)split * seg;
  long end = begin + seg;
  end = end < vocab ? end : vocab;

  RowStat st = {-INFINITY, 0.f, 0x7fffffffffffffffL};
  const bool vec_ok = (((uintptr_t)src) % 16) == 0;
  if (vec_ok) {
    for (long i = begin + 8L * threadIdx.x; i < end; i += 8L * 256) {
      if (i + 8 <= end) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src + i);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
        float x[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          x[2 * k] = bf16_bits_to_f32(w[k] & 0xffffu);
          x[2 * k + 1] = bf16_bits_to_f32(w[k] >> 16);
        }
        // vector step: one rescale for the 8 values; the position of a new maximum is only looked
        // for when there is one (rare once the running maximum has settled)
        const float vm = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
        if (vm > st.m) {
          int vi = 7;
#pragma unroll
          for (int k = 6; k >= 0; --k)
            if (x[k] == vm) vi = k;  // first position of the maximum
          st.s *= __builtin_amdgcn_exp2f((st.m - vm) * kLog2e);
          st.m = vm;
          st.idx = i + vi;
        }
        if (st.m > -INFINITY) {
          float acc = 0.f;
#pragma unroll
          for (int k = 0; k < 8; ++k) acc += __builtin_amdgcn_exp2f((x[k] - st.m) * kLog2e);
          st.s += acc;
        }
      } else {
        for (long j = i; j < end; ++j)
          stat_push(st, bf16_bits_to_f32(__builtin_bit_cast(unsigned short, src[j])), j);
      }
    }
  } else {
    for (long j = begin + threadIdx.x; j < end; j += 256)
      stat_push(st, bf16_bits_to_f32(__builtin_bit_cast(unsigned short, src[j])), j);
  }
  // wave reduction, then across the 4 waves through LDS
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    RowStat other;
    other.m = __shfl_xor(st.m, o, 64);
    other.s = __shfl_xor(st.s, o, 64);
    other.idx = __shfl_xor(st.idx, o, 64);
    stat_merge(st, other);
  }
  __shared__ float sm[4], ss[4];
  __shared__ long si[4];
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { sm[wave] = st.m; ss[wave] = st.s; si[wave] = st.idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    RowStat a = {sm[0], ss[0], si[0]};
    for (int w = 1; w < 4; ++w) {
      RowStat b = {sm[w], ss[w], si[w]};
      stat_merge(a, b);
    }
    const long o = row * nsplit + split;
    part_m[o] = a.m;
    part_s[o] = a.s;
    part_idx[o] = a.idx;
  }
}

// the split partials of a row, combined in split order
__device__ __forceinline__ RowStat row_stat(const float* __restrict__ part_m, const float* __restrict__ part_s,
                                            const long* __restrict__ part_idx, int nsplit, long row) {
  RowStat a = {part_m[row * nsplit], part_s[row * nsplit], part_idx[row * nsplit]};
  for (int s = 1; s < nsplit; ++s) {
    RowStat b = {part_m[row * nsplit + s], part_s[row * nsplit + s], part_idx[row * nsplit + s]};
    stat_merge(a, b);
  }
  return a;
}

// log-softmax of the label: logits[row, label] - logsumexp(row); labels outside the vocabulary give -inf
__device__ __forceinline__ float label_logprob(const RowStat& a, const __bf16* __restrict__ logits,
                                               long logits_stride, const long* __restrict__ labels, long vocab,
                                               long row) {
  const long lab = labels[row];
  if (lab < 0 || lab >= vocab) return -INFINITY;
  const float x = bf16_bits_to_f32(__builtin_bit_cast(unsigned short, logits[row * logits_stride + lab]));
  return (x - a.m) - __log2f(a.s) * kLn2;
}

// mode 0: logp[row] = logits[row, label] - logsumexp ; mode 1: conf = 1 / sum exp(x - max), token = argmax
__global__ __launch_bounds__(64) void vocab_final_kernel(
    const float* __restrict__ part_m, const float* __restrict__ part_s, const long* __restrict__ part_idx,
    int nsplit, long n_rows, int mode, const __bf16* __restrict__ logits, long logits_stride,
    const long* __restrict__ labels, long vocab, float* __restrict__ out_f, long* __restrict__ out_i) {
  const long row = (long)blockIdx.x * 64 + threadIdx.x;
  if (row >= n_rows) return;
  const RowStat a = row_stat(part_m, part_s, part_idx, nsplit, row);
  if (mode == 0) {
    out_f[row] = label_logprob(a, logits, logits_stride, labels, vocab, row);
  } else {
    out_f[row] = 1.f / a.s;
    out_i[row] = a.idx;
  }
}

__global__ __launch_bounds__(64) void chunk_score_reduce_kernel(const float* __restrict__ logp,
                                                                long n_chunks, long rows_per_chunk,
                                                                int mean, float* __restrict__ out) {
  const long c = (long)blockIdx.x * 64 + threadIdx.x;
  if (c >= n_chunks) return;
  float acc = 0.f;
  for (long j = 0; j < rows_per_chunk; ++j) acc += logp[c * rows_per_chunk + j];
  out[c] = mean ? acc / (float)rows_per_chunk : acc;
}

// Tail of the chunk scoring in one workgroup: row log-probabilities from the split partials, chunk
// scores (rows added in index order, optionally the mean), and the k best chunks by (score
// descending, index ascending; non-finite scores count as -inf), written in ascending index order
// or best first.  n_chunks <= kSelectMax.
constexpr int kSelectMax = 1024;
constexpr int kSelectRows = 4096;
__global__ __launch_bounds__(256) void score_select_kernel(
    const float* __restrict__ part_m, const float* __restrict__ part_s, const long* __restrict__ part_idx,
    int nsplit, long n_chunks, long rows_per_chunk, int mean, const __bf16* __restrict__ logits,
    long logits_stride, const long* __restrict__ labels, long vocab, long k, int sorted_ascending,
    float* __restrict__ logp_out, float* __restrict__ scores_out, long* __restrict__ idx_out) {
  __shared__ uint64_t keys[kSelectMax];
  __shared__ uint8_t taken[kSelectMax];
  __shared__ float row_lp[kSelectRows];
  const long n_rows = n_chunks * rows_per_chunk;
  const bool staged = n_rows <= kSelectRows;  // one thread per row first, so that the loads of the rows overlap
  if (staged) {
    for (long row = threadIdx.x; row < n_rows; row += 256) {
      const RowStat a = row_stat(part_m, part_s, part_idx, nsplit, row);
      const float r = label_logprob(a, logits, logits_stride, labels, vocab, row);
      if (logp_out) logp_out[row] = r;
      row_lp[row] = r;
    }
    __syncthreads();
  }
  for (long c = threadIdx.x; c < n_chunks; c += 256) {
    float acc = 0.f;
    for (long j = 0; j < rows_per_chunk; ++j) {
      const long row = c * rows_per_chunk + j;
      float r;
      if (staged) {
        r = row_lp[row];
      } else {
        const RowStat a = row_stat(part_m, part_s, part_idx, nsplit, row);
        r = label_logprob(a, logits, logits_stride, labels, vocab, row);
        if (logp_out) logp_out[row] = r;
      }
      acc += r;
    }
    const float score = mean ? acc / (float)rows_per_chunk : acc;
    scores_out[c] = score;
    float v = score;
    if (!(fabsf(v) <= 3.402823466e38f)) v = -INFINITY;
    // smaller key = better: inverted order-preserving image of the score, then the index
    uint32_t u = __float_as_uint(v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    keys[c] = ((uint64_t)(~u) << 32) | (uint32_t)c;
  }
  __syncthreads();
  for (long c = threadIdx.x; c < n_chunks; c += 256) {
    const uint64_t mine = keys[c];
    long rank = 0;
    for (long o = 0; o < n_chunks; ++o) rank += keys[o] < mine ? 1 : 0;
    taken[c] = rank < k ? 1 : 0;
    if (!sorted_ascending && rank < k) idx_out[rank] = c;
  }
  if (!sorted_ascending) return;
  __syncthreads();
  for (long c = threadIdx.x; c < n_chunks; c += 256) {
    if (!taken[c]) continue;
    long pos = 0;
    for (long o = 0; o < c; ++o) pos += taken[o];
    idx_out[pos] = c;
  }
}

// Tail of a denoise step, one wave per block of the batch: confidence (max softmax probability) and
// argmax token of every position from the split partials, then the transfer rule over the positions
// that still hold the mask token: the most confident one (lowest index on ties) always, the others
// when their confidence reaches the threshold.  Writes the tokens into block_ids.
__global__ __launch_bounds__(64) void unmask_tail_kernel(
    const float* __restrict__ part_m, const float* __restrict__ part_s, const long* __restrict__ part_idx,
    int nsplit, long* __restrict__ block_ids, long block_len, long mask_token_id, float threshold,
    float* __restrict__ conf_out, long* __restrict__ token_out, uint8_t* __restrict__ transfer,
    int* __restrict__ n_left) {
  const long b = blockIdx.x;
  const int lane = threadIdx.x;
  const long base = b * block_len;
  float best = -INFINITY;
  long besti = 0x7fffffffffffffffL;
  int n_masked = 0;
  for (long i = lane; i < block_len; i += 64) {
    const RowStat a = row_stat(part_m, part_s, part_idx, nsplit, base + i);
    const float c = 1.f / a.s;
    conf_out[base + i] = c;
    token_out[base + i] = a.idx;
    if (block_ids[base + i] == mask_token_id) {
      ++n_masked;
      if (c > best || besti == 0x7fffffffffffffffL) { best = c; besti = i; }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const long oi = __shfl_xor(besti, o, 64);
    n_masked += __shfl_xor(n_masked, o, 64);
    const bool o_valid = oi != 0x7fffffffffffffffL, s_valid = besti != 0x7fffffffffffffffL;
    const bool take = o_valid && (!s_valid || ob > best || (ob == best && oi < besti));
    if (take) { best = ob; besti = oi; }
  }
  int moved = 0;
  for (long i = lane; i < block_len; i += 64) {
    // this lane wrote conf_out / token_out of position i itself
    const bool masked = block_ids[base + i] == mask_token_id;
    const bool t = masked && (i == besti || conf_out[base + i] >= threshold);
    transfer[base + i] = t ? 1 : 0;
    if (t) { block_ids[base + i] = token_out[base + i]; ++moved; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) moved += __shfl_xor(moved, o, 64);
  if (lane == 0 && n_left) n_left[b] = n_masked - moved;
}

// one wave per block of the batch
__global__ __launch_bounds__(64) void threshold_unmask_kernel(
    const float* __restrict__ conf, const long* __restrict__ token, long* __restrict__ block_ids,
    long block_len, long mask_token_id, float threshold, uint8_t* __restrict__ transfer,
    int* __restrict__ n_left) {
  const long b = blockIdx.x;
  const int lane = threadIdx.x;
  const long base = b * block_len;
  // pass 1: most confident masked position (lowest index on ties)
  float best = -INFINITY;
  long besti = 0x7fffffffffffffffL;
  int n_masked = 0;
  for (long i = lane; i < block_len; i += 64) {
    if (block_ids[base + i] == mask_token_id) {
      ++n_masked;
      const float c = conf[base + i];
      if (c > best || besti == 0x7fffffffffffffffL) { best = c; besti = i; }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const long oi = __shfl_xor(besti, o, 64);
    n_masked += __shfl_xor(n_masked, o, 64);
    const bool o_valid = oi != 0x7fffffffffffffffL, s_valid = besti != 0x7fffffffffffffffL;
    const bool take = o_valid && (!s_valid || ob > best || (ob == best && oi < besti));
    if (take) { best = ob; besti = oi; }
  }
  int moved = 0;
  for (long i = lane; i < block_len; i += 64) {
    const bool masked = block_ids[base + i] == mask_token_id;
    const bool t = masked && (i == besti || conf[base + i] >= threshold);
    transfer[base + i] = t ? 1 : 0;
    if (t) { block_ids[base + i] = token[base + i]; ++moved; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) moved += __shfl_xor(moved, o, 64);
  if (lane == 0 && n_left) n_left[b] = n_masked - moved;
}

// one rotation in fp32 with every product and sum rounded on its own, as the unfused torch expression
// x1 * cos - x2 * sin, x2 * cos + x1 * sin evaluates (no fused multiply-add)
__device__ __forceinline__ void rope_pair(float x1, float x2, float c, float s, float& y1, float& y2) {
#pragma clang fp contract(off)
  const float a = x1 * c, b = x2 * s, e = x2 * c, f = x1 * s;
  y1 = a - b;
  y2 = e + f;
}

// neox rotary embedding in place: x [n_tokens, n_heads, d] bf16
__global__ __launch_bounds__(256) void rope_kernel(__bf16* __restrict__ x, long x_stride,
                                                   const long* __restrict__ positions,
                                                   const float* __restrict__ cos_sin, long max_pos,
                                                   long n_tokens, int n_heads, int head_dim) {
  const int half = head_dim / 2;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long per_tok = (long)n_heads * half;
  const long t = idx / per_tok;
  if (t >= n_tokens) return;
  const int rem = (int)(idx - t * per_tok);
  const int hd = rem / half, i = rem - hd * half;
  const long pos = positions[t];
  if (pos < 0 || pos >= max_pos) return;
  const float c = cos_sin[pos * head_dim + i];
  const float s = cos_sin[pos * head_dim + half + i];
  __bf16* p = x + t * x_stride + (long)hd * head_dim;
  const float x1 = (float)p[i], x2 = (float)p[i + half];
  float y1, y2;
  rope_pair(x1, x2, c, s, y1, y2);
  p[i] = (__bf16)y1;
  p[i + half] = (__bf16)y2;
}

// Rotary embedding of Q and K in place and the paged store of the rotated K and of V in one pass:
// what rope_kernel on Q, rope_kernel on K and the store kernel do one after the other, with K read
// once.  A thread rotates 8 + 8 elements of one head (16-byte loads) or copies 16 bytes of a V row.
__global__ __launch_bounds__(256) void rope_qk_store_kernel(
    __bf16* __restrict__ q, long q_stride, int Hq, __bf16* __restrict__ k, long k_stride,
    const __bf16* __restrict__ v, long v_stride, int Hkv, int head_dim, const long* __restrict__ positions,
    const float* __restrict__ cos_sin, long max_pos, long n_tokens, __bf16* __restrict__ k_cache,
    __bf16* __restrict__ v_cache, const int* __restrict__ slots, long n_slots) {
  const int half = head_dim / 2;
  const int hc = half / 8;  // 8-element groups per half head
  const int per_q = Hq * hc, per_k = Hkv * hc, per_v = Hkv * head_dim / 8;
  const long per_tok = per_q + per_k + per_v;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long t = idx / per_tok;
  if (t >= n_tokens) return;
  const int r = (int)(idx - t * per_tok);
  long slot = slots ? (long)slots[t] : -1;
  if (slot >= n_slots) slot = -1;
  const long row = (long)Hkv * head_dim;
  if (r >= per_q + per_k) {
    if (slot >= 0) {
      const int c = r - per_q - per_k;
      *reinterpret_cast<uint4*>(v_cache + slot * row + 8 * c) = *reinterpret_cast<const uint4*>(v + t * v_stride + 8 * c);
    }
    return;
  }
  const bool is_k = r >= per_q;
  const int rr = is_k ? r - per_q : r;
  const int hd = rr / hc, g = rr - hd * hc;
  __bf16* p = (is_k ? k + t * k_stride : q + t * q_stride) + (long)hd * head_dim + 8 * g;
  bf16x8 lo = *reinterpret_cast<const bf16x8*>(p);
  bf16x8 hi = *reinterpret_cast<const bf16x8*>(p + half);
  const long pos = positions[t];
  if (pos >= 0 && pos < max_pos) {
    const float* cs = cos_sin + pos * head_dim + 8 * g;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float c = cs[j], sn = cs[half + j];
      const float x1 = (float)lo[j], x2 = (float)hi[j];
      float y1, y2;
      rope_pair(x1, x2, c, sn, y1, y2);
      lo[j] = (__bf16)y1;
      hi[j] = (__bf16)y2;
    }
    *reinterpret_cast<bf16x8*>(p) = lo;
    *reinterpret_cast<bf16x8*>(p + half) = hi;
  }
  if (is_k && slot >= 0) {
    __bf16* dst = k_cache + slot * row + (long)hd * head_dim + 8 * g;
    *reinterpret_cast<bf16x8*>(dst) = lo;
    *reinterpret_cast<bf16x8*>(dst + half) = hi;
  }
}

static int vocab_nsplit(long n_rows, long vocab) {
  // aim at >= 1024 workgroups, at least 2048 elements per workgroup
  long want = (1024 + n_rows - 1) / n_rows;
  const long max_by_len = (vocab + 2047) / 2048;
  if (want > max_by_len) want = max_by_len;
  if (want < 1) want = 1;
  if (want > 64) want = 64;
  return (int)want;
}

static int64_t vocab_ws_bytes(long n_rows, long vocab) {
  const int ns = vocab_nsplit(n_rows, vocab);
  return (int64_t)n_rows * ns * (4 + 4 + 8);
}

static int vocab_launch(const void* logits, int64_t logits_stride, const void* last_logit,
                        int64_t last_stride, int64_t n_rows, int64_t block_len, int64_t vocab, int shift,
                        int mode, const int64_t* labels, void* workspace, int64_t workspace_bytes,
                        float* out_f, int64_t* out_i, hipStream_t stream) {
  if (!logits || (!out_f && mode != 2) || !workspace) return PDLLM_ERR_NULL;
  if (mode == 0 && !labels) return PDLLM_ERR_NULL;
  if (mode == 1 && !out_i) return PDLLM_ERR_NULL;
  if (n_rows < 0 || vocab <= 0 || logits_stride < vocab || block_len <= 0) return PDLLM_ERR_SHAPE;
  if (n_rows > 65535) return PDLLM_ERR_UNSUPPORTED;
  if (n_rows == 0) return PDLLM_OK;
  if (workspace_bytes < vocab_ws_bytes(n_rows, vocab) || ((uintptr_t)workspace % 8)) return PDLLM_ERR_WORKSPACE;
  const int ns = vocab_nsplit(n_rows, vocab);
  long* pi = static_cast<long*>(workspace);
  float* pm = reinterpret_cast<float*>(pi + n_rows * ns);
  float* ps = pm + n_rows * ns;
  hipLaunchKernelGGL(vocab_partial_kernel, dim3((unsigned)ns, (unsigned)n_rows), dim3(256), 0, stream,
                     static_cast<const __bf16*>(logits), (long)logits_stride,
                     static_cast<const __bf16*>(last_logit), (long)last_stride, (long)block_len, shift,
                     (long)vocab, ns, pm, ps, pi);
  int st = launch_status();
  if (st != PDLLM_OK) return st;
  if (mode == 2) return PDLLM_OK;  // the caller launches its own tail over the partials
  hipLaunchKernelGGL(vocab_final_kernel, dim3((unsigned)((n_rows + 63) / 64)), dim3(64), 0, stream, pm, ps,
                     pi, ns, (long)n_rows, mode, static_cast<const __bf16*>(logits), (long)logits_stride,
                     reinterpret_cast<const long*>(labels), (long)vocab, out_f,
                     reinterpret_cast<long*>(out_i));
  return launch_status();
}

}  // namespace pdllm

using namespace pdllm;

extern "C" int64_t pdllm_vocab_workspace_bytes(int64_t n_rows, int64_t vocab) {
  if (n_rows < 0 || vocab <= 0) return PDLLM_ERR_SHAPE;
  if (n_rows == 0) return 0;
  return vocab_ws_bytes(n_rows, vocab);
}

extern "C" int pdllm_selfinfo_logprob(const void* logits, int64_t logits_stride, const int64_t* labels,
                                      int64_t n_rows, int64_t vocab, void* workspace,
                                      int64_t workspace_bytes, float* logp_out, pdllm_stream_t stream) {
  return vocab_launch(logits, logits_stride, nullptr, 0, n_rows, 1, vocab, 0, 0, labels, workspace,
                      workspace_bytes, logp_out, nullptr, static_cast<hipStream_t>(stream));
}

extern "C" int pdllm_chunk_score_reduce(const float* logp, int64_t n_chunks, int64_t rows_per_chunk,
                                        int32_t mean, float* scores_out, pdllm_stream_t stream) {
  if (!logp || !scores_out) return PDLLM_ERR_NULL;
  if (n_chunks < 0 || rows_per_chunk <= 0) return PDLLM_ERR_SHAPE;
  if (n_chunks == 0) return PDLLM_OK;
  hipLaunchKernelGGL(chunk_score_reduce_kernel, dim3((unsigned)((n_chunks + 63) / 64)), dim3(64), 0,
                     static_cast<hipStream_t>(stream), logp, (long)n_chunks, (long)rows_per_chunk, mean,
                     scores_out);
  return launch_status();
}

extern "C" int pdllm_conf_argmax(const void* logits, int64_t logits_stride, const void* last_logit,
                                 int64_t last_logit_stride, int64_t n_seqs, int64_t block_len,
                                 int64_t vocab, int32_t shift, void* workspace, int64_t workspace_bytes,
                                 float* conf_out, int64_t* token_out, pdllm_stream_t stream) {
  if (n_seqs < 0 || block_len <= 0) return PDLLM_ERR_SHAPE;
  if (last_logit && last_logit_stride < vocab) return PDLLM_ERR_STRIDE;
  return vocab_launch(logits, logits_stride, last_logit, last_logit_stride, n_seqs * block_len, block_len,
                      vocab, shift ? 1 : 0, 1, nullptr, workspace, workspace_bytes, conf_out, token_out,
                      static_cast<hipStream_t>(stream));
}

extern "C" int pdllm_threshold_unmask(const float* conf, const int64_t* token, int64_t* block_ids,
                                      int64_t n_seqs, int64_t block_len, int64_t mask_token_id,
                                      float threshold, uint8_t* transfer_out, int32_t* n_masked_left,
                                      pdllm_stream_t stream) {
  if (!conf || !token || !block_ids || !transfer_out) return PDLLM_ERR_NULL;
  if (n_seqs < 0 || block_len <= 0) return PDLLM_ERR_SHAPE;
  if (n_seqs == 0) return PDLLM_OK;
  if (n_seqs > 0x7fffffffL) return PDLLM_ERR_SHAPE;
  hipLaunchKernelGGL(threshold_unmask_kernel, dim3((unsigned)n_seqs), dim3(64), 0,
                     static_cast<hipStream_t>(stream), conf, reinterpret_cast<const long*>(token),
                     reinterpret_cast<long*>(block_ids), (long)block_len, (long)mask_token_id, threshold,
                     transfer_out, n_masked_left);
  return launch_status();
}

extern "C" int pdllm_rope_inplace(void* x, int64_t x_stride, const int64_t* positions,
                                  const float* cos_sin_cache, int64_t max_positions, int64_t n_tokens,
                                  int32_t n_heads, int32_t head_dim, pdllm_stream_t stream) {
  if (!x || !positions || !cos_sin_cache) return PDLLM_ERR_NULL;
  if (n_tokens < 0 || n_heads <= 0 || head_dim <= 0 || (head_dim & 1) || max_positions <= 0) return PDLLM_ERR_SHAPE;
  if (x_stride < (int64_t)n_heads * head_dim) return PDLLM_ERR_STRIDE;
  if (n_tokens == 0) return PDLLM_OK;
  const long total = n_tokens * n_heads * (head_dim / 2);
  hipLaunchKernelGGL(rope_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<__bf16*>(x), (long)x_stride,
                     reinterpret_cast<const long*>(positions), cos_sin_cache, (long)max_positions,
                     (long)n_tokens, n_heads, head_dim);
  return launch_status();
}

extern "C" int pdllm_chunk_select(const void* logits, int64_t logits_stride, const int64_t* labels,
                                  int64_t n_chunks, int64_t rows_per_chunk, int64_t vocab, int32_t mean,
                                  int64_t k, int32_t sorted_ascending, void* workspace,
                                  int64_t workspace_bytes, float* logp_out, float* scores_out,
                                  int64_t* indices_out, pdllm_stream_t stream) {
  if (!labels || !scores_out || !indices_out) return PDLLM_ERR_NULL;
  if (n_chunks <= 0 || rows_per_chunk <= 0 || k <= 0 || k > n_chunks) return PDLLM_ERR_SHAPE;
  if (n_chunks > kSelectMax) return PDLLM_ERR_UNSUPPORTED;
  const int64_t n_rows = n_chunks * rows_per_chunk;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  const int st = vocab_launch(logits, logits_stride, nullptr, 0, n_rows, 1, vocab, 0, 2, labels, workspace,
                              workspace_bytes, nullptr, nullptr, hs);
  if (st != PDLLM_OK) return st;
  const int ns = vocab_nsplit(n_rows, vocab);
  long* pi = static_cast<long*>(workspace);
  float* pm = reinterpret_cast<float*>(pi + n_rows * ns);
  float* ps = pm + n_rows * ns;
  hipLaunchKernelGGL(score_select_kernel, dim3(1), dim3(256), 0, hs, pm, ps, pi, ns, (long)n_chunks,
                     (long)rows_per_chunk, mean, static_cast<const __bf16*>(logits), (long)logits_stride,
                     reinterpret_cast<const long*>(labels), (long)vocab, (long)k, sorted_ascending, logp_out,
                     scores_out, reinterpret_cast<long*>(indices_out));
  return launch_status();
}

static int denoise_unmask_launch(const void* logits, int64_t logits_stride, const void* last_logit,
                                 int64_t last_logit_stride, int64_t n_seqs, int64_t block_len,
                                 int64_t vocab, int32_t shift, int64_t* block_ids, int64_t mask_token_id,
                                 float threshold, void* workspace, int64_t workspace_bytes,
                                 float* conf_out, int64_t* token_out, uint8_t* transfer_out,
                                 int32_t* n_masked_left, pdllm_stream_t stream) {
  if (!block_ids || !conf_out || !token_out || !transfer_out) return PDLLM_ERR_NULL;
  if (n_seqs < 0 || block_len <= 0) return PDLLM_ERR_SHAPE;
  if (last_logit && last_logit_stride < vocab) return PDLLM_ERR_STRIDE;
  if (n_seqs == 0) return PDLLM_OK;
  const int64_t n_rows = n_seqs * block_len;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  const int st = vocab_launch(logits, logits_stride, last_logit, last_logit_stride, n_rows, block_len, vocab,
                              shift ? 1 : 0, 2, nullptr, workspace, workspace_bytes, nullptr, nullptr, hs);
  if (st != PDLLM_OK) return st;
  const int ns = vocab_nsplit(n_rows, vocab);
  long* pi = static_cast<long*>(workspace);
  float* pm = reinterpret_cast<float*>(pi + n_rows * ns);
  float* ps = pm + n_rows * ns;
  hipLaunchKernelGGL(unmask_tail_kernel, dim3((unsigned)n_seqs), dim3(64), 0, hs, pm, ps, pi, ns,
                     reinterpret_cast<long*>(block_ids), (long)block_len, (long)mask_token_id, threshold,
                     conf_out, reinterpret_cast<long*>(token_out), transfer_out, n_masked_left);
  return launch_status();
}

extern "C" int pdllm_denoise_unmask(const void* logits, int64_t logits_stride, const void* last_logit,
                                    int64_t last_logit_stride, int64_t n_seqs, int64_t block_len,
                                    int64_t vocab, int32_t shift, int64_t* block_ids, int64_t mask_token_id,
                                    float threshold, void* workspace, int64_t workspace_bytes,
                                    float* conf_out, int64_t* token_out, uint8_t* transfer_out,
                                    int32_t* n_masked_left, pdllm_stream_t stream) {
  return denoise_unmask_launch(logits, logits_stride, last_logit, last_logit_stride, n_seqs, block_len, vocab, shift,
                               block_ids, mask_token_id, threshold, workspace, workspace_bytes, conf_out, token_out,
                               transfer_out, n_masked_left, stream);
}

// ---------------------------------------------------------------------------------------------
// The same step for callers that cannot allocate a workspace: the per-row, per-split partials live
// in a static device array.  Every GPU the library runs on holds its own copy of the array at its
// own address; that address is looked up once per device, on the first call made with that device
// current, and host code uses the looked-up pointer only (the array's name is not a device address
// on the host).
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[PDLLM_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

static int static_scratch_ptr(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return PDLLM_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return PDLLM_ERR_LAUNCH;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return PDLLM_OK;
}

extern "C" int pdllm_denoise_unmask_static(const void* logits, int64_t logits_stride, const void* last_logit,
                                           int64_t last_logit_stride, int64_t n_seqs, int64_t block_len,
                                           int64_t vocab, int32_t shift, int64_t* block_ids,
                                           int64_t mask_token_id, float threshold, float* conf_out,
                                           int64_t* token_out, uint8_t* transfer_out, int32_t* n_masked_left,
                                           pdllm_stream_t stream) {
  if (n_seqs < 0 || block_len <= 0 || vocab <= 0) return PDLLM_ERR_SHAPE;
  if (n_seqs == 0) return PDLLM_OK;
  if (n_seqs * block_len > 65535) return PDLLM_ERR_UNSUPPORTED;
  if (vocab_ws_bytes(n_seqs * block_len, vocab) > (int64_t)PDLLM_STATIC_SCRATCH_BYTES) return PDLLM_ERR_SCRATCH_LIMIT;
  void* ptr = nullptr;
  const int st = static_scratch_ptr(&ptr);
  if (st != PDLLM_OK) return st;
  // every partial the tail reads is written by the scan of the same call: nothing has to start at zero
  return denoise_unmask_launch(logits, logits_stride, last_logit, last_logit_stride, n_seqs, block_len, vocab, shift,
                               block_ids, mask_token_id, threshold, ptr, (int64_t)PDLLM_STATIC_SCRATCH_BYTES, conf_out,
                               token_out, transfer_out, n_masked_left, stream);
}

extern "C" int pdllm_rope_qk_store(void* q, int64_t q_stride, int32_t num_q_heads, void* k, int64_t k_stride,
                                   const void* v, int64_t v_stride, int32_t num_kv_heads, int32_t head_dim,
                                   const int64_t* positions, const float* cos_sin_cache, int64_t max_positions,
                                   int64_t n_tokens, void* k_cache, void* v_cache, const int32_t* slot_mapping,
                                   int64_t n_slots, pdllm_stream_t stream) {
  if (!q || !k || !positions || !cos_sin_cache) return PDLLM_ERR_NULL;
  if (slot_mapping && (!v || !k_cache || !v_cache)) return PDLLM_ERR_NULL;
  if (n_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || head_dim % 16 || max_positions <= 0 ||
      n_slots < 0)
    return PDLLM_ERR_SHAPE;
  if (q_stride < (int64_t)num_q_heads * head_dim || k_stride < (int64_t)num_kv_heads * head_dim || q_stride % 8 ||
      k_stride % 8)
    return PDLLM_ERR_STRIDE;
  if (slot_mapping && (v_stride < (int64_t)num_kv_heads * head_dim || v_stride % 8)) return PDLLM_ERR_STRIDE;
  if (((uintptr_t)q % 16) || ((uintptr_t)k % 16) || ((uintptr_t)cos_sin_cache % 4)) return PDLLM_ERR_STRIDE;
  if (slot_mapping && (((uintptr_t)v % 16) || ((uintptr_t)k_cache % 16) || ((uintptr_t)v_cache % 16))) return PDLLM_ERR_STRIDE;
  if (n_tokens == 0) return PDLLM_OK;
  const long per_tok = (long)(num_q_heads + num_kv_heads) * (head_dim / 16) + (long)num_kv_heads * head_dim / 8;
  const long total = n_tokens * per_tok;
  if ((total + 255) / 256 > 0x7fffffffL) return PDLLM_ERR_SHAPE;
  hipLaunchKernelGGL(rope_qk_store_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<__bf16*>(q), (long)q_stride, num_q_heads,
                     static_cast<__bf16*>(k), (long)k_stride, static_cast<const __bf16*>(v), (long)v_stride,
                     num_kv_heads, head_dim, reinterpret_cast<const long*>(positions), cos_sin_cache,
                     (long)max_positions, (long)n_tokens, static_cast<__bf16*>(k_cache),
                     static_cast<__bf16*>(v_cache), slot_mapping, (long)n_slots);
  return launch_status();
}
