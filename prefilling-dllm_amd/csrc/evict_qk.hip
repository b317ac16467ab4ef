// Query-to-chunk eviction scores from q and k on the matrix cores (gfx950).
//
// Replaces query_to_chunk_attention_scores (layers/attention/ops/triton_eviction_scorer.py:6-210) and the torch
// path of _engine_chunk_attention_head_scores (fastdllm_engine.py:1279-1310): for every q-head the softmax of the
// last query_len rows over all visible keys (prefix || chunk || query rows, causal or full), summed over those rows
// on the chunk columns.
//
// Rows.  The G q-heads of a KV head share its keys, so they are folded into the row dimension: row = head * Lp + qi
// with Lp = query_len rounded up to a multiple of 8 (padding rows count for nothing).  Every aligned group of 8 rows
// then belongs to one head, which is what the column sums need.
//
// Two launches, both v_mfma_f32_32x32x16_bf16 with the K and Q fragments loaded straight from global memory in
// the operand layout (lane l, half h: row l, elements 16 ks + 8 h .. + 8):
//   1. statistics: D = K Q^T, a lane holds 16 keys of one query row, so the running maximum and the sum of
//      exponentials of a row are in-lane plus one half-wave exchange.  A workgroup takes a segment of the keys
//      (its four waves 32 keys each per step) and all rows; the (max, sum) of every row and segment go to the
//      workspace.
//   2. columns: D = Q K^T over 32 chunk keys per workgroup, a lane holds 16 rows of one key: p = 2^(c s - m) / sum
//      with the row's merged statistics, added over the rows of a head in a fixed order (in-lane, half-wave,
//      row groups, row blocks, waves), so the result is reproducible bit for bit.
// The scalar kernels in select_kernels.hip stay for head dims other than 128 and very wide head groups.

#include "pdllm_common.h"

namespace pdllm {

int evict_score_qk_scalar(const void* q, const void* k, int64_t prefix_len, int64_t chunk_len, int64_t query_len,
                          int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, float scale, int32_t reduce_mean,
                          int32_t causal, float* workspace, float* out, hipStream_t stream);  // select_kernels.hip

namespace {

constexpr int kEqD = 128;
constexpr int kEqMaxG = 16;     // q-heads per KV head the matrix-core path takes
constexpr int kEqMaxRows = kEqMaxG * 64;
constexpr int kEqStatBlocks = 2;  // row blocks per workgroup of the statistics launch
constexpr int kEqMaxSeg = 16;   // key segments of the statistics launch (every workgroup of the second one merges them)

struct EqParams {
  const __bf16* q;
  const __bf16* k;
  float* part;  // [Hkv][rows][n_seg][2]: running maximum (log2 units) and sum of a row over a key segment
  float* out;   // [Hq][chunk_len]
  long prefix_len, chunk_len, n_keys;
  int Lq, Lp, Hq, Hkv, G, rows, n_rb, n_seg, keys_per_seg, causal, reduce_mean;
  float c;  // scale * log2(e)
};

__device__ __forceinline__ float eq_half_max(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float eq_half_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// the eight operand fragments of row `row_ptr` (128 bf16): lane half h takes elements 16 ks + 8 h .. + 8
__device__ __forceinline__ void eq_load_frags(bf16x8 (&f)[8], const __bf16* row_ptr, int h, bool valid) {
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    if (valid) {
      f[ks] = *reinterpret_cast<const bf16x8*>(row_ptr + 16 * ks + 8 * h);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[ks][e] = (__bf16)0.f;
    }
  }
}

// ---- launch 1: row statistics over a segment of the keys -------------------------------------------------------
__global__ __launch_bounds__(256) void evict_qk_stats_kernel(const EqParams p) {
  __shared__ float s_m[4][kEqMaxRows];
  __shared__ float s_l[4][kEqMaxRows];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, h = lane >> 5;
  const int seg = blockIdx.x, kvh = blockIdx.y;
  const long seg0 = (long)seg * p.keys_per_seg;
  long seg1 = seg0 + p.keys_per_seg;
  seg1 = seg1 < p.n_keys ? seg1 : p.n_keys;
  const long q_row0 = p.prefix_len + p.chunk_len;  // sequence position of query row 0
  // (a workgroup takes kEqStatBlocks row blocks: each one costs two round trips to memory in a row, so the row
  // blocks are spread over workgroups rather than walked by one)
  const int rb0 = blockIdx.z * kEqStatBlocks;
  const int rb1 = rb0 + kEqStatBlocks < p.n_rb ? rb0 + kEqStatBlocks : p.n_rb;
  for (int rb = rb0; rb < rb1; ++rb) {
    const int r = 32 * rb + l32;
    const int hg = r / p.Lp, qi = r - hg * p.Lp;
    const bool valid = hg < p.G && qi < p.Lq;
    bf16x8 qf[8];
    eq_load_frags(qf, p.q + ((q_row0 + (valid ? qi : 0)) * p.Hq + kvh * p.G + (valid ? hg : 0)) * kEqD, h, valid);
    const long last_visible = p.causal ? q_row0 + qi : p.n_keys - 1;
    // running statistics of this lane's query row over its half of the keys of each step
    float m = -INFINITY, l = 0.f;
    for (long key0 = seg0 + 32 * wave; key0 < seg1; key0 += 128) {
      const long key = key0 + l32;
      bf16x8 kf[8];
      eq_load_frags(kf, p.k + ((key < p.n_keys ? key : p.n_keys - 1) * p.Hkv + kvh) * kEqD, h, true);
      f32x16 acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], acc, 0, 0, 0);
      // element i: key key0 + 8 (i / 4) + 4 h + i % 4 against this lane's query row
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const long kk = key0 + 8 * (i >> 2) + 4 * h + (i & 3);
        acc[i] = (kk < seg1 && kk <= last_visible) ? acc[i] * p.c : -INFINITY;
        mx = fmaxf(mx, acc[i]);
      }
      if (mx > -INFINITY) {
        const float mn = fmaxf(m, mx);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) s += __builtin_amdgcn_exp2f(acc[i] - mn);
        l = l * __builtin_amdgcn_exp2f(m - mn) + s;  // (m = -inf: l = 0, the factor is 0)
        m = mn;
      }
    }
    // the two halves of the wave
    const float mm = eq_half_max(m);
    const float ll = eq_half_sum(m == -INFINITY ? 0.f : l * __builtin_amdgcn_exp2f(m - mm));
    if (h == 0) { s_m[wave][r] = mm; s_l[wave][r] = ll; }
  }
  // the four waves, in a fixed order
  __syncthreads();
  for (int r = 32 * rb0 + threadIdx.x; r < 32 * rb1 && r < p.rows; r += 256) {
    float mm = s_m[0][r];
#pragma unroll
    for (int w = 1; w < 4; ++w) mm = fmaxf(mm, s_m[w][r]);
    float ll = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) ll += s_m[w][r] == -INFINITY ? 0.f : s_l[w][r] * __builtin_amdgcn_exp2f(s_m[w][r] - mm);
    float* dst = p.part + (((long)kvh * p.rows + r) * p.n_seg + seg) * 2;
    dst[0] = mm;
    dst[1] = ll;
  }
}

// ---- launch 2: column sums over the rows of every head, 32 chunk keys per workgroup ----------------------------
__global__ __launch_bounds__(256) void evict_qk_cols_kernel(const EqParams p) {
  __shared__ __attribute__((aligned(16))) float s_m[kEqMaxRows];   // merged maximum of a row
  __shared__ __attribute__((aligned(16))) float s_w[kEqMaxRows];   // 1 / sum, 0 for a row that counts for nothing
  __shared__ float s_col[4][kEqMaxG][32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, h = lane >> 5;
  const int kvh = blockIdx.y;
  const long col0 = (long)blockIdx.x * 32;
  // merge the segments' statistics (in segment order)
  for (int r = threadIdx.x; r < 32 * p.n_rb; r += 256) {
    float mm = -INFINITY, ll = 0.f;
    const int hg = r / p.Lp, qi = r - hg * p.Lp;
    if (r < p.rows && hg < p.G && qi < p.Lq) {
      const float* src = p.part + ((long)kvh * p.rows + r) * p.n_seg * 2;
      for (int s = 0; s < p.n_seg; ++s) mm = fmaxf(mm, src[2 * s]);
      for (int s = 0; s < p.n_seg; ++s)
        ll += src[2 * s] == -INFINITY ? 0.f : src[2 * s + 1] * __builtin_amdgcn_exp2f(src[2 * s] - mm);
    }
    s_m[r] = mm == -INFINITY ? 0.f : mm;
    s_w[r] = ll > 0.f ? 1.f / ll : 0.f;
  }
  for (int i = threadIdx.x; i < 4 * kEqMaxG * 32; i += 256) (&s_col[0][0][0])[i] = 0.f;
  __syncthreads();
  const long col = col0 + l32;
  bf16x8 kf[8];
  eq_load_frags(kf, p.k + ((p.prefix_len + (col < p.chunk_len ? col : p.chunk_len - 1)) * p.Hkv + kvh) * kEqD, h, true);
  const long q_row0 = p.prefix_len + p.chunk_len;
  auto load_q = [&](bf16x8 (&qf)[8], int rb) {
    const int r = 32 * rb + l32;
    const int hg = r / p.Lp, qi = r - hg * p.Lp;
    const bool valid = rb < p.n_rb && hg < p.G && qi < p.Lq;
    eq_load_frags(qf, p.q + ((q_row0 + (valid ? qi : 0)) * p.Hq + kvh * p.G + (valid ? hg : 0)) * kEqD, h, valid);
  };
  auto block = [&](const bf16x8 (&qf)[8], int rb) {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[ks], kf[ks], acc, 0, 0, 0);
    // element i: row 32 rb + 8 (i / 4) + 4 h + i % 4 against this lane's key; the chunk columns precede every query
    // row, so they are visible under a causal mask too
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rr = 32 * rb + 8 * j + 4 * h;
      const float4 mm = *reinterpret_cast<const float4*>(&s_m[rr]);
      const float4 ww = *reinterpret_cast<const float4*>(&s_w[rr]);
      float g = __builtin_amdgcn_exp2f(acc[4 * j + 0] * p.c - mm.x) * ww.x;
      g += __builtin_amdgcn_exp2f(acc[4 * j + 1] * p.c - mm.y) * ww.y;
      g += __builtin_amdgcn_exp2f(acc[4 * j + 2] * p.c - mm.z) * ww.z;
      g += __builtin_amdgcn_exp2f(acc[4 * j + 3] * p.c - mm.w) * ww.w;
      g = eq_half_sum(g);  // the 8 rows of group j (one head: Lp is a multiple of 8)
      const int head = (32 * rb + 8 * j) / p.Lp;
      if (h == 0 && head < p.G) s_col[wave][head][l32] += g;  // one wave, program order: a fixed order of additions
    }
  };
  // two sets of Q fragments: the next row block's are on their way while this one is computed
  bf16x8 qa[8], qb[8];
  load_q(qa, wave);
  for (int rb = wave; rb < p.n_rb; rb += 8) {
    load_q(qb, rb + 4);
    block(qa, rb);
    if (rb + 4 < p.n_rb) {
      load_q(qa, rb + 8);
      block(qb, rb + 4);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < p.G * 32; i += 256) {
    const int head = i >> 5, cc = i & 31;
    if (col0 + cc < p.chunk_len) {
      float v = s_col[0][head][cc];
#pragma unroll
      for (int w = 1; w < 4; ++w) v += s_col[w][head][cc];
      p.out[((long)kvh * p.G + head) * p.chunk_len + col0 + cc] = p.reduce_mean ? v / (float)p.Lq : v;
    }
  }
}

bool eq_fast_path(int64_t query_len, int32_t hq, int32_t hkv, int32_t d) {
  return d == kEqD && query_len >= 1 && query_len <= 64 && hq / hkv <= kEqMaxG;
}

void eq_shape(int64_t prefix_len, int64_t chunk_len, int64_t query_len, int32_t hq, int32_t hkv, EqParams& p) {
  p.prefix_len = prefix_len;
  p.chunk_len = chunk_len;
  p.n_keys = prefix_len + chunk_len + query_len;
  p.Lq = (int)query_len;
  p.Lp = (int)((query_len + 7) / 8 * 8);
  p.Hq = hq;
  p.Hkv = hkv;
  p.G = hq / hkv;
  p.rows = p.G * p.Lp;
  p.n_rb = (p.rows + 31) / 32;
  const long steps = (p.n_keys + 127) / 128;  // a workgroup takes 128 keys per step
  p.n_seg = (int)(steps < kEqMaxSeg ? steps : kEqMaxSeg);
  p.keys_per_seg = (int)((steps + p.n_seg - 1) / p.n_seg * 128);
  p.n_seg = (int)((p.n_keys + p.keys_per_seg - 1) / p.keys_per_seg);
}

}  // namespace
}  // namespace pdllm

using namespace pdllm;

extern "C" int64_t pdllm_evict_score_qk_workspace_bytes(int64_t prefix_len, int64_t chunk_len, int64_t query_len,
                                                        int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim) {
  if (prefix_len < 0 || chunk_len <= 0 || query_len <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 ||
      num_q_heads % num_kv_heads || head_dim <= 0)
    return PDLLM_ERR_SHAPE;
  if (!eq_fast_path(query_len, num_q_heads, num_kv_heads, head_dim)) return 2 * (int64_t)num_q_heads * query_len * 4;
  EqParams p = {};
  eq_shape(prefix_len, chunk_len, query_len, num_q_heads, num_kv_heads, p);
  return (int64_t)p.Hkv * p.rows * p.n_seg * 2 * 4;
}

extern "C" int pdllm_evict_score_qk(const void* q, const void* k, int64_t prefix_len, int64_t chunk_len,
                                    int64_t query_len, int32_t num_q_heads, int32_t num_kv_heads,
                                    int32_t head_dim, float scale, int32_t reduce_mean, int32_t causal,
                                    float* workspace, int64_t workspace_bytes, float* out, pdllm_stream_t stream) {
  if (!q || !k || !workspace || !out) return PDLLM_ERR_NULL;
  if (prefix_len < 0 || chunk_len <= 0 || query_len <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 ||
      num_q_heads % num_kv_heads || head_dim <= 0)
    return PDLLM_ERR_SHAPE;
  if (head_dim > 256 || query_len > 64) return PDLLM_ERR_UNSUPPORTED;  // limits of the reference scorer
  const int64_t need = pdllm_evict_score_qk_workspace_bytes(prefix_len, chunk_len, query_len, num_q_heads,
                                                            num_kv_heads, head_dim);
  if (workspace_bytes < need || ((uintptr_t)workspace % 4)) return PDLLM_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!eq_fast_path(query_len, num_q_heads, num_kv_heads, head_dim) || ((uintptr_t)q | (uintptr_t)k) % 16)
    return evict_score_qk_scalar(q, k, prefix_len, chunk_len, query_len, num_q_heads, num_kv_heads, head_dim, scale,
                                 reduce_mean, causal, workspace, out, st);
  EqParams p = {};
  eq_shape(prefix_len, chunk_len, query_len, num_q_heads, num_kv_heads, p);
  p.q = static_cast<const __bf16*>(q);
  p.k = static_cast<const __bf16*>(k);
  p.part = workspace;
  p.out = out;
  p.causal = causal;
  p.reduce_mean = reduce_mean;
  p.c = scale * 1.4426950408889634f;
  if (p.Hkv > 65535) return PDLLM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(evict_qk_stats_kernel,
                     dim3((unsigned)p.n_seg, (unsigned)p.Hkv, (unsigned)((p.n_rb + kEqStatBlocks - 1) / kEqStatBlocks)),
                     dim3(256), 0, st, p);
  int rc = launch_status();
  if (rc != PDLLM_OK) return rc;
  hipLaunchKernelGGL(evict_qk_cols_kernel, dim3((unsigned)((chunk_len + 31) / 32), (unsigned)p.Hkv), dim3(256), 0, st, p);
  return launch_status();
}
