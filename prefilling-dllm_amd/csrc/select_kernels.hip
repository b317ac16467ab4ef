// Selection kernels for gfx950: top-K of chunk scores, BOS-forced top-B of token scores
// (both with a total order: score first, lowest index on ties), column sums of attention
// probabilities, the query-to-chunk eviction scorer and token-score pooling.
//
// Reference: fastdllm_engine.py:1199-1204 (chunk ranking), :903-927 (token keep set),
// :1230-1322 + layers/attention/ops/triton_eviction_scorer.py:6-210 (eviction scores),
// :1405-1433 (pooling and per-KV-head grouping) of the reference engine.

#include <type_traits>
#include "pdllm_common.h"

namespace pdllm {

// Monotone map float -> uint32: a < b  <=>  ord(a) < ord(b); NaN above +inf.
__device__ __forceinline__ uint32_t float_ord(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN: largest
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// 64-bit sort key, smaller = better.  descending: high score first.
__device__ __forceinline__ uint64_t make_key(float score, uint32_t idx, bool descending) {
  const uint32_t o = float_ord(score);
  const uint32_t hi = descending ? ~o : o;
  return ((uint64_t)hi << 32) | idx;
}

constexpr int kSortMax = 2048;

// in-LDS bitonic sort (ascending) of npad (power of two <= kSortMax) keys by 256 threads
__device__ void bitonic_sort(uint64_t* keys, int npad) {
  for (int k = 2; k <= npad; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = threadIdx.x; i < npad; i += 256) {
        const int ixj = i ^ j;
        if (ixj > i) {
          const uint64_t a = keys[i], b = keys[ixj];
          const bool up = (i & k) == 0;
          if ((a > b) == up) { keys[i] = b; keys[ixj] = a; }
        }
      }
      __syncthreads();
    }
  }
}

// One workgroup per row, n <= kSortMax.
// mode 0: plain top-k (non-finite scores rank as -inf), mode 1: position 0 forced first.
__global__ __launch_bounds__(256) void topk_sort_kernel(const float* __restrict__ scores, long n,
                                                        long stride, long k, int descending,
                                                        int force_first, int nonfinite_to_neginf,
                                                        int sorted_ascending, long* __restrict__ out) {
  __shared__ uint64_t keys[kSortMax];
  __shared__ int flags[kSortMax];
  __shared__ int wave_tot[4];
  const long row = blockIdx.x;
  const float* s = scores + row * stride;
  int npad = 1;
  while (npad < n) npad <<= 1;
  for (int i = threadIdx.x; i < npad; i += 256) {
    uint64_t key = ~0ull;  // padding sorts last
    if (i < n) {
      float v = s[i];
      if (nonfinite_to_neginf && !(fabsf(v) <= 3.402823466e38f)) v = -INFINITY;
      key = make_key(v, (uint32_t)i, descending != 0);
      if (force_first && i == 0) key = 0ull;
    }
    keys[i] = key;
    flags[i] = 0;
  }
  __syncthreads();
  bitonic_sort(keys, npad);
  if (!sorted_ascending) {
    for (int i = threadIdx.x; i < k; i += 256) out[row * k + i] = (long)(keys[i] & 0xffffffffu);
    return;
  }
  for (int i = threadIdx.x; i < k; i += 256) flags[(int)(keys[i] & 0xffffffffu)] = 1;
  __syncthreads();
  // ordered compaction of the flagged indices: each thread owns a contiguous span
  const int span = npad / 256 > 0 ? npad / 256 : 1;
  const int begin = threadIdx.x * span;
  int cnt = 0;
  for (int i = begin; i < begin + span && i < npad; ++i) cnt += flags[i];
  // exclusive scan of cnt over the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(incl, o, 64);
    if (lane >= o) incl += v;
  }
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  int base = incl - cnt;
  for (int w = 0; w < wave; ++w) base += wave_tot[w];
  for (int i = begin; i < begin + span && i < npad; ++i)
    if (flags[i]) out[row * k + base++] = i;
}

// Radix select for long rows (n up to 65536): finds the k-th best 32-bit key, then keeps all
// better keys and the lowest-index ties.  Output ascending by index.  One workgroup per row.
template <bool CACHED>  // CACHED: n <= 2048, every thread keeps the keys of its span in registers
__global__ __launch_bounds__(256) void topk_radix_kernel(const float* __restrict__ scores, long n,
                                                         long stride, long k, int descending,
                                                         int force_first, int nonfinite_to_neginf,
                                                         long* __restrict__ out) {
  __shared__ int hist[256];
  __shared__ uint32_t s_prefix;
  __shared__ int s_need;
  __shared__ int wave_tot[4][2];
  const long row = blockIdx.x;
  const float* s = scores + row * stride;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  auto key_of = [&](long i) -> uint32_t {
    float v = s[i];
    if (nonfinite_to_neginf && !(fabsf(v) <= 3.402823466e38f)) v = -INFINITY;
    const uint32_t o = float_ord(v);
    uint32_t kk = descending ? ~o : o;  // smaller = better
    if (force_first && i == 0) kk = 0u;
    return kk;
  };
  // note: with force_first the forced element shares key 0 only with scores that map to 0,
  // i.e. +NaN in descending order; index order still puts position 0 first.
  // Every thread owns a contiguous span of indices (the output is in index order).
  const long span = CACHED ? 8 : (n + 255) / 256;
  const long begin = threadIdx.x * span;
  long end = begin + span;
  end = end < n ? end : n;
  uint32_t ck[8];
  if (CACHED) {
#pragma unroll
    for (int u = 0; u < 8; ++u) ck[u] = begin + u < n ? key_of(begin + u) : 0xffffffffu;
  }
  if (threadIdx.x == 0) { s_prefix = 0u; s_need = (int)k; }
  __syncthreads();
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    hist[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t prefix = s_prefix;
    const int need = s_need;
    const uint32_t pmask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    if (CACHED) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (begin + u < n && (ck[u] & pmask) == prefix) atomicAdd(&hist[(ck[u] >> shift) & 255], 1);
    } else {
      for (long i = threadIdx.x; i < n; i += 256) {
        const uint32_t kk = key_of(i);
        if ((kk & pmask) == prefix) atomicAdd(&hist[(kk >> shift) & 255], 1);
      }
    }
    __syncthreads();
    // the bin that holds the need-th smallest key: inclusive scan of the 256 bins, one per thread
    const int mine = hist[threadIdx.x];
    int incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int v = __shfl_up(incl, o, 64);
      if (lane >= o) incl += v;
    }
    if (lane == 63) wave_tot[wave][0] = incl;
    __syncthreads();
    for (int w = 0; w < wave; ++w) incl += wave_tot[w][0];
    if (incl >= need && incl - mine < need) {  // exactly one thread
      s_need = need - (incl - mine);
      s_prefix = prefix | ((uint32_t)threadIdx.x << shift);
    }
    __syncthreads();
  }
  const uint32_t kth = s_prefix;  // key of the k-th best element
  const int need_eq = s_need;     // how many elements equal to kth are kept (lowest indices)
  int c_lt = 0, c_eq = 0;
  if (CACHED) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (begin + u < n) { c_lt += ck[u] < kth; c_eq += ck[u] == kth; }
  } else {
    for (long i = begin; i < end; ++i) {
      const uint32_t kk = key_of(i);
      c_lt += kk < kth;
      c_eq += kk == kth;
    }
  }
  int i_lt = c_lt, i_eq = c_eq;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int a = __shfl_up(i_lt, o, 64), b = __shfl_up(i_eq, o, 64);
    if (lane >= o) { i_lt += a; i_eq += b; }
  }
  if (lane == 63) { wave_tot[wave][0] = i_lt; wave_tot[wave][1] = i_eq; }
  __syncthreads();
  int b_lt = i_lt - c_lt, b_eq = i_eq - c_eq;
  for (int w = 0; w < wave; ++w) { b_lt += wave_tot[w][0]; b_eq += wave_tot[w][1]; }
  // position in the output = (#kept with lower index)
  auto place = [&](long i, uint32_t kk) {
    const int eq_kept_before = b_eq < need_eq ? b_eq : need_eq;
    if (kk < kth) {
      out[row * k + b_lt + eq_kept_before] = i;
      ++b_lt;
    } else if (kk == kth) {
      if (b_eq < need_eq) out[row * k + b_lt + b_eq] = i;
      ++b_eq;
    }
  };
  if (CACHED) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (begin + u < n) place(begin + u, ck[u]);
  } else {
    for (long i = begin; i < end; ++i) place(i, key_of(i));
  }
}

// ---------------------------------------------------------------------------------------
// column sums of probabilities: out[c, g, k] = sum_{h in group g} ( sum_q p[c, h, q, k] )
// inner sums run over q in index order, then heads in index order (fixed, reproducible).
// ---------------------------------------------------------------------------------------
// One workgroup = (chunk, block of CB key columns).  Its 256 threads form 256/CB head slots x CB
// columns; a thread adds the query rows of a head in index order for its column (a row of CB columns is
// one contiguous segment), then the heads of a group are added in index order from LDS.  The summation
// order depends on nothing but the indices, so the result is reproducible bit for bit.  Narrow column
// blocks are used when there are few chunks, so that the grid still fills the chip.
template <int CB>
__global__ __launch_bounds__(256) void evict_colsum_kernel(const float* __restrict__ probs, long n_heads,
                                                           long n_q, long n_keys, long hpg,
                                                           float* __restrict__ out) {
  constexpr int NH = 256 / CB;
  extern __shared__ float head_sum[];  // [n_heads][CB]
  const long chunk = blockIdx.y;
  const int c = threadIdx.x % CB;
  const int sub = threadIdx.x / CB;
  const long col = (long)blockIdx.x * CB + c;
  const float* base = probs + chunk * n_heads * n_q * n_keys;
  for (long hd = sub; hd < n_heads; hd += NH) {
    float acc = 0.f;
    if (col < n_keys) {
      const float* p = base + hd * n_q * n_keys + col;
      long q = 0;
      for (; q + 16 <= n_q; q += 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = p[(q + u) * n_keys];
#pragma unroll
        for (int u = 0; u < 16; ++u) acc += v[u];
      }
      for (; q < n_q; ++q) acc += p[q * n_keys];
    }
    head_sum[hd * CB + c] = acc;
  }
  __syncthreads();
  const long n_groups = n_heads / hpg;
  for (long g = sub; g < n_groups; g += NH) {
    float acc = 0.f;
    for (long hh = 0; hh < hpg; ++hh) acc += head_sum[(g * hpg + hh) * CB + c];
    if (col < n_keys) out[(chunk * n_groups + g) * n_keys + col] = acc;
  }
}

// The same sums in two launches for few chunks: a workgroup owns one head and a contiguous range of
// columns, so that every query row contributes one long contiguous segment (the narrow column blocks
// above touch 128 bytes per row and keep few DRAM pages open); the per-head sums go to a workspace and
// a second kernel adds the heads of a group in index order.  Same order of additions, same bits.
constexpr int kHeadsumCols = 4;  // columns per thread at most
// NCOL columns per thread (c0 + t + 256 j); a thread past the end of the range reads the range's last column again
// and does not store.  No branch around a load: with one per load the kernel was bound by instruction issue.
// The row's base address is uniform (scalar registers), the column a 32-bit byte offset per lane.
template <int NCOL>
__global__ __launch_bounds__(256) void evict_headsum_kernel(const float* __restrict__ probs, long n_heads, long n_q,
                                                            long n_keys, long width, float* __restrict__ hsum) {
  const long chunk = blockIdx.z, head = blockIdx.y;
  const long c0 = (long)blockIdx.x * width;
  long c1 = c0 + width;
  c1 = c1 < n_keys ? c1 : n_keys;
  const char* p = reinterpret_cast<const char*>(probs + (chunk * n_heads + head) * n_q * n_keys + c0);
  const unsigned last = (unsigned)(c1 - c0 - 1);
  const long row_bytes = n_keys * 4;
  float acc[NCOL];
  unsigned off[NCOL];
#pragma unroll
  for (int j = 0; j < NCOL; ++j) {
    acc[j] = 0.f;
    const unsigned c = threadIdx.x + 256u * j;
    off[j] = (c < last ? c : last) * 4u;
  }
  long q = 0;
  constexpr int R = 8;  // rows in flight (16: no faster)
  for (; q + R <= n_q; q += R) {
    float v[R][NCOL];
#pragma unroll
    for (int u = 0; u < R; ++u)
#pragma unroll
      for (int j = 0; j < NCOL; ++j) v[u][j] = *reinterpret_cast<const float*>(p + (q + u) * row_bytes + off[j]);
#pragma unroll
    for (int u = 0; u < R; ++u)
#pragma unroll
      for (int j = 0; j < NCOL; ++j) acc[j] += v[u][j];
  }
  for (; q < n_q; ++q)
#pragma unroll
    for (int j = 0; j < NCOL; ++j) acc[j] += *reinterpret_cast<const float*>(p + q * row_bytes + off[j]);
#pragma unroll
  for (int j = 0; j < NCOL; ++j) {
    const long c = c0 + threadIdx.x + 256L * j;
    if (c < c1) hsum[(chunk * n_heads + head) * n_keys + c] = acc[j];
  }
}

// Column ranges and launch of evict_headsum_kernel: enough workgroups for two per compute unit where the shape has
// them, ranges of at most 256 * kHeadsumCols columns.
static int launch_headsum(const float* probs, long n_chunks, long n_heads, long n_queries, long n_keys, float* hsum,
                          hipStream_t st) {
  long parts = (512 + n_heads * n_chunks - 1) / (n_heads * n_chunks);
  const long min_parts = (n_keys + 256 * kHeadsumCols - 1) / (256 * kHeadsumCols);
  parts = parts < min_parts ? min_parts : parts;
  const long width = (n_keys + parts - 1) / parts;
  parts = (n_keys + width - 1) / width;
  const dim3 grid((unsigned)parts, (unsigned)n_heads, (unsigned)n_chunks);
  switch ((width + 255) / 256) {
    case 1: hipLaunchKernelGGL(evict_headsum_kernel<1>, grid, dim3(256), 0, st, probs, n_heads, n_queries, n_keys, width, hsum); break;
    case 2: hipLaunchKernelGGL(evict_headsum_kernel<2>, grid, dim3(256), 0, st, probs, n_heads, n_queries, n_keys, width, hsum); break;
    case 3: hipLaunchKernelGGL(evict_headsum_kernel<3>, grid, dim3(256), 0, st, probs, n_heads, n_queries, n_keys, width, hsum); break;
    default: hipLaunchKernelGGL(evict_headsum_kernel<4>, grid, dim3(256), 0, st, probs, n_heads, n_queries, n_keys, width, hsum); break;
  }
  return launch_status();
}

__global__ __launch_bounds__(256) void evict_groupsum_kernel(const float* __restrict__ hsum, long n_heads, long hpg,
                                                             long n_keys, float* __restrict__ out) {
  const long chunk = blockIdx.z, g = blockIdx.y;
  const long c = (long)blockIdx.x * 256 + threadIdx.x;
  if (c >= n_keys) return;
  const long n_groups = n_heads / hpg;
  const float* src = hsum + (chunk * n_heads + g * hpg) * n_keys + c;
  float acc = 0.f;
  long hh = 0;
  for (; hh + 8 <= hpg; hh += 8) {  // eight loads in flight, added in head order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[(hh + u) * n_keys];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  for (; hh < hpg; ++hh) acc += src[hh * n_keys];
  out[(chunk * n_groups + g) * n_keys + c] = acc;
}


// Sum over the heads of a group and the keep set of the row in one launch: evict_groupsum_kernel followed by
// topk_radix_kernel<true> with position 0 forced first, for rows of at most 2048 keys.  One workgroup of 1024
// threads per (chunk, group): thread t owns keys t and t + 1024, adds their per-head sums in head order (the same
// additions as evict_groupsum_kernel: the scores it writes are the same bits), keeps the two 32-bit keys in
// registers and finds the k-th best key by four 8-bit radix passes over a histogram in LDS.  A segment of 1024
// consecutive keys is laid over the threads in index order, so the position of a kept key in the ascending output is a
// count over wave ballots.
constexpr int kSelThreads = 1024;
__global__ __launch_bounds__(kSelThreads) void evict_groupsum_select_kernel(
    const float* __restrict__ hsum, long n_heads, long hpg, long n_keys, long k, int descending, int force_first,
    float* __restrict__ scores, long* __restrict__ out) {
  __shared__ int hist[256];
  __shared__ int scan_tot[4];
  __shared__ uint32_t s_prefix;
  __shared__ int s_need;
  __shared__ int seg_lt[2][16], seg_eq[2][16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;
  const long n_groups = n_heads / hpg;
  const long chunk = row / n_groups, g = row - chunk * n_groups;
  uint32_t key[2];
  bool valid[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const long c = tid + 1024L * u;
    valid[u] = c < n_keys;
    key[u] = 0xffffffffu;
    if (valid[u]) {
      const float* src = hsum + (chunk * n_heads + g * hpg) * n_keys + c;
      float acc = 0.f;
      long hh = 0;
      // batches of 32, 28, 16, 8, 4, 2, 1 loads in flight (a group of 28 or 32 heads: one round trip), added in
      // head order
      auto batch = [&](auto n_tag) __attribute__((always_inline)) {
        constexpr int N = decltype(n_tag)::value;
        float v[N];
#pragma unroll
        for (int x = 0; x < N; ++x) v[x] = src[(hh + x) * n_keys];
#pragma unroll
        for (int x = 0; x < N; ++x) acc += v[x];
        hh += N;
      };
      while (hh + 32 <= hpg) batch(std::integral_constant<int, 32>{});
      if (hh + 28 <= hpg) batch(std::integral_constant<int, 28>{});
      if (hh + 16 <= hpg) batch(std::integral_constant<int, 16>{});
      if (hh + 8 <= hpg) batch(std::integral_constant<int, 8>{});
      if (hh + 4 <= hpg) batch(std::integral_constant<int, 4>{});
      if (hh + 2 <= hpg) batch(std::integral_constant<int, 2>{});
      if (hh < hpg) batch(std::integral_constant<int, 1>{});
      scores[row * n_keys + c] = acc;
      const uint32_t o = float_ord(acc);
      key[u] = descending ? ~o : o;  // smaller = better
      if (force_first && c == 0) key[u] = 0u;
    }
  }
  if (tid == 0) { s_prefix = 0u; s_need = (int)k; }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t prefix = s_prefix;
    const int need = s_need;
    const uint32_t pmask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (valid[u] && (key[u] & pmask) == prefix) atomicAdd(&hist[(key[u] >> shift) & 255], 1);
    }
    __syncthreads();
    // the bin that holds the need-th smallest key: inclusive scan of the 256 bins by the first four waves
    int mine = 0, incl = 0;
    if (tid < 256) {
      mine = hist[tid];
      incl = mine;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int v = __shfl_up(incl, o, 64);
        if (lane >= o) incl += v;
      }
      if (lane == 63) scan_tot[wave] = incl;
    }
    __syncthreads();
    if (tid < 256) {
      for (int w = 0; w < wave; ++w) incl += scan_tot[w];
      if (incl >= need && incl - mine < need) {  // exactly one thread
        s_need = need - (incl - mine);
        s_prefix = prefix | ((uint32_t)tid << shift);
      }
    }
    __syncthreads();
  }
  const uint32_t kth = s_prefix;  // key of the k-th best element
  const int need_eq = s_need;     // how many elements equal to kth are kept (lowest indices)
  bool lt[2], eq[2];
  int p_lt[2], p_eq[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    lt[u] = valid[u] && key[u] < kth;
    eq[u] = valid[u] && key[u] == kth;
    const unsigned long b_lt = __builtin_amdgcn_ballot_w64(lt[u]), b_eq = __builtin_amdgcn_ballot_w64(eq[u]);
    const unsigned long below = (1ul << lane) - 1ul;
    p_lt[u] = __builtin_popcountl(b_lt & below);
    p_eq[u] = __builtin_popcountl(b_eq & below);
    if (lane == 0) { seg_lt[u][wave] = __builtin_popcountl(b_lt); seg_eq[u][wave] = __builtin_popcountl(b_eq); }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    if (!lt[u] && !eq[u]) continue;
    int b_lt = p_lt[u], b_eq = p_eq[u];  // kept-candidates with a lower index
    for (int uu = 0; uu <= u; ++uu) {
      const int wn = uu < u ? 16 : wave;
      for (int w = 0; w < wn; ++w) { b_lt += seg_lt[uu][w]; b_eq += seg_eq[uu][w]; }
    }
    const long c = tid + 1024L * u;
    if (lt[u]) out[row * k + b_lt + (b_eq < need_eq ? b_eq : need_eq)] = c;
    else if (b_eq < need_eq) out[row * k + b_lt + b_eq] = c;
  }
}

// votes[idx[i]] += 1 for every index inside [0, length); the counts are integers, so the order of the
// additions does not matter
__global__ __launch_bounds__(256) void vote_histogram_kernel(const long* __restrict__ idx, long n, long length,
                                                             float* __restrict__ votes) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const long t = idx[i];
  if (t >= 0 && t < length) atomicAdd(votes + t, 1.f);
}

// ---------------------------------------------------------------------------------------
// query-to-chunk eviction scorer from q / k (bf16), fp32 math
// ---------------------------------------------------------------------------------------
// pass 1: one workgroup per (q-head, query row): softmax max and denominator over visible keys
__global__ __launch_bounds__(256) void evict_maxden_kernel(const __bf16* __restrict__ q,
                                                           const __bf16* __restrict__ k, long prefix_len,
                                                           long chunk_len, long query_len, int Hq, int Hkv,
                                                           int d, float scale, int causal,
                                                           float* __restrict__ mx, float* __restrict__ den) {
  __shared__ float qrow[256];
  __shared__ float red_m[4], red_s[4];
  const int head = blockIdx.x, qi = blockIdx.y;
  const int kvh = head / (Hq / Hkv);
  const long row = prefix_len + chunk_len + qi;
  const long key_len = prefix_len + chunk_len + query_len;
  for (int i = threadIdx.x; i < d; i += 256) qrow[i] = (float)q[(row * Hq + head) * d + i];
  __syncthreads();
  const long last = causal ? row : key_len - 1;
  float m = -INFINITY, s = 0.f;
  for (long j = threadIdx.x; j <= last; j += 256) {
    const __bf16* kp = k + (j * Hkv + kvh) * d;
    float acc = 0.f;
    for (int i = 0; i < d; ++i) acc += (float)kp[i] * qrow[i];
    const float x = acc * scale;
    if (x > m) { s = s * __expf(m - x) + 1.f; m = x; }
    else s += __expf(x - m);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(m, o, 64), os = __shfl_xor(s, o, 64);
    const float mm = fmaxf(m, om);
    s = (m == -INFINITY ? 0.f : s * __expf(m - mm)) + (om == -INFINITY ? 0.f : os * __expf(om - mm));
    m = mm;
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { red_m[wave] = m; red_s[wave] = s; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float M = red_m[0], S = red_s[0];
    for (int w = 1; w < 4; ++w) {
      const float mm = fmaxf(M, red_m[w]);
      S = (M == -INFINITY ? 0.f : S * __expf(M - mm)) + (red_m[w] == -INFINITY ? 0.f : red_s[w] * __expf(red_m[w] - mm));
      M = mm;
    }
    mx[head * query_len + qi] = M;
    den[head * query_len + qi] = S;
  }
}

// pass 2: one thread per (q-head, chunk column): sum over the query rows in index order
__global__ __launch_bounds__(64) void evict_chunk_scores_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k, const float* __restrict__ mx,
    const float* __restrict__ den, long prefix_len, long chunk_len, long query_len, int Hq, int Hkv, int d,
    float scale, int reduce_mean, float* __restrict__ out) {
  extern __shared__ float qs[];  // [query_len][d]
  const int head = blockIdx.x;
  const int kvh = head / (Hq / Hkv);
  const long c = (long)blockIdx.y * 64 + threadIdx.x;
  const long qrow0 = prefix_len + chunk_len;
  for (long i = threadIdx.x; i < query_len * d; i += 64) {
    const long qi = i / d, e = i - qi * d;
    qs[i] = (float)q[((qrow0 + qi) * Hq + head) * d + e];
  }
  __syncthreads();
  if (c >= chunk_len) return;
  const __bf16* kp = k + ((prefix_len + c) * Hkv + kvh) * d;
  float acc = 0.f;
  for (long qi = 0; qi < query_len; ++qi) {
    float dot = 0.f;
    for (int e = 0; e < d; ++e) dot += (float)kp[e] * qs[qi * d + e];
    // chunk columns precede every query row, so they are visible under a causal mask too
    acc += __expf(dot * scale - mx[head * query_len + qi]) / den[head * query_len + qi];
  }
  out[(long)head * chunk_len + c] = reduce_mean ? acc / (float)query_len : acc;
}

// pooling (max / avg, stride 1, padding kernel/2) then mean over groups of heads
__global__ __launch_bounds__(256) void pool_group_kernel(const float* __restrict__ scores, long n_heads,
                                                         long n, int pool, int kernel, long hpg,
                                                         float* __restrict__ out) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  const long g = blockIdx.y;
  if (i >= n) return;
  const int pad = kernel / 2;
  float acc = 0.f;
  for (long hh = 0; hh < hpg; ++hh) {
    const float* s = scores + (g * hpg + hh) * n;
    float v;
    if (pool == 0) {
      v = s[i];
    } else if (pool == 1) {
      v = -INFINITY;
      for (int w = 0; w < kernel; ++w) {
        const long j = i - pad + w;
        if (j >= 0 && j < n) v = fmaxf(v, s[j]);
      }
    } else {
      float t = 0.f;
      for (int w = 0; w < kernel; ++w) {
        const long j = i - pad + w;
        if (j >= 0 && j < n) t += s[j];
      }
      v = t / (float)kernel;
    }
    acc += v;
  }
  out[g * n + i] = hpg > 1 ? acc / (float)hpg : acc;
}

int evict_score_qk_scalar(const void* q, const void* k, int64_t prefix_len, int64_t chunk_len, int64_t query_len,
                          int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, float scale, int32_t reduce_mean,
                          int32_t causal, float* workspace, float* out, hipStream_t stream);

static int topk_launch(const float* scores, int64_t n_rows, int64_t n, int64_t stride, int64_t k,
                       int descending, int force_first, int nonfinite, int sorted_ascending,
                       int64_t* out, hipStream_t stream) {
  if (!scores || !out) return PDLLM_ERR_NULL;
  if (n_rows < 0 || n <= 0 || k < 0 || k > n || stride < n || n > 65536) return PDLLM_ERR_SHAPE;
  if (n_rows == 0 || k == 0) return PDLLM_OK;
  if (n_rows > 0x7fffffffL) return PDLLM_ERR_SHAPE;
  // an ascending index set only needs the k-th key (radix select); the full sort is for rank order
  if (n <= kSortMax && (!sorted_ascending || n <= 256)) {
    hipLaunchKernelGGL(topk_sort_kernel, dim3((unsigned)n_rows), dim3(256), 0, stream, scores, (long)n,
                       (long)stride, (long)k, descending, force_first, nonfinite, sorted_ascending,
                       reinterpret_cast<long*>(out));
  } else {
    if (!sorted_ascending) return PDLLM_ERR_UNSUPPORTED;
    if (n <= 2048)
      hipLaunchKernelGGL(topk_radix_kernel<true>, dim3((unsigned)n_rows), dim3(256), 0, stream, scores, (long)n,
                         (long)stride, (long)k, descending, force_first, nonfinite, reinterpret_cast<long*>(out));
    else
      hipLaunchKernelGGL(topk_radix_kernel<false>, dim3((unsigned)n_rows), dim3(256), 0, stream, scores, (long)n,
                         (long)stride, (long)k, descending, force_first, nonfinite, reinterpret_cast<long*>(out));
  }
  return launch_status();
}

}  // namespace pdllm

using namespace pdllm;

extern "C" int pdllm_topk_lowest_index(const float* scores, int64_t n_rows, int64_t n,
                                       int64_t scores_stride, int64_t k, int32_t sorted_ascending,
                                       int64_t* indices_out, pdllm_stream_t stream) {
  return topk_launch(scores, n_rows, n, scores_stride, k, 1, 0, 1, sorted_ascending, indices_out,
                     static_cast<hipStream_t>(stream));
}

extern "C" int pdllm_topb_keep_bos(const float* scores, int64_t n_rows, int64_t chunk_len,
                                   int64_t scores_stride, int64_t capacity, int32_t keep_high,
                                   int32_t force_keep_first, int64_t* indices_out,
                                   pdllm_stream_t stream) {
  if (chunk_len <= 0) return PDLLM_ERR_SHAPE;
  int64_t keep = capacity < 1 ? 1 : capacity;
  if (keep > chunk_len) keep = chunk_len;
  return topk_launch(scores, n_rows, chunk_len, scores_stride, keep, keep_high ? 1 : 0,
                     force_keep_first ? 1 : 0, 0, 1, indices_out, static_cast<hipStream_t>(stream));
}

extern "C" int64_t pdllm_evict_colsum_workspace_bytes(int64_t n_chunks, int64_t n_heads, int64_t n_keys) {
  if (n_chunks < 0 || n_heads <= 0 || n_keys <= 0) return PDLLM_ERR_SHAPE;
  return n_chunks * n_heads * n_keys * 4;
}

extern "C" int pdllm_evict_colsum(const float* probs, int64_t n_chunks, int64_t n_heads,
                                  int64_t n_queries, int64_t n_keys, int64_t heads_per_group,
                                  void* workspace, int64_t workspace_bytes, float* scores_out,
                                  pdllm_stream_t stream) {
  if (!probs || !scores_out) return PDLLM_ERR_NULL;
  if (n_chunks < 0 || n_heads <= 0 || n_queries <= 0 || n_keys <= 0 || heads_per_group <= 0 ||
      n_heads % heads_per_group)
    return PDLLM_ERR_SHAPE;
  if (n_chunks == 0) return PDLLM_OK;
  if (n_chunks > 65535 || n_heads * 64 * 4 > 64 * 1024) return PDLLM_ERR_UNSUPPORTED;
  const size_t lds = (size_t)(n_heads * 64 * 4);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const long blocks64 = (n_keys + 63) / 64 * n_chunks;
  if (workspace != nullptr && blocks64 < 1024 && n_heads <= 65535) {
    // few chunks: one workgroup per (chunk, head, column range), per-head sums through the workspace
    if (workspace_bytes < n_chunks * n_heads * n_keys * 4 || ((uintptr_t)workspace % 4)) return PDLLM_ERR_WORKSPACE;
    float* hsum = static_cast<float*>(workspace);
    int rc = launch_headsum(probs, n_chunks, n_heads, n_queries, n_keys, hsum, st);
    if (rc != PDLLM_OK) return rc;
    hipLaunchKernelGGL(evict_groupsum_kernel,
                       dim3((unsigned)((n_keys + 255) / 256), (unsigned)(n_heads / heads_per_group), (unsigned)n_chunks),
                       dim3(256), 0, st, hsum, (long)n_heads, (long)heads_per_group, (long)n_keys, scores_out);
    return launch_status();
  }
  if (blocks64 >= 1024) {
    hipLaunchKernelGGL(evict_colsum_kernel<64>, dim3((unsigned)((n_keys + 63) / 64), (unsigned)n_chunks), dim3(256),
                       lds, st, probs, (long)n_heads, (long)n_queries, (long)n_keys, (long)heads_per_group, scores_out);
  } else if (blocks64 >= 128) {
    hipLaunchKernelGGL(evict_colsum_kernel<32>, dim3((unsigned)((n_keys + 31) / 32), (unsigned)n_chunks), dim3(256),
                       lds, st, probs, (long)n_heads, (long)n_queries, (long)n_keys, (long)heads_per_group, scores_out);
  } else {
    hipLaunchKernelGGL(evict_colsum_kernel<16>, dim3((unsigned)((n_keys + 15) / 16), (unsigned)n_chunks), dim3(256),
                       lds, st, probs, (long)n_heads, (long)n_queries, (long)n_keys, (long)heads_per_group, scores_out);
  }
  return launch_status();
}

extern "C" int pdllm_evict_keep_from_probs(const float* probs, int64_t n_chunks, int64_t n_heads, int64_t n_queries,
                                           int64_t n_keys, int64_t heads_per_group, int64_t capacity,
                                           int32_t keep_high, int32_t force_keep_first, void* workspace,
                                           int64_t workspace_bytes, float* scores_out, int64_t* indices_out,
                                           pdllm_stream_t stream) {
  if (!probs || !scores_out || !indices_out) return PDLLM_ERR_NULL;
  if (n_chunks < 0 || n_heads <= 0 || n_queries <= 0 || n_keys <= 0 || heads_per_group <= 0 ||
      n_heads % heads_per_group)
    return PDLLM_ERR_SHAPE;
  if (n_chunks == 0) return PDLLM_OK;
  const int64_t n_groups = n_heads / heads_per_group;
  int64_t keep = capacity < 1 ? 1 : capacity;
  if (keep > n_keys) keep = n_keys;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const long blocks64 = (n_keys + 63) / 64 * n_chunks;
  const bool two_launches = workspace != nullptr && blocks64 < 1024 && n_heads <= 65535 && n_chunks <= 65535 &&
                            n_keys <= 2 * kSelThreads && n_chunks * n_groups <= 0x7fffffffL;
  if (!two_launches) {
    const int rc = pdllm_evict_colsum(probs, n_chunks, n_heads, n_queries, n_keys, heads_per_group, workspace,
                                      workspace_bytes, scores_out, stream);
    if (rc != PDLLM_OK) return rc;
    return pdllm_topb_keep_bos(scores_out, n_chunks * n_groups, n_keys, n_keys, capacity, keep_high,
                               force_keep_first, indices_out, stream);
  }
  if (workspace_bytes < n_chunks * n_heads * n_keys * 4 || ((uintptr_t)workspace % 4)) return PDLLM_ERR_WORKSPACE;
  float* hsum = static_cast<float*>(workspace);
  const int rc = launch_headsum(probs, n_chunks, n_heads, n_queries, n_keys, hsum, st);
  if (rc != PDLLM_OK) return rc;
  hipLaunchKernelGGL(evict_groupsum_select_kernel, dim3((unsigned)(n_chunks * n_groups)), dim3(kSelThreads), 0, st,
                     hsum, (long)n_heads, (long)heads_per_group, (long)n_keys, (long)keep, keep_high ? 1 : 0,
                     force_keep_first ? 1 : 0, scores_out, reinterpret_cast<long*>(indices_out));
  return launch_status();
}

// The eviction scorer on the vector unit, any head dim up to 256 (pdllm_evict_score_qk in evict_qk.hip takes
// head dim 128 to the matrix cores and everything else here).  workspace: 2 * Hq * query_len floats; the
// arguments have been checked.
int pdllm::evict_score_qk_scalar(const void* q, const void* k, int64_t prefix_len, int64_t chunk_len,
                                 int64_t query_len, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                 float scale, int32_t reduce_mean, int32_t causal, float* workspace, float* out,
                                 hipStream_t st) {
  float* mx = workspace;
  float* den = workspace + (int64_t)num_q_heads * query_len;
  hipLaunchKernelGGL(evict_maxden_kernel, dim3((unsigned)num_q_heads, (unsigned)query_len), dim3(256), 0, st,
                     static_cast<const __bf16*>(q), static_cast<const __bf16*>(k), (long)prefix_len,
                     (long)chunk_len, (long)query_len, num_q_heads, num_kv_heads, head_dim, scale, causal,
                     mx, den);
  int rc = launch_status();
  if (rc != PDLLM_OK) return rc;
  hipLaunchKernelGGL(evict_chunk_scores_kernel,
                     dim3((unsigned)num_q_heads, (unsigned)((chunk_len + 63) / 64)), dim3(64),
                     (size_t)(query_len * head_dim * 4), st, static_cast<const __bf16*>(q),
                     static_cast<const __bf16*>(k), mx, den, (long)prefix_len, (long)chunk_len,
                     (long)query_len, num_q_heads, num_kv_heads, head_dim, scale, reduce_mean, out);
  return launch_status();
}

extern "C" int pdllm_token_score_pool_group(const float* scores, int64_t n_heads, int64_t n, int32_t pool,
                                            int32_t kernel, int64_t heads_per_group, float* out,
                                            pdllm_stream_t stream) {
  if (!scores || !out) return PDLLM_ERR_NULL;
  if (n_heads <= 0 || n <= 0 || heads_per_group <= 0 || n_heads % heads_per_group) return PDLLM_ERR_SHAPE;
  if (pool < 0 || pool > 2) return PDLLM_ERR_DTYPE;
  if (pool != 0 && kernel < 1) return PDLLM_ERR_SHAPE;
  const long groups = n_heads / heads_per_group;
  if (groups > 65535) return PDLLM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(pool_group_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)groups), dim3(256), 0,
                     static_cast<hipStream_t>(stream), scores, (long)n_heads, (long)n, pool, kernel,
                     (long)heads_per_group, out);
  return launch_status();
}

extern "C" int pdllm_vote_histogram(const int64_t* indices, int64_t n, int64_t length, float* votes,
                                    pdllm_stream_t stream) {
  if (!indices || !votes) return PDLLM_ERR_NULL;
  if (n < 0 || length <= 0 || length >= (1l << 24)) return PDLLM_ERR_SHAPE;  // counts stay exact in fp32
  if (n == 0) return PDLLM_OK;
  hipLaunchKernelGGL(vote_histogram_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), reinterpret_cast<const long*>(indices), (long)n, (long)length,
                     votes);
  return launch_status();
}
