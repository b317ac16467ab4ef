// Sparse-prefix attention for gfx950 (MI355X): the active block (query + masked
// response rows) attends to the selected, non-contiguous chunk KV pages and to itself.
//
// Replaces load_kvcache + flex/SDPA attention and _fwd_kernel_d2f of the reference
// (layers/attention/attention_v4.py:368-397, layers/attention/ops/prefix_prefill.py:25-230)
// and, with a causal mask and no cached prefix, the block-diagonal chunk prefill
// (attention_v4.py:336-367).
//
// Work decomposition
//   One workgroup (4 wavefronts) = one (request, KV head, row group, KV split).
//   A row group is J blocks of 32 "rows"; a row is one (query token, q-head of the GQA
//   group) pair, ordered token-major, so all G q-heads of a KV head reuse every K/V tile.
//   With J >= 4 wave w owns row block w ("slot A") for all keys.  The remaining blocks
//   ("slot B") are split over waves INSIDE every 128-key tile, so that all waves do the same
//   amount of MFMA work per tile: J=5 -> block 4, wave w takes key block w of each tile;
//   J=6 -> blocks 4,5, two key blocks per wave; J=8 -> a second full block per wave.
//   J=1,2 have only shared blocks (intra-workgroup split-KV for short active blocks).
//   Slot B issues its MFMAs on the operand fragments slot A has just read, so it adds no
//   LDS traffic; shared blocks are merged through LDS with a log-sum-exp reduction.
//   An optional split over workgroups writes fp32 partials + LSE to a workspace that
//   attn_merge_kernel reduces.
//
// Per 128-key tile
//   K and V rows are copied HBM -> LDS by global_load_lds (16 bytes per lane, no registers);
//   the row addresses come from a slot table that 128 threads resolve through the page table
//   two tiles ahead.  Rows are 256 bytes = 16 chunks; chunk c of row r is stored at position
//   c ^ rotl4(r & 15), which makes the 128-bit K operand reads and the transposing
//   ds_read_b64_tr_b16 V operand reads bank-conflict free.
//   S^T = K Q^T and O^T += V^T P^T use v_mfma_f32_32x32x16_bf16; in the S^T accumulator
//   layout a lane holds 16 keys of one query, so softmax statistics are lane-local plus
//   one half-wave exchange, and P^T feeds the second MFMA straight from registers.  The
//   running maximum is only advanced (and O rescaled) when a tile exceeds it by more than
//   2^8, which removes most rescale work without changing the result.
//   fp8 e4m3 pages are dequantised (x * scale[page]) in registers while staging.

#include <type_traits>

#include "pdllm_common.h"

namespace pdllm {

int kv_store_launch(const void* key, const void* value, void* k_cache, void* v_cache,
                    const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                    int64_t key_stride, int64_t value_stride, int64_t n_slots, hipStream_t stream);

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int kD = 128;          // head dim
constexpr int kKT = 128;         // keys per tile
constexpr int kThreads = 256;    // 4 wavefronts
constexpr int kRowBytes = 256;   // one K or V row in LDS
constexpr int kTileBytes = kKT * kRowBytes;      // 32768
constexpr int kBufBytes = 2 * kTileBytes;        // K tile + V tile
constexpr int kMainBytes = 2 * kBufBytes;        // double buffered: 131072
constexpr int kPartStride = 33;                  // floats per d-row of an LDS partial
constexpr int kPartBytes = kD * kPartStride * 4; // 16896
constexpr int kMaxRanges = 128;
constexpr int kMaxTok = 264;                     // query tokens a row group of 256 rows can touch (+ slack)
constexpr float kRescaleSlack = 8.f;             // log2 units
static_assert(4 * kPartBytes <= kMainBytes, "partials must fit the tile buffers");

struct AttnKParams {
  const __bf16* q;
  const __bf16* k_new;
  const __bf16* v_new;
  __bf16* out;
  const void* k_cache;
  const void* v_cache;
  const float* k_scale;
  const float* v_scale;
  const int* block_table;
  const int* q_start_loc;
  const int* range_ptr;
  const int* range_start;
  const int* range_len;
  const uint8_t* mask;
  float* ws_o;
  float* ws_lse;
  long q_stride, kn_stride, vn_stride, o_stride;
  long cache_page_stride, cache_token_stride, cache_head_stride;
  long mask_stride;
  long n_tokens;
  int n_pages;
  int bt_stride;
  int scale_page_stride, scale_head_stride;
  int n_req, Hq, Hkv, G;
  int page_shift;
  int mask_mode;
  int J;
  int row_tiles;
  int num_splits;
  int max_q_len;
  float scale_log2;  // sm_scale * log2(e)
};

// combine lane l with lane l ^ 32: v_permlane32_swap exchanges the upper half of its first
// operand with the lower half of its second, so swapping a value with itself yields
// {lower half in every lane, upper half in every lane}
__device__ __forceinline__ float half_swap_max(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// position swizzle of the 16 chunks of a row: rotate the low 4 row bits left by one
__device__ __forceinline__ int swz(int row) {
  const int r = row & 15;
  return ((r & 7) << 1) | (r >> 3);
}

// 8 e4m3 values (two dwords) * scale -> 8 bf16 (four dwords)
__device__ __forceinline__ uint4 dequant_fp8x8(uint32_t lo, uint32_t hi, float scale) {
  f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false);
  f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
  f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
  f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
  uint4 r;
  r.x = pack_bf16x2(a[0] * scale, a[1] * scale);
  r.y = pack_bf16x2(b[0] * scale, b[1] * scale);
  r.z = pack_bf16x2(c[0] * scale, c[1] * scale);
  r.w = pack_bf16x2(d[0] * scale, d[1] * scale);
  return r;
}

// Softmax update of one row block over NKB key blocks of 32 keys (S holds raw scores in the
// S^T accumulator layout: element i of a lane is key 8*(i/4) + 4*h + i%4 of the block).
// generic (wave-uniform): keys >= lim_tile (per lane: tile bound and causal bound) and keys whose
// bit in mrow[key block] is clear are masked out.
template <int NKB>
__device__ __forceinline__ void softmax_update(f32x16 (&S)[NKB], bf16x8 (&P)[NKB][2], f32x16 (&O)[4],
                                               float& M, float& l, float c, int h, int kb_first, bool generic,
                                               int lim_tile, const uint32_t* mrow) {
  if (generic) {
#pragma unroll
    for (int b = 0; b < NKB; ++b) {
      const int lim = lim_tile - 32 * (kb_first + b);
      uint32_t W = lim >= 32 ? 0xffffffffu : (lim <= 0 ? 0u : ((1u << lim) - 1u));
      if (mrow != nullptr) W &= mrow[kb_first + b];
      W >>= 4 * h;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        constexpr uint32_t one = 1u;
        const uint32_t bit = one << (8 * (i >> 2) + (i & 3));
        S[b][i] = (W & bit) ? S[b][i] : -INFINITY;
      }
    }
  }
  float mx = S[0][0];
#pragma unroll
  for (int b = 0; b < NKB; ++b)
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, S[b][i]);
  mx = half_swap_max(mx) * c;  // scaled to log2 units (c > 0)
  // advance the reference maximum only when some row of the wave needs it
  const bool need = mx > M + kRescaleSlack || (M == -INFINITY && mx > -INFINITY);
  if (__builtin_amdgcn_ballot_w64(need) != 0) {
    const float Mn = fmaxf(M, mx);
    const float alpha = (Mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(M - Mn);  // M = -inf -> 0
    M = Mn;
    l *= alpha;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
      for (int i = 0; i < 16; ++i) O[db][i] *= alpha;
      __builtin_amdgcn_sched_barrier(0);  // one accumulator block at a time through the VALU registers
    }
  }
  const float Muse = (M == -INFINITY) ? 0.f : M;
  float psum = 0.f;
#pragma unroll
  for (int b = 0; b < NKB; ++b) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(S[b][i], c, -Muse));
      S[b][i] = pv;
      psum += pv;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) P[b][j][e] = (__bf16)S[b][8 * j + e];
  }
  l += psum;
}

template <int KV_FP8, int J>
__global__ __launch_bounds__(kThreads) void attn_fwd_kernel(const AttnKParams p) {
  constexpr bool HAS_A = J >= 4;
  constexpr int NB = (J == 1 || J == 5) ? 1 : (J == 2 || J == 6) ? 2 : (J == 8) ? 4 : 0;
  constexpr int NBA = NB > 0 ? NB : 1;  // array extents must be positive
  constexpr int GS = (J == 1 || J == 5) ? 4 : (J == 2 || J == 6) ? 2 : 1;  // waves sharing a B block

  __shared__ __attribute__((aligned(1024))) char lds[kMainBytes];
  __shared__ float s_ml[4][2][32];
  __shared__ int s_cum[kMaxRanges + 1];
  __shared__ int s_start[kMaxRanges];
  __shared__ int s_len[kMaxRanges];
  __shared__ unsigned s_koff[3][kKT];  // row offsets of a tile's keys in 16-byte units (K and V source)
  __shared__ unsigned s_voff[3][kKT];
  __shared__ int s_page[KV_FP8 ? 3 : 1][KV_FP8 ? kKT : 1];  // fp8: page of each key (scale lookup)
  __shared__ uint32_t s_maskbits[2][kMaxTok][4];  // dense mask of an active tile, one bit per key

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int h = lane >> 5;

  int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int row_tile = lid % p.row_tiles;
  lid /= p.row_tiles;
  const int split = lid % p.num_splits;
  lid /= p.num_splits;
  const int kvh = lid % p.Hkv;
  const int req = lid / p.Hkv;

  const int G = p.G;
  const int q0 = p.q_start_loc[req];
  const int Sq = p.q_start_loc[req + 1] - q0;
  if (q0 < 0 || Sq <= 0 || (long)q0 + Sq > p.n_tokens || Sq > p.max_q_len) return;
  const int rows = Sq * G;
  const int row0 = row_tile * 32 * J;
  if (row0 >= rows) return;

  // ---- visible prefix ranges of this request -> cumulative key counts in LDS ----
  int nr = 0;
  if (p.k_cache != nullptr && p.range_ptr != nullptr) {
    const int r0 = p.range_ptr[req];
    nr = p.range_ptr[req + 1] - r0;
    nr = nr < 0 ? 0 : (nr > kMaxRanges ? kMaxRanges : nr);
    if (tid < nr) {
      const int len = p.range_len[r0 + tid];
      s_len[tid] = len > 0 ? len : 0;
      s_start[tid] = p.range_start[r0 + tid];
    }
  }
  __syncthreads();
  if (tid <= nr) {
    int cc = 0;
    for (int i = 0; i < tid; ++i) cc += s_len[i];
    s_cum[tid] = cc;
  }
  __syncthreads();
  const int ctx_total = s_cum[nr];

  const int Tc = (ctx_total + kKT - 1) / kKT;
  int Sa = Sq;
  if (p.mask_mode == PDLLM_MASK_CAUSAL) {
    const int last_row = (row0 + 32 * J < rows ? row0 + 32 * J : rows) - 1;
    const int lim = last_row / G + 1;
    Sa = lim < Sq ? lim : Sq;
  }
  const int Ta = (Sa + kKT - 1) / kKT;
  const int T = Tc + Ta;
  const int tps = (T + p.num_splits - 1) / p.num_splits;
  const int T0 = split * tps < T ? split * tps : T;
  const int T1 = T0 + tps < T ? T0 + tps : T;

  // ---- row blocks of this wave ----
  const int blkA = wave;
  int blkB = -1, kb0 = 0, gi = 0;
  if (J == 1) { blkB = 0; kb0 = wave; gi = wave; }
  else if (J == 2) { blkB = wave >> 1; kb0 = 2 * (wave & 1); gi = wave & 1; }
  else if (J == 5) { blkB = 4; kb0 = wave; gi = wave; }
  else if (J == 6) { blkB = 4 + (wave >> 1); kb0 = 2 * (wave & 1); gi = wave & 1; }
  else if (J == 8) { blkB = 4 + wave; }
  const int bmask = ((1 << NB) - 1) << kb0;  // key blocks of a tile this wave handles for slot B

  // ---- Q fragments (B operand of S^T = K Q^T), rows of this lane ----
  bf16x8 QA[8], QB[8];
  int srowA = 0, srowB = 0, ridxA = -1, ridxB = -1;
  auto load_q = [&](int blk, bf16x8 (&Q)[8], int& srow, int& ridx) __attribute__((always_inline)) {
    const int r = row0 + 32 * blk + l32;
    const bool valid = blk >= 0 && r < rows;
    const int rr = valid ? r : 0;
    const int tq = rr / G;
    const int g = rr - tq * G;
    srow = tq;
    ridx = valid ? r : -1;
    const __bf16* qp = p.q + (long)(q0 + tq) * p.q_stride + (long)(kvh * G + g) * kD + 8 * h;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      if (valid) {
        Q[ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) Q[ks][e] = (__bf16)0.f;
      }
    }
  };
  if (HAS_A) load_q(blkA, QA, srowA, ridxA);
  if (NB > 0) load_q(blkB, QB, srowB, ridxB);

  f32x16 OA[4], OB[4];
  float MA = -INFINITY, MB = -INFINITY, lA = 0.f, lB = 0.f;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { OA[db][i] = 0.f; OB[db][i] = 0.f; }

  // ---- per-lane LDS operand offsets (bytes inside a tile) ----
  int koff[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) koff[ks] = l32 * kRowBytes + (((2 * ks + h) ^ swz(l32)) << 4);
  int voff[2][4];
  {
    const int i16 = lane & 15, g4 = l32 >> 4;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int keyrow = 4 * h + 8 * r + (i16 >> 2);
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const int cg = 4 * db + 2 * g4 + ((i16 & 3) >> 1);
        voff[r][db] = keyrow * kRowBytes + ((cg ^ swz(keyrow)) << 4) + ((i16 & 1) << 3);
      }
    }
  }

  // ---- slot table: logical key of a tile -> cache slot (or active row), resolved by 128 threads ----
  // Two phases so that the page-table load is in flight while the tile is computed:
  // resolve_begin finds the logical token and issues the load, resolve_end publishes the slot.
  const int page_mask = (1 << p.page_shift) - 1;
  int rp = 0;
  int rs_page = 0, rs_low = 0;
  auto resolve_begin = [&](int t) __attribute__((always_inline)) {
    if (tid >= kKT) return;
    if (t < Tc) {
      int v = t * kKT + tid;
      if (v >= ctx_total) v = t * kKT;  // padding rows copy the first (always valid) row; they are masked
      if (v < s_cum[rp]) rp = 0;
      while (v >= s_cum[rp + 1]) ++rp;
      const int tok = s_start[rp] + (v - s_cum[rp]);
      int pi = tok >> p.page_shift;
      pi = pi < 0 ? 0 : (pi >= p.bt_stride ? p.bt_stride - 1 : pi);
      rs_page = p.block_table[(long)req * p.bt_stride + pi];
      rs_low = tok & page_mask;
    } else {
      const int a = (t - Tc) * kKT + tid;
      rs_page = -1;
      rs_low = a < Sa ? a : (t - Tc) * kKT;
    }
  };
  const long cache_row_bytes = p.cache_token_stride * (KV_FP8 ? 1 : 2);
  auto resolve_end = [&](int t, int sb) __attribute__((always_inline)) {
    if (tid >= kKT) return;
    if (t < Tc) {
      int page = rs_page;
      page = page < 0 ? 0 : (page >= p.n_pages ? p.n_pages - 1 : page);  // never read out of bounds
      const long slot = ((long)page << p.page_shift) + rs_low;
      const unsigned off = (unsigned)((slot * cache_row_bytes) >> 4);
      s_koff[sb][tid] = off;
      s_voff[sb][tid] = off;
      if (KV_FP8) s_page[sb][tid] = page;
    } else {
      s_koff[sb][tid] = (unsigned)(((long)rs_low * p.kn_stride * 2) >> 4);
      s_voff[sb][tid] = (unsigned)(((long)rs_low * p.vn_stride * 2) >> 4);
    }
  };

  // dense mask of active tile t -> bit rows in LDS (built one tile ahead, like the slot table)
  const uint8_t* mask_base = p.mask != nullptr ? p.mask + (long)q0 * p.mask_stride + q0 : nullptr;
  const int tq_first = row0 / G;
  int ntok = ((row0 + 32 * J < rows ? row0 + 32 * J : rows) - 1) / G - tq_first + 1;
  ntok = ntok < kMaxTok ? ntok : kMaxTok;
  auto build_mask = [&](int t, int par) __attribute__((always_inline)) {
    if (p.mask_mode != PDLLM_MASK_DENSE || t < Tc) return;
    const int a0 = (t - Tc) * kKT;
    for (int idx = tid; idx < ntok * 4; idx += kThreads) {
      const int tok = idx >> 2, w = idx & 3;
      const uint8_t* mp = mask_base + (long)(tq_first + tok) * p.mask_stride + a0 + 32 * w;
      uint32_t bits = 0;
      for (int j = 0; j < 32; ++j)
        if (a0 + 32 * w + j < Sq && mp[j] != 0) bits |= 1u << j;
      s_maskbits[par][tok][w] = bits;
    }
  };

  // fp8 staging registers (only used by the fp8 instantiations)
  uint2 st_k[8], st_v[8];
  float st_ks[8], st_vs[8];

  // issue the copy of tile t into buffer `buf`: rows 4*ii + lane/16 for ii = i*4 + wave.
  // The chunk a lane fetches, (lane & 15) ^ swz(row), does not depend on i because 16 | 16*i.
  const int lane_row = 4 * wave + (lane >> 4);
  const int lane_ch = (lane & 15) ^ swz(lane_row);
  const long cache_lane_off = ((long)kvh * p.cache_head_stride + 8 * lane_ch) * (KV_FP8 ? 1 : 2);
  const char* kc_lane = static_cast<const char*>(p.k_cache) + cache_lane_off;
  const char* vc_lane = static_cast<const char*>(p.v_cache) + cache_lane_off;
  const char* kn_lane = reinterpret_cast<const char*>(p.k_new + (long)q0 * p.kn_stride + kvh * kD + 8 * lane_ch);
  const char* vn_lane = reinterpret_cast<const char*>(p.v_new + (long)q0 * p.vn_stride + kvh * kD + 8 * lane_ch);
  // Tile copy = 16 wave-level instructions (8 row groups x {K, V}).  They are handed out one at a
  // time between the MFMAs of the tile before, so that the memory pipeline never blocks the wave.
  unsigned dma_ko[8], dma_vo[8];
  const char* dma_kb = nullptr;
  const char* dma_vb = nullptr;
  char* dma_dst = nullptr;
  bool dma_on = false, dma_fp8 = false;
  int dma_sb = 0;
  auto dma_begin = [&](int t, int sb, int buf, bool on) __attribute__((always_inline)) {
    dma_on = on;
    const bool ctx = t < Tc;
    dma_fp8 = KV_FP8 && ctx;
    dma_sb = sb;
    dma_kb = ctx ? kc_lane : kn_lane;
    dma_vb = ctx ? vc_lane : vn_lane;
    dma_dst = lds + buf * kBufBytes + wave * 1024;
  };
  // load the source offsets of row groups [I0, I1) from the slot table
  auto dma_offsets = [&](auto i0_tag, auto i1_tag) __attribute__((always_inline)) {
    constexpr int I0 = decltype(i0_tag)::value, I1 = decltype(i1_tag)::value;
    if (!dma_on) return;
#pragma unroll
    for (int i = I0; i < I1; ++i) {
      dma_ko[i] = s_koff[dma_sb][16 * i + lane_row];
      dma_vo[i] = s_voff[dma_sb][16 * i + lane_row];
    }
  };
  // issue instruction `k` of the tile copy: row group k / 2, K (even k) or V (odd k)
  auto dma_one = [&](auto k_tag) __attribute__((always_inline)) {
    constexpr int K = decltype(k_tag)::value;
    constexpr int i = K >> 1;
    if (!dma_on) return;
    if (KV_FP8 && dma_fp8) {
      if (K & 1) {
        st_v[i] = *reinterpret_cast<const uint2*>(dma_vb + ((unsigned long)dma_vo[i] << 4));
      } else {
        st_k[i] = *reinterpret_cast<const uint2*>(dma_kb + ((unsigned long)dma_ko[i] << 4));
        const long so = (long)s_page[KV_FP8 ? dma_sb : 0][KV_FP8 ? 16 * i + lane_row : 0] * p.scale_page_stride +
                        (long)kvh * p.scale_head_stride;
        st_ks[i] = p.k_scale[so];
        st_vs[i] = p.v_scale[so];
      }
    } else if (K & 1) {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(dma_vb + ((unsigned long)dma_vo[i] << 4)),
          (__attribute__((address_space(3))) void*)(dma_dst + i * 4096 + kTileBytes), 16, 0, 0);
    } else {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(dma_kb + ((unsigned long)dma_ko[i] << 4)),
          (__attribute__((address_space(3))) void*)(dma_dst + i * 4096), 16, 0, 0);
    }
  };
  auto dma_all = [&]() __attribute__((always_inline)) {
#define PDLLM_DMA(K) dma_one(std::integral_constant<int, K>{})
    PDLLM_DMA(0); PDLLM_DMA(1); PDLLM_DMA(2); PDLLM_DMA(3); PDLLM_DMA(4); PDLLM_DMA(5); PDLLM_DMA(6); PDLLM_DMA(7);
    PDLLM_DMA(8); PDLLM_DMA(9); PDLLM_DMA(10); PDLLM_DMA(11); PDLLM_DMA(12); PDLLM_DMA(13); PDLLM_DMA(14);
    PDLLM_DMA(15);
#undef PDLLM_DMA
  };
  // fp8: dequantise the staged rows into the LDS tile (same layout the direct copies produce)
  auto finish_tile = [&](int t, int buf) __attribute__((always_inline)) {
    if (KV_FP8 && t < Tc) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int ii = i * 4 + wave;
        char* kdst = lds + buf * kBufBytes + ii * 1024 + lane * 16;
        *reinterpret_cast<uint4*>(kdst) = dequant_fp8x8(st_k[i].x, st_k[i].y, st_ks[i]);
        *reinterpret_cast<uint4*>(kdst + kTileBytes) = dequant_fp8x8(st_v[i].x, st_v[i].y, st_vs[i]);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct-to-LDS copies have landed
  };

  const float c = p.scale_log2;

  // ---- one pass: row block(s) x NKB key blocks of the tile in LDS ----
  // DUAL: slot B uses the same key blocks and rides on the operand fragments slot A reads.
  // Operand reads run two steps ahead of the MFMAs; the scheduling barriers keep that order.
  // dma_tag: first tile-copy instruction this pass hands out (8 per two-key-block pass), or 16 = none
  auto pass = [&](bool generic, auto nkb_tag, auto dual_tag, auto dma_tag, bool forA, int kb_first, int bufoff,
                  int nvalid, bool active, int a0, int par) __attribute__((always_inline)) {
    constexpr int DMA0 = decltype(dma_tag)::value;
    if constexpr (DMA0 < 16) dma_offsets(std::integral_constant<int, DMA0 / 2>{},
                                         std::integral_constant<int, DMA0 / 2 + 4>{});
    constexpr int NKB = decltype(nkb_tag)::value;
    constexpr bool DUAL = decltype(dual_tag)::value;
    const int kbase_bytes = bufoff + kb_first * 32 * kRowBytes;
    const int vbase_bytes = kbase_bytes + kTileBytes;
    bf16x8 (&Q1)[8] = forA ? QA : QB;
    f32x16 (&O1)[4] = forA ? OA : OB;
    float& M1 = forA ? MA : MB;
    float& l1 = forA ? lA : lB;
    const int srow1 = forA ? srowA : srowB;

    f32x16 S1[NKB], S2[DUAL ? NKB : 1];
#pragma unroll
    for (int b = 0; b < NKB; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        S1[b][i] = 0.f;
        if constexpr (DUAL) S2[b][i] = 0.f;
      }
    {
      auto ldk = [&](int stp) __attribute__((always_inline)) {
        const int kb = stp >> 3, ks = stp & 7;
        return *reinterpret_cast<const bf16x8*>(lds + koff[ks] + kbase_bytes + kb * 32 * kRowBytes);
      };
      bf16x8 kf[2];
      kf[0] = ldk(0);
      kf[1] = ldk(1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int stp = 0; stp < 8 * NKB; ++stp) {
        const int kb = stp >> 3, ks = stp & 7;
        const bf16x8 cur = kf[stp & 1];
        S1[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur, Q1[ks], S1[kb], 0, 0, 0);
        if constexpr (DUAL) S2[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur, QB[ks], S2[kb], 0, 0, 0);
        if (stp + 2 < 8 * NKB) kf[stp & 1] = ldk(stp + 2);
        if constexpr (DMA0 < 16 && NKB == 2) {
          if (stp == 1) dma_one(std::integral_constant<int, DMA0 + 0>{});
          if (stp == 5) dma_one(std::integral_constant<int, DMA0 + 1>{});
          if (stp == 9) dma_one(std::integral_constant<int, DMA0 + 2>{});
          if (stp == 13) dma_one(std::integral_constant<int, DMA0 + 3>{});
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    bf16x8 P1[NKB][2], P2[DUAL ? NKB : 1][2];
    const bool causal_here = active && p.mask_mode == PDLLM_MASK_CAUSAL;
    const bool dense_here = active && p.mask_mode == PDLLM_MASK_DENSE;
    {
      int lim = nvalid;
      if (causal_here) { const int cl = srow1 - a0 + 1; lim = cl < lim ? cl : lim; }
      int tl = srow1 - tq_first;
      tl = tl < 0 ? 0 : (tl >= kMaxTok ? kMaxTok - 1 : tl);
      softmax_update<NKB>(S1, P1, O1, M1, l1, c, h, kb_first, generic, lim,
                          dense_here ? &s_maskbits[par][tl][0] : nullptr);
    }
    if constexpr (DUAL) {
      int lim = nvalid;
      if (causal_here) { const int cl = srowB - a0 + 1; lim = cl < lim ? cl : lim; }
      int tl = srowB - tq_first;
      tl = tl < 0 ? 0 : (tl >= kMaxTok ? kMaxTok - 1 : tl);
      softmax_update<NKB>(S2, P2, OB, MB, lB, c, h, kb_first, generic, lim,
                          dense_here ? &s_maskbits[par][tl][0] : nullptr);
    }
    __builtin_amdgcn_sched_barrier(0);
    {
      typedef __attribute__((ext_vector_type(8))) short s16x8;
      // step = (kb, j, db): V^T fragment of keys 32 kb + 16 j .. +16, columns 32 db .. +32
      auto ldv = [&](int stp, int r) __attribute__((always_inline)) {
        const int db = stp & 3, kj = stp >> 2;
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s16x4*)(lds + voff[r][db] + vbase_bytes + kj * 16 * kRowBytes));
      };
      s16x4 lo[2], hi[2];
      lo[0] = ldv(0, 0); hi[0] = ldv(0, 1);
      lo[1] = ldv(1, 0); hi[1] = ldv(1, 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int stp = 0; stp < 8 * NKB; ++stp) {
        const int db = stp & 3, kj = stp >> 2;
        const s16x4 a = lo[stp & 1], b2 = hi[stp & 1];
        const s16x8 both = {a[0], a[1], a[2], a[3], b2[0], b2[1], b2[2], b2[3]};
        const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
        O1[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, P1[kj >> 1][kj & 1], O1[db], 0, 0, 0);
        if constexpr (DUAL) OB[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, P2[kj >> 1][kj & 1], OB[db], 0, 0, 0);
        if (stp + 2 < 8 * NKB) { lo[stp & 1] = ldv(stp + 2, 0); hi[stp & 1] = ldv(stp + 2, 1); }
        if constexpr (DMA0 < 16 && NKB == 2) {
          if (stp == 1) dma_one(std::integral_constant<int, DMA0 + 4>{});
          if (stp == 5) dma_one(std::integral_constant<int, DMA0 + 5>{});
          if (stp == 9) dma_one(std::integral_constant<int, DMA0 + 6>{});
          if (stp == 13) dma_one(std::integral_constant<int, DMA0 + 7>{});
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  using I0 = std::integral_constant<int, 0>;
  using I8 = std::integral_constant<int, 8>;
  using I16 = std::integral_constant<int, 16>;
  auto compute = [&](bool gen_tag, int t, int buf, bool has_next, int sb_next) __attribute__((always_inline)) {
    const int bufoff = buf * kBufBytes;
    const bool active = t >= Tc;
    const int a0 = active ? (t - Tc) * kKT : 0;
    int nvalid = active ? Sa - a0 : ctx_total - t * kKT;
    nvalid = nvalid < kKT ? nvalid : kKT;
    using N1 = std::integral_constant<int, 1>;
    using N2 = std::integral_constant<int, 2>;
    using Dual = std::integral_constant<bool, NB == 4>;
    using Single = std::integral_constant<bool, false>;
    if (has_next) {
      // the whole copy of the next tile is issued up front (the copy instructions are scheduling
      // boundaries; spreading them through the MFMA loops measured slower)
      dma_begin(t + 1, sb_next, buf ^ 1, true);
      dma_offsets(I0{}, I8{});
      dma_all();
    }
    if (HAS_A) {
      pass(gen_tag, N2{}, Dual{}, I16{}, true, 0, bufoff, nvalid, active, a0, buf);
      pass(gen_tag, N2{}, Dual{}, I16{}, true, 2, bufoff, nvalid, active, a0, buf);
    }
    if (NB == 1) pass(gen_tag, N1{}, Single{}, I16{}, false, kb0, bufoff, nvalid, active, a0, buf);
    if (NB == 2) pass(gen_tag, N2{}, Single{}, I16{}, false, kb0, bufoff, nvalid, active, a0, buf);
  };

  auto step = [&](int t) __attribute__((always_inline)) {
    const int rel = t - T0;
    const int buf = rel & 1;
    if (t + 2 < T1) resolve_begin(t + 2);
    if (t + 1 < T1) build_mask(t + 1, buf ^ 1);
    const bool active = t >= Tc;
    const int a0 = active ? (t - Tc) * kKT : 0;
    const int nv = active ? Sa - a0 : ctx_total - t * kKT;
    const bool generic = nv < kKT || (active && p.mask_mode != PDLLM_MASK_FULL);
    compute(generic, t, buf, t + 1 < T1, (rel + 1) % 3);
    if (t + 2 < T1) resolve_end(t + 2, (rel + 2) % 3);
    if (t + 1 < T1) finish_tile(t + 1, buf ^ 1);
    __syncthreads();
  };

  if (T0 < T1) {
    resolve_begin(T0);
    resolve_end(T0, 0);
    if (T0 + 1 < T1) { resolve_begin(T0 + 1); resolve_end(T0 + 1, 1); }
    __syncthreads();
    dma_begin(T0, 0, 0, true);
    dma_offsets(I0{}, I8{});
    dma_all();
    build_mask(T0, 0);
    finish_tile(T0, 0);
    __syncthreads();
    for (int t = T0; t < T1; ++t) step(t);
  }

  // ---- epilogue ----
  auto emit = [&](int ridx, int db, const f32x16& o, float mfin, float lfin) __attribute__((always_inline)) {
    if (ridx < 0) return;
    const int tq = ridx / G;
    const int g = ridx - tq * G;
    const float inv = lfin > 0.f ? 1.f / lfin : 0.f;
    if (p.num_splits == 1) {
      __bf16* op = p.out + (long)(q0 + tq) * p.o_stride + (long)(kvh * G + g) * kD + 32 * db + 4 * h;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        uint2 w;
        w.x = pack_bf16x2(o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv);
        w.y = pack_bf16x2(o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv);
        *reinterpret_cast<uint2*>(op + 8 * i4) = w;
      }
    } else {
      const long R = ((long)(q0 + tq) * p.Hq + kvh * G + g) * p.num_splits + split;
      float* wp = p.ws_o + R * kD + 32 * db + 4 * h;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        float4 w = {o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv, o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv};
        *reinterpret_cast<float4*>(wp + 8 * i4) = w;
      }
      if (db == 0 && h == 0) p.ws_lse[R] = lfin > 0.f ? mfin + __log2f(lfin) : -INFINITY;  // log2 domain
    }
  };

  if (HAS_A) {
    lA = half_swap_sum(lA);
#pragma unroll
    for (int db = 0; db < 4; ++db) emit(ridxA, db, OA[db], MA, lA);
  }
  if (NB > 0) {
    lB = half_swap_sum(lB);
    if (GS == 1) {
#pragma unroll
      for (int db = 0; db < 4; ++db) emit(ridxB, db, OB[db], MB, lB);
    } else {
      // merge the GS partial results of a shared block through LDS (the tile buffers are free now)
      float* part = reinterpret_cast<float*>(lds) + wave * (kPartBytes / 4);
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int d = 32 * db + 8 * (i >> 2) + 4 * h + (i & 3);
          part[d * kPartStride + l32] = OB[db][i];
        }
      if (h == 0) {
        s_ml[wave][0][l32] = MB;
        s_ml[wave][1][l32] = lB;
      }
      __syncthreads();
      const int wbase = wave - gi;
      float M = -INFINITY;
#pragma unroll
      for (int w = 0; w < GS; ++w) M = fmaxf(M, s_ml[wbase + w][0][l32]);
      const float Muse = (M == -INFINITY) ? 0.f : M;
      float wgt[GS];
      float L = 0.f;
#pragma unroll
      for (int w = 0; w < GS; ++w) {
        wgt[w] = __builtin_amdgcn_exp2f(s_ml[wbase + w][0][l32] - Muse);
        L += wgt[w] * s_ml[wbase + w][1][l32];
      }
      constexpr int NDB = 4 / GS;  // column blocks this wave finishes
#pragma unroll
      for (int dd = 0; dd < NDB; ++dd) {
        const int db = gi * NDB + dd;
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int w = 0; w < GS; ++w) {
          const float* pw = reinterpret_cast<const float*>(lds) + (wbase + w) * (kPartBytes / 4);
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int d = 32 * db + 8 * (i >> 2) + 4 * h + (i & 3);
            acc[i] += wgt[w] * pw[d * kPartStride + l32];
          }
        }
        emit(ridxB, db, acc, M, L);
      }
    }
  }
}

// Reduce the split-KV partials: one wave per (token, q-head) row.
__global__ __launch_bounds__(256) void attn_merge_kernel(const float* __restrict__ ws_o,
                                                         const float* __restrict__ ws_lse,
                                                         __bf16* __restrict__ out, long o_stride,
                                                         const int* __restrict__ q_start_loc,
                                                         int n_req, int max_q_len, int Hq,
                                                         int num_splits, long n_tokens) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const long per_req = (long)max_q_len * Hq;
  if (row >= per_req * n_req) return;
  const int req = (int)(row / per_req);
  const int rem = (int)(row - (long)req * per_req);
  const int tq = rem / Hq;
  const int head = rem - tq * Hq;
  const int q0 = q_start_loc[req];
  const int Sq = q_start_loc[req + 1] - q0;
  if (q0 < 0 || tq >= Sq || (long)q0 + Sq > n_tokens || Sq > max_q_len) return;
  const long R = ((long)(q0 + tq) * Hq + head) * num_splits;
  float M = -INFINITY;
  for (int s = 0; s < num_splits; ++s) M = fmaxf(M, ws_lse[R + s]);
  float2 acc = {0.f, 0.f};
  float L = 0.f;
  if (M > -INFINITY) {
    for (int s = 0; s < num_splits; ++s) {
      const float w = __builtin_amdgcn_exp2f(ws_lse[R + s] - M);
      const float2 o = *reinterpret_cast<const float2*>(ws_o + (R + s) * kD + 2 * lane);
      acc.x += w * o.x;
      acc.y += w * o.y;
      L += w;
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  *reinterpret_cast<uint32_t*>(out + (long)(q0 + tq) * o_stride + (long)head * kD + 2 * lane) =
      pack_bf16x2(acc.x * inv, acc.y * inv);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct AttnPlan {
  int J;
  int num_splits;
  int row_tiles;
};

static int ilog2_exact(int v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

static int validate_desc(const pdllm_attn_desc* d, bool prefill) {
  if (!d) return PDLLM_ERR_NULL;
  if (!d->q || !d->k_new || !d->v_new || !d->out || !d->q_start_loc) return PDLLM_ERR_NULL;
  if (d->head_dim != kD) return PDLLM_ERR_UNSUPPORTED;
  if (d->num_q_heads <= 0 || d->num_kv_heads <= 0 || d->num_q_heads % d->num_kv_heads) return PDLLM_ERR_SHAPE;
  if (d->n_req <= 0 || d->max_q_len <= 0 || d->n_tokens <= 0 || d->max_ctx_len < 0) return PDLLM_ERR_SHAPE;
  if (d->n_tokens > (1ll << 30)) return PDLLM_ERR_SHAPE;
  if (d->n_tokens * (d->kn_stride > d->vn_stride ? d->kn_stride : d->vn_stride) * 2 >= (1ll << 36)) return PDLLM_ERR_SHAPE;
  if (d->mask_mode < PDLLM_MASK_FULL || d->mask_mode > PDLLM_MASK_DENSE) return PDLLM_ERR_DTYPE;
  if (d->mask_mode == PDLLM_MASK_DENSE && (!d->mask || d->mask_stride < d->n_tokens)) return PDLLM_ERR_NULL;
  const int64_t hq = (int64_t)d->num_q_heads * kD, hk = (int64_t)d->num_kv_heads * kD;
  if (d->q_stride < hq || d->o_stride < hq || d->kn_stride < hk || d->vn_stride < hk) return PDLLM_ERR_STRIDE;
  if ((d->q_stride | d->o_stride | d->kn_stride | d->vn_stride) % 8) return PDLLM_ERR_STRIDE;
  if (((uintptr_t)d->q | (uintptr_t)d->k_new | (uintptr_t)d->v_new | (uintptr_t)d->out) % 16) return PDLLM_ERR_STRIDE;
  const bool has_cache = !prefill && d->k_cache != nullptr && d->max_ctx_len > 0;
  if (has_cache) {
    if (!d->v_cache || !d->block_table || !d->range_ptr || !d->range_start || !d->range_len) return PDLLM_ERR_NULL;
    if (d->kv_dtype != PDLLM_KV_BF16 && d->kv_dtype != PDLLM_KV_FP8_E4M3) return PDLLM_ERR_DTYPE;
    if (d->kv_dtype == PDLLM_KV_FP8_E4M3 && (!d->k_scale || !d->v_scale)) return PDLLM_ERR_NULL;
    if (ilog2_exact(d->page_size) < 0) return PDLLM_ERR_SHAPE;
    if (d->n_pages <= 0 || d->n_pages * (int64_t)d->page_size >= (1ll << 31)) return PDLLM_ERR_SHAPE;
    if (d->bt_stride <= 0) return PDLLM_ERR_SHAPE;
    if (d->max_ranges < 0 || d->max_ranges > kMaxRanges) return PDLLM_ERR_UNSUPPORTED;
    const int64_t align = d->kv_dtype == PDLLM_KV_FP8_E4M3 ? 8 : 8;  // 8 elements per lane load
    if (d->cache_head_stride < kD || d->cache_token_stride < hk || d->cache_page_stride < d->cache_token_stride)
      return PDLLM_ERR_STRIDE;
    if ((d->cache_head_stride | d->cache_token_stride | d->cache_page_stride) % align) return PDLLM_ERR_STRIDE;
    {
      const int64_t esz = d->kv_dtype == PDLLM_KV_FP8_E4M3 ? 1 : 2;
      if ((d->cache_token_stride * esz) % 16) return PDLLM_ERR_STRIDE;
      if (d->n_pages * d->cache_page_stride * esz >= (1ll << 36)) return PDLLM_ERR_SHAPE;  // 32-bit offsets of 16 B
    }
    // slots are addressed as slot * token_stride: pages must be laid out back to back
    if (d->cache_page_stride != d->cache_token_stride * d->page_size) return PDLLM_ERR_STRIDE;
    const uintptr_t palign = d->kv_dtype == PDLLM_KV_FP8_E4M3 ? 8 : 16;
    if (((uintptr_t)d->k_cache | (uintptr_t)d->v_cache) % palign) return PDLLM_ERR_STRIDE;
  }
  if (d->num_splits < 0 || d->num_splits > 64) return PDLLM_ERR_SHAPE;
  if (d->rows_per_group != 0) {
    const int j = d->rows_per_group / 32;
    if (d->rows_per_group % 32 || !(j == 1 || j == 2 || j == 4 || j == 5 || j == 6 || j == 8)) return PDLLM_ERR_SHAPE;
  }
  return PDLLM_OK;
}

// Pick the row-group size J and the number of KV splits: minimise the modelled
// makespan (rounds of workgroups over 256 CUs x key tiles x row blocks per wave,
// floored by the cost of staging a tile) plus the HBM cost of split partials.
static AttnPlan make_plan(const pdllm_attn_desc* d, bool prefill) {
  const int G = d->num_q_heads / d->num_kv_heads;
  const long rows = (long)d->max_q_len * G;
  const long nblk = (rows + 31) / 32;
  const long ctx = prefill ? 0 : d->max_ctx_len;
  const long T = (ctx + kKT - 1) / kKT + (d->max_q_len + kKT - 1) / kKT;
  const long units = (long)d->n_req * d->num_kv_heads;
  const int cus = 256;
  static const int js[] = {1, 2, 4, 5, 6, 8};
  AttnPlan best = {4, 1, 1};
  double best_cost = 1e300;
  for (int ji = 0; ji < 6; ++ji) {
    const int J = js[ji];
    if (d->rows_per_group && d->rows_per_group != 32 * J) continue;
    if (!d->rows_per_group && J == 8) continue;  // two full row blocks per wave spill registers: only on request
    const long row_tiles = (nblk + J - 1) / J;
    const int max_splits = prefill ? 1 : 16;
    for (int S = 1; S <= max_splits; ++S) {
      if (d->num_splits && d->num_splits != S) continue;
      if (S > 1 && S > T) break;
      const long wgs = units * row_tiles * S;
      const int per_cu = 1;  // 128 KB of LDS tile buffers: one workgroup per CU
      const double rounds = (double)((wgs + (long)cus * per_cu - 1) / ((long)cus * per_cu));
      const double tiles = (double)((T + S - 1) / S);
      double per_tile = J / 4.0;           // MFMA block-tiles per wave per key tile
      if (per_tile < 0.6) per_tile = 0.6;  // staging / barrier floor
      double cost = rounds * per_cu * tiles * per_tile;
      if (S > 1) {
        // fp32 partial write + read, in units of "key tile of one wave" (~1024 cycles)
        const double part_bytes = (double)units * rows * S * (kD + 1) * 4.0 * 2.0;
        cost += part_bytes / (8e12 / 2.4e9 * 1024.0) + 4.0;
      }
      if (cost < best_cost) {
        best_cost = cost;
        best.J = J;
        best.num_splits = S;
        best.row_tiles = (int)row_tiles;
      }
    }
  }
  return best;
}

static int64_t ws_bytes_for(const pdllm_attn_desc* d, int num_splits) {
  if (num_splits <= 1) return 0;
  const int64_t rows = d->n_tokens * d->num_q_heads;
  return rows * num_splits * (int64_t)(kD + 1) * 4;
}

static int launch_attn(const pdllm_attn_desc* d, bool prefill, hipStream_t stream) {
  int st = validate_desc(d, prefill);
  if (st != PDLLM_OK) return st;
  const AttnPlan plan = make_plan(d, prefill);
  const int64_t need = ws_bytes_for(d, plan.num_splits);
  if (need > 0 && (!d->workspace || d->workspace_bytes < need)) return PDLLM_ERR_WORKSPACE;
  if (need > 0 && ((uintptr_t)d->workspace % 16)) return PDLLM_ERR_STRIDE;

  AttnKParams p;
  p.q = static_cast<const __bf16*>(d->q);
  p.k_new = static_cast<const __bf16*>(d->k_new);
  p.v_new = static_cast<const __bf16*>(d->v_new);
  p.out = static_cast<__bf16*>(d->out);
  const bool has_cache = !prefill && d->k_cache != nullptr && d->max_ctx_len > 0;
  p.k_cache = has_cache ? d->k_cache : nullptr;
  p.v_cache = has_cache ? d->v_cache : nullptr;
  p.k_scale = d->k_scale;
  p.v_scale = d->v_scale;
  p.block_table = d->block_table;
  p.q_start_loc = d->q_start_loc;
  p.range_ptr = has_cache ? d->range_ptr : nullptr;
  p.range_start = d->range_start;
  p.range_len = d->range_len;
  p.mask = d->mask_mode == PDLLM_MASK_DENSE ? d->mask : nullptr;
  const int64_t rows = d->n_tokens * d->num_q_heads;
  p.ws_o = static_cast<float*>(d->workspace);
  p.ws_lse = p.ws_o ? p.ws_o + rows * plan.num_splits * kD : nullptr;
  p.q_stride = d->q_stride; p.kn_stride = d->kn_stride; p.vn_stride = d->vn_stride; p.o_stride = d->o_stride;
  p.cache_page_stride = d->cache_page_stride;
  p.cache_token_stride = d->cache_token_stride;
  p.cache_head_stride = d->cache_head_stride;
  p.mask_stride = d->mask_stride;
  p.n_tokens = d->n_tokens;
  p.n_pages = (int)d->n_pages;
  p.bt_stride = d->bt_stride;
  p.scale_page_stride = d->scale_page_stride;
  p.scale_head_stride = d->scale_head_stride;
  p.n_req = d->n_req; p.Hq = d->num_q_heads; p.Hkv = d->num_kv_heads; p.G = d->num_q_heads / d->num_kv_heads;
  p.page_shift = has_cache ? ilog2_exact(d->page_size) : 0;
  p.mask_mode = d->mask_mode;
  p.J = plan.J;
  p.row_tiles = plan.row_tiles;
  p.num_splits = plan.num_splits;
  p.max_q_len = d->max_q_len;
  p.scale_log2 = d->sm_scale * 1.4426950408889634f;

  const long nblocks = (long)d->n_req * d->num_kv_heads * plan.row_tiles * plan.num_splits;
  if (nblocks <= 0 || nblocks > 0x7fffffffL) return PDLLM_ERR_SHAPE;
  const dim3 grid((unsigned)nblocks), block(kThreads);
  const bool fp8 = has_cache && d->kv_dtype == PDLLM_KV_FP8_E4M3;
#define PDLLM_LAUNCH(JJ)                                                                              \
  do {                                                                                                \
    if (fp8) hipLaunchKernelGGL((attn_fwd_kernel<1, JJ>), grid, block, 0, stream, p);                 \
    else hipLaunchKernelGGL((attn_fwd_kernel<0, JJ>), grid, block, 0, stream, p);                     \
  } while (0)
  switch (plan.J) {
    case 1: PDLLM_LAUNCH(1); break;
    case 2: PDLLM_LAUNCH(2); break;
    case 4: PDLLM_LAUNCH(4); break;
    case 5: PDLLM_LAUNCH(5); break;
    case 6: PDLLM_LAUNCH(6); break;
    case 8: PDLLM_LAUNCH(8); break;
    default: return PDLLM_ERR_SHAPE;
  }
#undef PDLLM_LAUNCH
  st = launch_status();
  if (st != PDLLM_OK) return st;
  if (plan.num_splits > 1) {
    const long mrows = (long)d->n_req * d->max_q_len * d->num_q_heads;
    hipLaunchKernelGGL(attn_merge_kernel, dim3((unsigned)((mrows + 3) / 4)), dim3(256), 0, stream,
                       p.ws_o, p.ws_lse, p.out, p.o_stride, p.q_start_loc, p.n_req, p.max_q_len,
                       p.Hq, p.num_splits, p.n_tokens);
    st = launch_status();
  }
  return st;
}

}  // namespace pdllm

extern "C" int64_t pdllm_attn_workspace_bytes(const pdllm_attn_desc* desc) {
  const int st = pdllm::validate_desc(desc, false);
  if (st != PDLLM_OK) return st;
  return pdllm::ws_bytes_for(desc, pdllm::make_plan(desc, false).num_splits);
}

extern "C" int pdllm_sparse_decode_attn(const pdllm_attn_desc* desc, pdllm_stream_t stream) {
  return pdllm::launch_attn(desc, false, static_cast<hipStream_t>(stream));
}

extern "C" int pdllm_chunk_prefill_attn(const pdllm_attn_desc* desc, const int32_t* slot_mapping,
                                        pdllm_stream_t stream) {
  const int st = pdllm::validate_desc(desc, true);
  if (st != PDLLM_OK) return st;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (slot_mapping != nullptr) {
    // paged store of the chunk K/V rows (bf16 cache, unified layout)
    if (!desc->k_cache || !desc->v_cache) return PDLLM_ERR_NULL;
    if (desc->kv_dtype != PDLLM_KV_BF16) return PDLLM_ERR_UNSUPPORTED;
    const int64_t row = (int64_t)desc->num_kv_heads * desc->head_dim;
    if (desc->cache_token_stride != row || desc->cache_head_stride != desc->head_dim ||
        desc->cache_page_stride != row * desc->page_size)
      return PDLLM_ERR_STRIDE;
    const int rc = pdllm::kv_store_launch(desc->k_new, desc->v_new, const_cast<void*>(desc->k_cache),
                                          const_cast<void*>(desc->v_cache), slot_mapping, desc->n_tokens,
                                          row, desc->kn_stride, desc->vn_stride,
                                          desc->n_pages * (int64_t)desc->page_size, hs);
    if (rc != PDLLM_OK) return rc;
  }
  return pdllm::launch_attn(desc, true, hs);
}

extern "C" int pdllm_attn_plan(const pdllm_attn_desc* desc, int32_t prefill, int32_t* rows_per_group,
                               int32_t* num_splits) {
  const int st = pdllm::validate_desc(desc, prefill != 0);
  if (st != PDLLM_OK) return st;
  const pdllm::AttnPlan plan = pdllm::make_plan(desc, prefill != 0);
  if (rows_per_group) *rows_per_group = 32 * plan.J;
  if (num_splits) *num_splits = plan.num_splits;
  return PDLLM_OK;
}
