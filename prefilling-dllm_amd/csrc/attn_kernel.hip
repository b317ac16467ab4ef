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
//   Wave w owns row block w for all key tiles; with J in {5,6,8} it has a second block:
//   a full one (J=8) or a share of the key tiles of a block that several waves split
//   (J=5: block 4 split four ways, J=6: blocks 4,5 split two ways).  J=1,2 split the key
//   tiles of every block across waves (intra-workgroup split-KV).  Shared blocks are
//   merged through LDS with a log-sum-exp reduction, so the merge costs no HBM traffic.
//   An optional split over workgroups writes fp32 partials + LSE to a workspace that
//   attn_merge_kernel reduces.
//
// Per 64-key tile
//   K/V rows are fetched through the page table with 128-bit loads (the 16 lanes of a
//   quarter-wave cover one 256-byte row), staged in registers one tile ahead (page-table
//   entries two tiles ahead) and written to LDS: K row-major (padded rows), V transposed
//   (d-major, XOR-swizzled) so that both MFMA operands are single 128-bit LDS reads.
//   S^T = K Q^T and O^T += V^T P^T use v_mfma_f32_32x32x16_bf16; in the S^T accumulator
//   layout a lane holds 16 keys of one query, so softmax statistics are lane-local plus
//   one half-wave exchange, and P^T feeds the second MFMA straight from registers.
//   fp8 e4m3 pages are dequantised (x * scale[page]) in registers while staging.

#include "pdllm_common.h"

namespace pdllm {

int kv_store_launch(const void* key, const void* value, void* k_cache, void* v_cache,
                    const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                    int64_t key_stride, int64_t value_stride, int64_t n_slots, hipStream_t stream);

constexpr int kD = 128;          // head dim
constexpr int kKT = 64;          // keys per tile
constexpr int kThreads = 256;    // 4 wavefronts
constexpr int kKsRowBytes = 272; // 128 bf16 + 16 B pad: conflict-free 128-bit row reads
constexpr int kKsBytes = kKT * kKsRowBytes;        // 17408
constexpr int kVtBytes = kD * kKT * 2;             // 16384
constexpr int kBufBytes = kKsBytes + kVtBytes;     // 33792
constexpr int kPartStride = 33;                    // floats per d-row of an LDS partial
constexpr int kPartBytes = kD * kPartStride * 4;   // 16896
constexpr int kMainBytes = 2 * kBufBytes;          // 67584 == 4 * kPartBytes
constexpr int kMaxRanges = 128;
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

struct Slot {
  int blk;     // row block inside the row group
  int t0, t1;  // key tiles this wave processes for the block
  int gs, gi;  // waves sharing the block, index of this wave among them
};

struct Stage {
  uint4 k[4];
  uint4 v[4];
  float ks[4];
  float vs[4];
  bool fp8;
};

__device__ __forceinline__ float half_swap_max(float x) {
  return fmaxf(x, __shfl_xor(x, 32, 64));
}
__device__ __forceinline__ float half_swap_sum(float x) {
  return x + __shfl_xor(x, 32, 64);
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

// One 64-key tile for the row blocks selected by ACT (bit 0: slot 0, bit 1: slot 1).
// GENERIC adds key-validity / causal / dense-mask handling.
template <int NSLOT, int ACT, bool GENERIC>
__device__ __forceinline__ void compute_tile(const char* __restrict__ Ks, const char* __restrict__ Vt,
                                             const bf16x8 (&Q)[NSLOT][8], f32x16 (&O)[NSLOT][4],
                                             float (&m)[NSLOT], float (&l)[NSLOT], float c,
                                             int l32, int h, int nvalid, bool active, int a0,
                                             int mask_mode, const int (&srow)[NSLOT],
                                             const uint8_t* __restrict__ mask_base, long mask_stride) {
  f32x16 S[NSLOT][2];
#pragma unroll
  for (int s = 0; s < NSLOT; ++s)
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) S[s][kb][i] = 0.f;

  // S^T[key, query] = K Q^T.  Operand reads run two steps ahead of the MFMAs; the
  // scheduling barriers keep the compiler from hoisting all 16 reads (register pressure).
  {
    auto ldk = [&](int step) {
      const int ks = step >> 1, kb = step & 1;
      return *reinterpret_cast<const bf16x8*>(Ks + (32 * kb + l32) * kKsRowBytes + (16 * ks + 8 * h) * 2);
    };
    bf16x8 kf[2];
    kf[0] = ldk(0);
    kf[1] = ldk(1);
#pragma unroll
    for (int step = 0; step < 16; ++step) {
      const int ks = step >> 1, kb = step & 1;
      const bf16x8 cur = kf[step & 1];
#pragma unroll
      for (int s = 0; s < NSLOT; ++s)
        if (ACT & (1 << s))
          S[s][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur, Q[s][ks], S[s][kb], 0, 0, 0);
      if (step + 2 < 16) kf[step & 1] = ldk(step + 2);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  bf16x8 P[NSLOT][4];
#pragma unroll
  for (int s = 0; s < NSLOT; ++s) {
    if (!(ACT & (1 << s))) continue;
    if (GENERIC) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int kk = 32 * kb + 8 * (i >> 2) + 4 * h + (i & 3);
          bool vis = kk < nvalid;
          if (active && vis) {
            const int a = a0 + kk;
            if (mask_mode == PDLLM_MASK_CAUSAL) vis = a <= srow[s];
            else if (mask_mode == PDLLM_MASK_DENSE)
              vis = mask_base[(long)srow[s] * mask_stride + a] != 0;
          }
          S[s][kb][i] = vis ? S[s][kb][i] : -INFINITY;
        }
    }
    float mx = S[s][0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, S[s][kb][i]);
    mx = half_swap_max(mx);
    const float m_new = fmaxf(m[s], mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m[s] - m_use) * c);  // m = -inf -> 0
    m[s] = m_new;
    l[s] *= alpha;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[s][db][i] *= alpha;
    const float mc = m_use * c;
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(S[s][kb][i], c, -mc));
        S[s][kb][i] = pv;
        psum += pv;
      }
    l[s] += psum;
#pragma unroll
    for (int j2 = 0; j2 < 4; ++j2) {
      const int kb = j2 >> 1, r0 = 8 * (j2 & 1);
#pragma unroll
      for (int e = 0; e < 8; ++e) P[s][j2][e] = (__bf16)S[s][kb][r0 + e];
    }
  }

  // O^T[d, query] += V^T P^T
  {
    auto ldv = [&](int step) {
      const int j2 = step >> 2, db = step & 3;
      const int d = 32 * db + l32;
      const int g = ((d >> 1) ^ (d >> 3)) & 7;
      return *reinterpret_cast<const bf16x8*>(Vt + d * (kKT * 2) + (((2 * j2 + h) ^ g) << 4));
    };
    bf16x8 vf[2];
    vf[0] = ldv(0);
    vf[1] = ldv(1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int step = 0; step < 16; ++step) {
      const int j2 = step >> 2, db = step & 3;
      const bf16x8 cur = vf[step & 1];
#pragma unroll
      for (int s = 0; s < NSLOT; ++s)
        if (ACT & (1 << s))
          O[s][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur, P[s][j2], O[s][db], 0, 0, 0);
      if (step + 2 < 16) vf[step & 1] = ldv(step + 2);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

template <int KV_FP8, int NSLOT>
__global__ __launch_bounds__(kThreads) void attn_fwd_kernel(const AttnKParams p) {
  __shared__ __attribute__((aligned(16))) char lds[kMainBytes];
  __shared__ float s_ml[4][2][32];
  __shared__ int s_cum[kMaxRanges + 1];
  __shared__ int s_start[kMaxRanges];
  __shared__ int s_len[kMaxRanges];

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
  const int J = p.J;
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
    int c = 0;
    for (int i = 0; i < tid; ++i) c += s_len[i];
    s_cum[tid] = c;
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

  // ---- row-block slots of this wave ----
  Slot slot[2];
  slot[0].blk = wave; slot[0].gs = 1; slot[0].gi = 0;
  slot[1].blk = -1;   slot[1].gs = 1; slot[1].gi = 0;
  if (J == 1) { slot[0].blk = 0; slot[0].gs = 4; slot[0].gi = wave; }
  else if (J == 2) { slot[0].blk = wave >> 1; slot[0].gs = 2; slot[0].gi = wave & 1; }
  else if (J == 5) { slot[1].blk = 4; slot[1].gs = 4; slot[1].gi = wave; }
  else if (J == 6) { slot[1].blk = 4 + (wave >> 1); slot[1].gs = 2; slot[1].gi = wave & 1; }
  else if (J == 8) { slot[1].blk = 4 + wave; }
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int n = T1 - T0;
    const int per = (n + slot[s].gs - 1) / slot[s].gs;
    int t0 = T0 + slot[s].gi * per;
    t0 = t0 < T1 ? t0 : T1;
    int t1 = t0 + per < T1 ? t0 + per : T1;
    if (slot[s].blk < 0 || row0 + 32 * slot[s].blk >= rows) { t0 = T0; t1 = T0; }
    slot[s].t0 = t0;
    slot[s].t1 = t1;
  }

  // ---- Q fragments (B operand of S^T = K Q^T) ----
  bf16x8 Q[NSLOT][8];
  int srow[NSLOT];     // query token index of this lane's row (clamped)
  int rowidx[NSLOT];   // row index inside the request, or -1
#pragma unroll
  for (int s = 0; s < NSLOT; ++s) {
    const int r = row0 + 32 * slot[s].blk + l32;
    const bool valid = slot[s].blk >= 0 && r < rows;
    const int rr = valid ? r : 0;
    const int tq = rr / G;
    const int g = rr - tq * G;
    srow[s] = tq;
    rowidx[s] = valid ? r : -1;
    const __bf16* qp = p.q + (long)(q0 + tq) * p.q_stride + (long)(kvh * G + g) * kD + 8 * h;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      if (valid) {
        Q[s][ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) Q[s][ks][e] = (__bf16)0.f;
      }
    }
  }

  f32x16 O[NSLOT][4];
  float m[NSLOT], l[NSLOT];
#pragma unroll
  for (int s = 0; s < NSLOT; ++s) {
    m[s] = -INFINITY;
    l[s] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[s][db][i] = 0.f;
  }

  // ---- staging roles: thread = (key quad kq, 8-element column group dofs) ----
  const int kq = tid >> 4;
  const int dofs = tid & 15;
  const int page_mask = (1 << p.page_shift) - 1;
  int rp = 0;  // running range pointer of this thread

  auto resolve = [&](int t, int (&idx)[4]) {
    if (t < Tc) {
      const int v0 = t * kKT + 4 * kq;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int v = v0 + j;
        int res = -1;
        if (v < ctx_total) {
          while (v >= s_cum[rp + 1]) ++rp;
          const int tok = s_start[rp] + (v - s_cum[rp]);
          const int pi = tok >> p.page_shift;
          if (tok >= 0 && pi < p.bt_stride) {
            const int page = p.block_table[(long)req * p.bt_stride + pi];
            if (page >= 0 && page < p.n_pages) res = (page << p.page_shift) + (tok & page_mask);
          }
        }
        idx[j] = res;
      }
    } else {
      const int a0 = (t - Tc) * kKT + 4 * kq;
#pragma unroll
      for (int j = 0; j < 4; ++j) idx[j] = (a0 + j < Sa) ? a0 + j : -1;
    }
  };

  auto issue = [&](int t, const int (&idx)[4], Stage& st) {
    const uint4 z = {0u, 0u, 0u, 0u};
    if (t < Tc) {
      st.fp8 = KV_FP8 != 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        st.k[j] = z;
        st.v[j] = z;
        st.ks[j] = 0.f;
        st.vs[j] = 0.f;
        if (idx[j] >= 0) {
          const int page = idx[j] >> p.page_shift;
          const int off = idx[j] & page_mask;
          const long eoff = (long)page * p.cache_page_stride + (long)off * p.cache_token_stride +
                            (long)kvh * p.cache_head_stride + 8 * dofs;
          if (KV_FP8) {
            const uint2 kk = *reinterpret_cast<const uint2*>(static_cast<const char*>(p.k_cache) + eoff);
            const uint2 vv = *reinterpret_cast<const uint2*>(static_cast<const char*>(p.v_cache) + eoff);
            st.k[j].x = kk.x; st.k[j].y = kk.y;
            st.v[j].x = vv.x; st.v[j].y = vv.y;
            const long so = (long)page * p.scale_page_stride + (long)kvh * p.scale_head_stride;
            st.ks[j] = p.k_scale[so];
            st.vs[j] = p.v_scale[so];
          } else {
            st.k[j] = *reinterpret_cast<const uint4*>(static_cast<const __bf16*>(p.k_cache) + eoff);
            st.v[j] = *reinterpret_cast<const uint4*>(static_cast<const __bf16*>(p.v_cache) + eoff);
          }
        }
      }
    } else {
      st.fp8 = false;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        st.k[j] = z;
        st.v[j] = z;
        if (idx[j] >= 0) {
          const long tokrow = (long)(q0 + idx[j]);
          st.k[j] = *reinterpret_cast<const uint4*>(p.k_new + tokrow * p.kn_stride + kvh * kD + 8 * dofs);
          st.v[j] = *reinterpret_cast<const uint4*>(p.v_new + tokrow * p.vn_stride + kvh * kD + 8 * dofs);
        }
      }
    }
  };

  auto write_lds = [&](Stage& st, int buf) {
    char* Ks = lds + buf * kBufBytes;
    char* Vt = Ks + kKsBytes;
    if (KV_FP8 && st.fp8) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        st.k[j] = dequant_fp8x8(st.k[j].x, st.k[j].y, st.ks[j]);
        st.v[j] = dequant_fp8x8(st.v[j].x, st.v[j].y, st.vs[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<uint4*>(Ks + (4 * kq + j) * kKsRowBytes + dofs * 16) = st.k[j];
    // V: 4 keys x 8 d  ->  8 rows (d) x 4 keys.  Key kk of the tile sits in 16-byte slot
    // 2*(kk/16) + ((kk/4)&1) at element 4*((kk%16)/8) + kk%4, which is the order in which
    // the S^T accumulator of the first MFMA presents the keys to the second one.
    const int j2 = kq >> 2, qq = kq & 3;
    const int slot16 = 2 * j2 + (qq & 1);
    const int sub = (qq >> 1) * 8;
    const uint32_t w0[4] = {st.v[0].x, st.v[0].y, st.v[0].z, st.v[0].w};
    const uint32_t w1[4] = {st.v[1].x, st.v[1].y, st.v[1].z, st.v[1].w};
    const uint32_t w2[4] = {st.v[2].x, st.v[2].y, st.v[2].z, st.v[2].w};
    const uint32_t w3[4] = {st.v[3].x, st.v[3].y, st.v[3].z, st.v[3].w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int w = i >> 1;
      uint2 o;
      if (i & 1) {
        o.x = (w0[w] >> 16) | (w1[w] & 0xffff0000u);
        o.y = (w2[w] >> 16) | (w3[w] & 0xffff0000u);
      } else {
        o.x = (w0[w] & 0xffffu) | (w1[w] << 16);
        o.y = (w2[w] & 0xffffu) | (w3[w] << 16);
      }
      const int d = 8 * dofs + i;
      const int g = ((d >> 1) ^ (d >> 3)) & 7;
      *reinterpret_cast<uint2*>(Vt + d * (kKT * 2) + ((slot16 ^ g) << 4) + sub) = o;
    }
  };

  const uint8_t* mask_base =
      p.mask != nullptr ? p.mask + (long)q0 * p.mask_stride + q0 : nullptr;
  const float c = p.scale_log2;

  // ---- main loop over key tiles: loads one tile ahead, page lookups two ahead ----
  if (T0 < T1) {
    Stage st;
    int idx_next[4];
    {
      int idx0[4];
      resolve(T0, idx0);
      issue(T0, idx0, st);
      if (T0 + 1 < T1) resolve(T0 + 1, idx_next);
      write_lds(st, 0);
    }
    __syncthreads();
    for (int t = T0; t < T1; ++t) {
      const int buf = (t - T0) & 1;
      if (t + 1 < T1) {
        issue(t + 1, idx_next, st);
        if (t + 2 < T1) resolve(t + 2, idx_next);
      }
      const char* Ks = lds + buf * kBufBytes;
      const char* Vt = Ks + kKsBytes;
      const bool active = t >= Tc;
      const int a0 = active ? (t - Tc) * kKT : 0;
      int nvalid = active ? Sa - a0 : ctx_total - t * kKT;
      nvalid = nvalid < kKT ? nvalid : kKT;
      const bool generic = nvalid < kKT || (active && p.mask_mode != PDLLM_MASK_FULL);
      const bool a0s = t >= slot[0].t0 && t < slot[0].t1;
      const bool a1s = NSLOT > 1 && t >= slot[1].t0 && t < slot[1].t1;
#define PDLLM_TILE(ACT, GEN)                                                                   \
  compute_tile<NSLOT, ACT, GEN>(Ks, Vt, Q, O, m, l, c, l32, h, nvalid, active, a0, p.mask_mode, \
                                srow, mask_base, p.mask_stride)
      if (NSLOT > 1 && a0s && a1s) {
        if (generic) PDLLM_TILE(3, true); else PDLLM_TILE(3, false);
      } else if (a0s) {
        if (generic) PDLLM_TILE(1, true); else PDLLM_TILE(1, false);
      } else if (NSLOT > 1 && a1s) {
        if (generic) PDLLM_TILE(2, true); else PDLLM_TILE(2, false);
      }
#undef PDLLM_TILE
      if (t + 1 < T1) write_lds(st, buf ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue ----
  // emit one 32(d) x 32(query) block held in the accumulator layout
  auto emit = [&](int s, int db, const f32x16& o, float mfin, float lfin) {
    if (rowidx[s] < 0) return;
    const int r = rowidx[s];
    const int tq = r / G;
    const int g = r - tq * G;
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
      if (db == 0 && h == 0)
        p.ws_lse[R] = lfin > 0.f ? mfin * c + __log2f(lfin) : -INFINITY;  // log2 domain
    }
  };

  bool any_shared = false;
#pragma unroll
  for (int s = 0; s < NSLOT; ++s) {
    l[s] = half_swap_sum(l[s]);
    if (slot[s].gs == 1) {
      if (slot[s].blk >= 0) {
#pragma unroll
        for (int db = 0; db < 4; ++db) emit(s, db, O[s][db], m[s], l[s]);
      }
    } else {
      any_shared = true;
    }
  }
  // shared blocks: every wave of the workgroup has exactly one shared slot (J in {1,2,5,6})
  if (J == 1 || J == 2 || J == 5 || J == 6) {
    constexpr int SS = NSLOT - 1;  // J=1,2 run with NSLOT=1 (slot 0), J=5,6 with NSLOT=2 (slot 1)
    (void)any_shared;
    float* part = reinterpret_cast<float*>(lds) + wave * (kPartBytes / 4);
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int d = 32 * db + 8 * (i >> 2) + 4 * h + (i & 3);
        part[d * kPartStride + l32] = O[SS][db][i];
      }
    if (h == 0) {
      s_ml[wave][0][l32] = m[SS];
      s_ml[wave][1][l32] = l[SS];
    }
    __syncthreads();
    const int gs = slot[SS].gs, gi = slot[SS].gi;
    const int wbase = wave - gi;
    float M = -INFINITY;
    for (int w = 0; w < gs; ++w) M = fmaxf(M, s_ml[wbase + w][0][l32]);
    const float Muse = (M == -INFINITY) ? 0.f : M;
    float wgt[4];
    float L = 0.f;
    for (int w = 0; w < gs; ++w) {
      wgt[w] = __builtin_amdgcn_exp2f((s_ml[wbase + w][0][l32] - Muse) * c);
      L += wgt[w] * s_ml[wbase + w][1][l32];
    }
    const int ndb = 4 / gs;  // column blocks this wave finishes
    for (int dd = 0; dd < ndb; ++dd) {
      const int db = gi * ndb + dd;
      f32x16 acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
      for (int w = 0; w < gs; ++w) {
        const float* pw = reinterpret_cast<const float*>(lds) + (wbase + w) * (kPartBytes / 4);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int d = 32 * db + 8 * (i >> 2) + 4 * h + (i & 3);
          acc[i] += wgt[w] * pw[d * kPartStride + l32];
        }
      }
      if (slot[SS].blk >= 0) emit(SS, db, acc, M, L);
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
    const long row_tiles = (nblk + J - 1) / J;
    const int max_splits = prefill ? 1 : 16;
    for (int S = 1; S <= max_splits; ++S) {
      if (d->num_splits && d->num_splits != S) continue;
      if (S > 1 && S > T) break;
      const long wgs = units * row_tiles * S;
      const int per_cu = J <= 4 ? 2 : 1;  // co-resident workgroups
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
  const bool two = plan.J > 4;
  if (fp8) {
    if (two) hipLaunchKernelGGL((attn_fwd_kernel<1, 2>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_fwd_kernel<1, 1>), grid, block, 0, stream, p);
  } else {
    if (two) hipLaunchKernelGGL((attn_fwd_kernel<0, 2>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_fwd_kernel<0, 1>), grid, block, 0, stream, p);
  }
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
