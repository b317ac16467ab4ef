// Sparse-prefix attention for gfx950, wide form: a workgroup owns 256 rows and runs the softmax as a pipeline
// over blocks of 32 keys.  Two shapes of the workgroup are written here:
//
//   NW = 8, NB = 1   eight wavefronts, one 32-row block each (two waves per SIMD, at most 256 registers).
//                    This is the shape that is launched.
//   NW = 4, NB = 2   four wavefronts, two 32-row blocks each: every K fragment (and V^T fragment) a wave reads
//                    from LDS feeds two MFMAs, which halves the LDS operand traffic per MFMA.  It needs more
//                    than 256 registers per lane, so a compute unit holds one wave per SIMD, and a wave alone
//                    on its SIMD issues one instruction every 4-8 clocks whatever the instruction is: measured
//                    on an MI355X, 32 MFMAs with the softmax arithmetic of 32 keys between them take ~1450
//                    clocks from one wave and ~2150-2600 clocks from each of two waves sharing a SIMD (that
//                    is 64 MFMAs), and the whole kernel came out 10-20 % slower than NW = 8 on every shape
//                    tried (165 vs 142 us at 8 x 256 query rows over 4096 keys, 749 vs 659 us at 8 x 1024).
//                    It is kept as a compile-time option of the same code, not instantiated.
//
// The loop runs as a pipeline over blocks of 32 keys in which the matrix and the vector work are spread
// evenly: the step of block k computes the scores of block k + 1 (8 MFMAs per row block), turns the scores of
// block k into probabilities (16 values per lane and row block) and multiplies the probabilities of block
// k - 1 with V (8 MFMAs per row block) -- one exponential between any two MFMAs.  The running maximum of a row
// is advanced when a block exceeds it by more than 2^8; the accumulators are rescaled at the end of the step,
// when the MFMAs that still belong to the old maximum have been issued.
//
// K and V tiles (64 keys) live in two rings of three LDS buffers: a step reads K one block ahead and V one
// block behind, and the copies of the tiles after the next land while a whole tile is computed.
//
// Same work decomposition, swizzled LDS tile layout, slot table, masks, partial results and output path as
// attn_fwd_kernel (attn_kernel.hip); bf16 caches only.  Replaces the same reference code:
// layers/attention/attention_v4.py:336-397, layers/attention/ops/prefix_prefill.py:25-230.

#include <type_traits>

#include "attn_common.h"

namespace pdllm {

namespace {

constexpr int kRing = 3;                          // tiles per ring
constexpr int kVRing = kRing * kTileBytes;        // byte offset of the V ring behind the K ring
constexpr int kWideLds = 2 * kRing * kTileBytes;  // 98304

// LDS reads of one step, in the order they are issued: K fragment q (one ds_read_b128) feeds slot 2q, V^T
// fragment v (two ds_read_b64_tr_b16) feeds slot 2v + 1; fragments 0 and 1 of each kind are issued before the
// first slot, fragment f + 2 right after fragment f has been consumed.  Returns how many younger reads may
// still be outstanding when the fragment of `slot` is needed (the operand of s_waitcnt lgkmcnt).
constexpr int sched_wait(bool qk, bool pv, int slot) {
  int issued = 0;
  int k_pos[8] = {0, 0, 0, 0, 0, 0, 0, 0}, v_pos[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int f = 0; f < 2; ++f) {
    if (qk) { k_pos[f] = issued; issued += 1; }
    if (pv) { issued += 2; v_pos[f] = issued - 1; }
  }
  for (int s = 0; s < 16; ++s) {
    const int f = s >> 1;
    const bool is_k = (s & 1) == 0;
    if (is_k ? !qk : !pv) continue;
    if (s == slot) return issued - 1 - (is_k ? k_pos[f] : v_pos[f]);
    if (f + 2 < 8) {
      if (is_k) { k_pos[f + 2] = issued; issued += 1; }
      else { issued += 2; v_pos[f + 2] = issued - 1; }
    }
  }
  return 0;
}

template <int N, typename T>
__device__ __forceinline__ void lds_wait_k(T& x) {
  static_assert(N >= 0 && N <= 7, "unexpected LDS queue depth");
  if constexpr (N == 0) lds_wait<0>(x);
  else if constexpr (N == 1) lds_wait<1>(x);
  else if constexpr (N == 2) lds_wait<2>(x);
  else if constexpr (N == 3) lds_wait<3>(x);
  else if constexpr (N == 4) lds_wait<4>(x);
  else if constexpr (N == 5) lds_wait<5>(x);
  else if constexpr (N == 6) lds_wait<6>(x);
  else lds_wait<7>(x);
}
template <int N, typename T>
__device__ __forceinline__ void lds_wait_v(T& x, T& y) {
  static_assert(N >= 0 && N <= 7, "unexpected LDS queue depth");
  if constexpr (N == 0) lds_wait2<0>(x, y);
  else if constexpr (N == 1) lds_wait2<1>(x, y);
  else if constexpr (N == 2) lds_wait2<2>(x, y);
  else if constexpr (N == 3) lds_wait2<3>(x, y);
  else if constexpr (N == 4) lds_wait2<4>(x, y);
  else if constexpr (N == 5) lds_wait2<5>(x, y);
  else if constexpr (N == 6) lds_wait2<6>(x, y);
  else lds_wait2<7>(x, y);
}

}  // namespace

template <int NW, int NB, bool BUF>  // wavefronts per workgroup, row blocks per wave
__global__ __launch_bounds__(NW * 64, 1) void attn_fwd2_kernel(const AttnKParams p) {
  static_assert((NW == 4 && NB == 2) || (NW == 8 && NB == 1), "256 rows per workgroup");
  constexpr int J = NW * NB;           // row blocks per workgroup
  constexpr int kDmaGroups = 16 / NW;  // a tile is 16 groups of 4 rows; a wave copies this many of them

  __shared__ __attribute__((aligned(1024))) char lds[kWideLds];
  // dynamic part: the dense-mask bit rows [2][kMaxTok][kNKB] of an active tile (only with PDLLM_MASK_DENSE)
  extern __shared__ __attribute__((aligned(16))) char dyn_lds[];
  uint32_t (*s_maskbits)[kMaxTok][kNKB] = reinterpret_cast<uint32_t (*)[kMaxTok][kNKB]>(dyn_lds);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int h = lane >> 5;

  const int G = p.G;
  const float c = p.scale_log2;
  const unsigned lds_base = (unsigned)(size_t)lds;

  // this workgroup's span of the tile line (see attn_fwd_kernel)
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  int col0 = 0;
  int head_rt = -1;
  int y;
  if (p.head > 0) {
    const int set = wg / p.wg_set;
    const int j = wg - set * p.wg_set;
    col0 = set * p.row_tiles;
    head_rt = j < p.row_tiles ? j : -1;
    y = j < p.row_tiles ? p.n_lin : (j - p.row_tiles) * p.span;
  } else {
    y = wg * p.span;
  }
  const int y_end = y + p.span < p.n_lin ? y + p.span : p.n_lin;
  const int tail_len = p.t_lin - p.head;
  while (head_rt >= 0 || y < y_end) {
    int rt_lin, tb, te;
    if (head_rt >= 0) {
      rt_lin = head_rt;
      tb = 0;
      te = p.head;
      head_rt = -1;
    } else {
      rt_lin = y / tail_len;
      tb = p.head + (y - rt_lin * tail_len);
      tb = __builtin_amdgcn_readfirstlane(tb);
      te = tb + (y_end - y) < p.t_lin ? tb + (y_end - y) : p.t_lin;
      y += te - tb;
    }
    const int col = __builtin_amdgcn_readfirstlane(col0 + rt_lin);
    const int piece =
        __builtin_amdgcn_readfirstlane(tb < p.head ? 0 : (p.head > 0 ? 1 : 0) + (tb - p.head + p.span - 1) / p.span);
    const bool whole = tb == 0 && te == p.t_lin;
    const int row_tile = p.mask_mode == PDLLM_MASK_CAUSAL ? p.row_tiles - 1 - col % p.row_tiles : col % p.row_tiles;
    const int kvh = (col / p.row_tiles) % p.Hkv;
    const int req = col / (p.row_tiles * p.Hkv);

    // Everything the piece needs from memory before its first copy is requested here at once: the row range of
    // the request, the number of prefix keys, and -- before that number is known -- the slot-table entries its
    // first three tiles would use if they are prefix tiles (in-bounds reads of the request's table row, taken or
    // dropped once the count has arrived).  One round trip to memory instead of three in a row.
    const int q0 = p.q_start_loc[req];
    const int q1 = p.q_start_loc[req + 1];
    const int* tbl = p.slot_table != nullptr ? p.slot_table + (long)req * p.slot_stride : nullptr;
    int ctx_total = tbl != nullptr ? tbl[p.slot_stride - 1] : 0;
    const int lane_row = 4 * wave + (lane >> 4);  // row (of every group of 4 NW rows) this lane copies
    int spec[3][16 / NW];
    if (tbl != nullptr) {
      const int last = (int)p.slot_stride - 2;
#pragma unroll
      for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int i = 0; i < 16 / NW; ++i) {
          const int idx = (tb + j) * kKT + 4 * NW * i + lane_row;
          spec[j][i] = tbl[idx < last ? idx : last];
        }
    }
    const int Sq = q1 - q0;
    if (q0 < 0 || Sq <= 0 || (long)q0 + Sq > p.n_tokens || Sq > p.max_q_len) continue;
    const int rows = Sq * G;
    const int row0 = row_tile * 32 * J;
    if (row0 >= rows) continue;
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int l32e = lane_e & 31;
    const int he = lane_e >> 5;

    ctx_total = __builtin_amdgcn_readfirstlane(ctx_total);
    const int Tc = (ctx_total + kKT - 1) / kKT;
    int Sa = Sq;
    if (p.mask_mode == PDLLM_MASK_CAUSAL) {
      const int last_row = (row0 + 32 * J < rows ? row0 + 32 * J : rows) - 1;
      const int lim = last_row / G + 1;
      Sa = lim < Sq ? lim : Sq;
    }
    const int Ta = (Sa + kKT - 1) / kKT;
    const int T = Tc + Ta;
    const int T0 = tb < T ? tb : T;
    const int T1 = te < T ? te : T;

    // ---- Q fragments (B operand of S^T = K Q^T) of the wave's two row blocks, as loaded ----
    bf16x8 Q[NB][8];
    int srow[NB], ridx[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int r = row0 + 32 * (NB * wave + b) + l32e;
      const bool valid = r < rows;
      const int rr = valid ? r : 0;
      const int tq = rr / G;
      const int g = rr - tq * G;
      srow[b] = tq;
      ridx[b] = valid ? r : -1;
      const __bf16* qp = p.q + (long)(q0 + tq) * p.q_stride + (long)(kvh * G + g) * kD + 8 * he;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (valid) {
          Q[b][ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) Q[b][ks][e] = (__bf16)0.f;
        }
      }
    }

    f32x16 O[NB][4];
    float M[NB], l[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      M[b] = -INFINITY;
      l[b] = 0.f;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[b][db][i] = 0.f;
    }

    // dense mask of active tile t -> bit rows in LDS (built one tile ahead)
    const uint8_t* mask_base = p.mask != nullptr ? p.mask + (long)q0 * p.mask_stride + q0 : nullptr;
    const int tq_first = row0 / G;
    int ntok = ((row0 + 32 * J < rows ? row0 + 32 * J : rows) - 1) / G - tq_first + 1;
    ntok = ntok < kMaxTok ? ntok : kMaxTok;
    auto build_mask = [&](int t, int par) __attribute__((always_inline)) {
      if (p.mask_mode != PDLLM_MASK_DENSE || t < Tc) return;
      const int a0 = (t - Tc) * kKT;
      for (int idx = tid; idx < ntok * kNKB; idx += NW * 64) {
        const int tok = idx / kNKB, w = idx % kNKB;
        const uint8_t* mp = mask_base + (long)(tq_first + tok) * p.mask_stride + a0 + 32 * w;
        uint32_t bits = 0;
        for (int j = 0; j < 32; ++j)
          if (a0 + 32 * w + j < Sq && mp[j] != 0) bits |= 1u << j;
        s_maskbits[par][tok][w] = bits;
      }
    };

    // ---- K/V copies HBM -> LDS: this wave moves rows 4*NW*i + 4*wave + lane/16 of a tile, i < kDmaGroups ----
    const int lane_ch = (lane & 15) ^ swz(lane_row);
    const unsigned cache_row16 = (unsigned)((p.cache_token_stride * 2) >> 4);  // 16-byte units
    const unsigned kn_row16 = (unsigned)((p.kn_stride * 2) >> 4);
    const unsigned vn_row16 = (unsigned)((p.vn_stride * 2) >> 4);
    int nslot[kDmaGroups];  // slots of the next K tile to copy
    int nsv[kDmaGroups];    // slots of the next V tile to copy
    int nnext[kDmaGroups];  // slots of the tile after those, on their way from the slot table
    // j >= 0: tile t is the piece's j-th tile, whose table entries have been requested above
    auto load_slots = [&](int (&dst)[kDmaGroups], int t, int j = -1) __attribute__((always_inline)) {
      if (t < Tc) {
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) dst[i] = j >= 0 ? spec[j][i] : tbl[t * kKT + 4 * NW * i + lane_row];
      } else {
        // padding rows copy the first row of the tile, tiles past the end of the column the last tile's rows: always
        // a valid row (they are masked, or never read)
        int a0 = (t - Tc) * kKT;
        a0 = a0 < (Ta - 1) * kKT ? a0 : (Ta - 1) * kKT;
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) {
          const int a = a0 + 4 * NW * i + lane_row;
          dst[i] = a < Sa ? a : a0;
        }
      }
    };
    const char* kc_base = static_cast<const char*>(p.k_cache) + (long)kvh * p.cache_head_stride * 2;
    const char* vc_base = static_cast<const char*>(p.v_cache) + (long)kvh * p.cache_head_stride * 2;
    const char* kn_base = reinterpret_cast<const char*>(p.k_new + (long)q0 * p.kn_stride + kvh * kD);
    const char* vn_base = reinterpret_cast<const char*>(p.v_new + (long)q0 * p.vn_stride + kvh * kD);
    const unsigned lane_b16 = (unsigned)lane_ch << 4;
    auto copy_row = [&](const char* base, unsigned row16, int slot, char* dst) __attribute__((always_inline)) {
      if constexpr (BUF) {
        const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base), 0, 0xffffffff, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)dst, 16,
                                                 __umul24((unsigned)slot, row16 << 4) + lane_b16, 0, 0, 0);
      } else {
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(base + ((unsigned long)((unsigned)slot * row16 + lane_ch) << 4)),
            (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
      }
    };
    // Copy of rows of group i of a K / V tile into ring buffer `ring` (a tile number modulo kRing).  The source of a
    // tile (cache through its slots for prefix tiles, else the new rows) is chosen once per tile: src_k / src_v.
    struct TileSrc { const char* base; unsigned row16; };
    auto src_of = [&](int t, const char* cache, const char* fresh, unsigned fresh_row16) __attribute__((always_inline)) {
      TileSrc r;
      const bool ctx = t < Tc;
      r.base = ctx ? cache : fresh;
      r.row16 = ctx ? cache_row16 : fresh_row16;
      return r;
    };
    auto issue_k1 = [&](const TileSrc& src, int ring, int i) __attribute__((always_inline)) {
      copy_row(src.base, src.row16, nslot[i], lds + ring * kTileBytes + wave * 1024 + i * (NW * 1024));
    };
    auto issue_v1 = [&](const TileSrc& src, int ring, int i) __attribute__((always_inline)) {
      copy_row(src.base, src.row16, nsv[i], lds + kVRing + ring * kTileBytes + wave * 1024 + i * (NW * 1024));
    };

    if (T0 < T1) {
      typedef __attribute__((ext_vector_type(8))) short s16x8;
      // LDS addresses of this lane's operand fragments (K: 128-bit reads of row l32 of a key block; V:
      // transposing 64-bit reads).  ka points into the ring buffer of the K tile whose blocks the next QK reads,
      // va into that of the V tile the next PV reads; both move on by one tile in the middle of an iteration.
      unsigned ka[8], va[2][4];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) ka[ks] = lds_base + l32 * kRowBytes + (((2 * ks + h) ^ swz(l32)) << 4);
      {
        const int i16 = lane & 15, g4 = l32 >> 4;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const int keyrow = 4 * h + 8 * r + (i16 >> 2);
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            const int cg = 4 * db + 2 * g4 + ((i16 & 3) >> 1);
            va[r][db] = lds_base + kVRing + keyrow * kRowBytes + ((cg ^ swz(keyrow)) << 4) + ((i16 & 1) << 3);
          }
        }
      }
      int k_ring = 0;  // ring buffer ka points into
      int v_ring = 0;  // ring buffer va points into

      // K fragment ks of key block `half` of the tile at ka; V^T fragment (16 keys kj of block `half`, columns db)
      auto rdk = [&](bf16x8& dst, int half, int ks) __attribute__((always_inline)) {
        if (half == 0) lds_read_b128<0>(dst, ka[ks]);
        else lds_read_b128<32 * kRowBytes>(dst, ka[ks]);
      };
      auto rdv = [&](s16x4& dst, int half, int v, int r) __attribute__((always_inline)) {
        const int db = v & 3, kj = 2 * half + (v >> 2);
        if (kj == 0) lds_read_tr16_b64<0>(dst, va[r][db]);
        else if (kj == 1) lds_read_tr16_b64<16 * kRowBytes>(dst, va[r][db]);
        else if (kj == 2) lds_read_tr16_b64<32 * kRowBytes>(dst, va[r][db]);
        else lds_read_tr16_b64<48 * kRowBytes>(dst, va[r][db]);
      };

      f32x16 S[2][NB];        // raw scores of the block being exponentiated / of the block after it
      uint32_t Pw[2][NB][8];  // probabilities of the block before / of this block, two bf16 per word
#pragma unroll
      for (int rb = 0; rb < NB; ++rb)
#pragma unroll
        for (int w = 0; w < 8; ++w) Pw[1][rb][w] = 0u;  // "the block before the first one": contributes nothing
      bool pending = false;   // the accumulators still have to be rescaled by alpha[]
      float alpha[NB];
      float negM[NB];   // -M, or 0 while M is still -inf (then every score is -inf as well)
      float Mneed[NB];  // M + slack: a block maximum above it moves the running maximum
#pragma unroll
      for (int rb = 0; rb < NB; ++rb) {
        alpha[rb] = 1.f;
        negM[rb] = 0.f;
        Mneed[rb] = -INFINITY;
      }

      // One step of the pipeline.  E = parity of block k inside its tile (0: first 32 keys).
      //   softmax of block k: scores S[E] -> Pw[E]          (masks: lim[rb] = visible keys of the tile, mrow)
      //   scores of block k + 1 -> S[E ^ 1]                 (K block E ^ 1 of the tile at ka)
      //   O += V^T P^T of block k - 1 with Pw[E ^ 1]        (V block E ^ 1 of the tile at va)
      //   dma(f): called once in every even slot for the copies of the tiles ahead
      // There is one form of the step: before the first block the probabilities are zero and the V tile read is the
      // first one itself; after the last block the scores of a block that does not exist are computed from
      // whatever the K ring holds and never used.
      auto step = [&](auto e_tag, bool generic, const int (&lim)[NB], const uint32_t* const (&mrow)[NB],
                      auto&& dma) __attribute__((always_inline)) {
        constexpr int E = decltype(e_tag)::value;
        f32x16 (&Sc)[NB] = S[E];
        f32x16 (&Sn)[NB] = S[E ^ 1];
        bf16x8 kf[3];
        s16x4 vlo[2], vhi[2];
        // ---- masks (rare), row maxima of block k, decision about the running maximum ----
        if (generic) {
#pragma unroll
          for (int rb = 0; rb < NB; ++rb) {
            if (mrow[rb] != nullptr || __builtin_amdgcn_ballot_w64(lim[rb] < kKT) != 0) {
              const int lb = lim[rb] - 32 * E;
              uint32_t W = lb >= 32 ? 0xffffffffu : (lb <= 0 ? 0u : ((1u << lb) - 1u));
              if (mrow[rb] != nullptr) W &= mrow[rb][E];
              W >>= 4 * h;
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                constexpr uint32_t one = 1u;
                const uint32_t bit = one << (8 * (i >> 2) + (i & 3));
                Sc[rb][i] = (W & bit) ? Sc[rb][i] : -INFINITY;
              }
            }
          }
        }
        // fragments 0 and 1 of each kind
#pragma unroll
        for (int f = 0; f < 2; ++f) {
          rdk(kf[f], E ^ 1, f);
          rdv(vlo[f], E ^ 1, f, 0);
          rdv(vhi[f], E ^ 1, f, 1);
        }
#pragma unroll
        for (int rb = 0; rb < NB; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) Sn[rb][i] = 0.f;
        float mx[NB];
        bool need = false;
#pragma unroll
        for (int rb = 0; rb < NB; ++rb) {
          float m0 = fmaxf(Sc[rb][0], Sc[rb][1]);
#pragma unroll
          for (int i = 2; i < 16; i += 2) m0 = fmaxf(fmaxf(m0, Sc[rb][i]), Sc[rb][i + 1]);
          mx[rb] = half_swap_max(m0) * c;  // log2 units; -inf (nothing visible) stays -inf
          need = need || mx[rb] > Mneed[rb];
        }
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
#pragma unroll
          for (int rb = 0; rb < NB; ++rb) {
            const float Mn = fmaxf(M[rb], mx[rb]);
            const float a = (Mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(M[rb] - Mn);  // M = -inf -> 0
            alpha[rb] = a;
            M[rb] = Mn;
            l[rb] *= a;
            negM[rb] = (Mn == -INFINITY) ? 0.f : -Mn;
            Mneed[rb] = Mn + kRescaleSlack;
          }
          pending = true;
        }
        const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
        float psum[NB];
#pragma unroll
        for (int rb = 0; rb < NB; ++rb) psum[rb] = 0.f;
        // B operand of the second MFMA: 8 probabilities (keys 16 j .. 16 j + 15 of the block, this lane's half)
        auto p_frag = [&](int e, int rb, int j) __attribute__((always_inline)) {
          const uint4 w = {Pw[e][rb][4 * j], Pw[e][rb][4 * j + 1], Pw[e][rb][4 * j + 2], Pw[e][rb][4 * j + 3]};
          return __builtin_bit_cast(bf16x8, w);
        };
        auto exp2s = [&](float e, int rb) __attribute__((always_inline)) {
          return __builtin_amdgcn_exp2f(__builtin_fmaf(e, c, negM[rb]));
        };
        __builtin_amdgcn_sched_barrier(0);
        // ---- 16 slots of two MFMAs each.  A wave alone on its SIMD issues in order, and the matrix unit takes a new
        // MFMA every 32 clocks: the second MFMA of a slot would hold up everything behind it, so each half of a slot
        // is one MFMA followed by the arithmetic of one probability (pair pr = s of the block: row block s / 8,
        // scores 2 (s % 8) and + 1).  The scores and the intermediate results pass through (empty) asm statements
        // of their half: that keeps the arithmetic there -- the instruction selector would otherwise gather all of
        // it in one place.
        float xa = 0.f, xb = 0.f;  // the probabilities of the pair that is packed next
#pragma unroll
        for (int s = 0; s < 16; ++s) {
          const int f = s >> 1;
          bf16x8 frag;
          if ((s & 1) == 0) {
            // wait for K fragment f
            if (s == 0) lds_wait_k<sched_wait(true, true, 0)>(kf[f % 3]);
            else if (s == 2) lds_wait_k<sched_wait(true, true, 2)>(kf[f % 3]);
            else if (s == 4) lds_wait_k<sched_wait(true, true, 4)>(kf[f % 3]);
            else if (s == 6) lds_wait_k<sched_wait(true, true, 6)>(kf[f % 3]);
            else if (s == 8) lds_wait_k<sched_wait(true, true, 8)>(kf[f % 3]);
            else if (s == 10) lds_wait_k<sched_wait(true, true, 10)>(kf[f % 3]);
            else if (s == 12) lds_wait_k<sched_wait(true, true, 12)>(kf[f % 3]);
            else lds_wait_k<sched_wait(true, true, 14)>(kf[f % 3]);
            frag = kf[f % 3];
          } else {
            if (s == 1) lds_wait_v<sched_wait(true, true, 1)>(vlo[f & 1], vhi[f & 1]);
            else if (s == 3) lds_wait_v<sched_wait(true, true, 3)>(vlo[f & 1], vhi[f & 1]);
            else if (s == 5) lds_wait_v<sched_wait(true, true, 5)>(vlo[f & 1], vhi[f & 1]);
            else if (s == 7) lds_wait_v<sched_wait(true, true, 7)>(vlo[f & 1], vhi[f & 1]);
            else if (s == 9) lds_wait_v<sched_wait(true, true, 9)>(vlo[f & 1], vhi[f & 1]);
            else if (s == 11) lds_wait_v<sched_wait(true, true, 11)>(vlo[f & 1], vhi[f & 1]);
            else if (s == 13) lds_wait_v<sched_wait(true, true, 13)>(vlo[f & 1], vhi[f & 1]);
            else lds_wait_v<sched_wait(true, true, 15)>(vlo[f & 1], vhi[f & 1]);
            const s16x4 a = vlo[f & 1], b2 = vhi[f & 1];
            const s16x8 both = {a[0], a[1], a[2], a[3], b2[0], b2[1], b2[2], b2[3]};
            frag = __builtin_bit_cast(bf16x8, both);
          }
          // The two probabilities of a pair are packed (and added to the row sum) one half-slot after the second
          // exponential: a result of the transcendental unit read by the very next instruction costs a wait state.
          if constexpr (NB == 2) {
            const int prb = s >> 3, pi = 2 * (s & 7);
            float e0 = Sc[prb][pi], e1 = Sc[prb][pi + 1];
            // ---- first half: MFMA of row block 0, pack of the previous pair, first probability ----
            asm volatile("" : "+v"(e0), "+v"(psum[0]), "+v"(psum[1]), "+v"(xa), "+v"(xb));
            if ((s & 1) == 0) Sn[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, Q[0][f], Sn[0], 0, 0, 0);
            else O[0][f & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, p_frag(E ^ 1, 0, f >> 2), O[0][f & 3], 0, 0, 0);
            if (s > 0) {
              const bf16x2 pv2 = {(__bf16)xa, (__bf16)xb};
              psum[(s - 1) >> 3] = __builtin_amdgcn_fdot2_f32_bf16(pv2, ones, psum[(s - 1) >> 3], false);
              Pw[E][(s - 1) >> 3][(s - 1) & 7] = __builtin_bit_cast(uint32_t, pv2);
            }
            xa = exp2s(e0, prb);
            __builtin_amdgcn_sched_barrier(0);
            // ---- second half: MFMA of row block 1, second probability; next fragment ----
            asm volatile("" : "+v"(e1), "+v"(xa));
            if ((s & 1) == 0) {
              Sn[NB - 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, Q[NB - 1][f], Sn[NB - 1], 0, 0, 0);
              if (f + 2 < 8) rdk(kf[(f + 2) % 3], E ^ 1, f + 2);
              dma(f);
            } else {
              O[NB - 1][f & 3] =
                  __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, p_frag(E ^ 1, NB - 1, f >> 2), O[NB - 1][f & 3], 0, 0, 0);
              if (f + 2 < 8) { rdv(vlo[f & 1], E ^ 1, f + 2, 0); rdv(vhi[f & 1], E ^ 1, f + 2, 1); }
            }
            xb = exp2s(e1, prb);
          } else {
            // one row block per wave: one MFMA and one probability per slot; the pair of slots s - 2, s - 1 is
            // packed in the even slot s
            float e = Sc[0][s];
            asm volatile("" : "+v"(e), "+v"(psum[0]), "+v"(xa), "+v"(xb));
            if ((s & 1) == 0) {
              Sn[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, Q[0][f], Sn[0], 0, 0, 0);
              if (s > 0) {
                const bf16x2 pv2 = {(__bf16)xa, (__bf16)xb};
                psum[0] = __builtin_amdgcn_fdot2_f32_bf16(pv2, ones, psum[0], false);
                Pw[E][0][(s >> 1) - 1] = __builtin_bit_cast(uint32_t, pv2);
              }
              if (f + 2 < 8) rdk(kf[(f + 2) % 3], E ^ 1, f + 2);
              dma(f);
              xa = exp2s(e, 0);
            } else {
              O[0][f & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag, p_frag(E ^ 1, 0, f >> 2), O[0][f & 3], 0, 0, 0);
              if (f + 2 < 8) { rdv(vlo[f & 1], E ^ 1, f + 2, 0); rdv(vhi[f & 1], E ^ 1, f + 2, 1); }
              xb = exp2s(e, 0);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        {
          // the last pair
          asm volatile("" : "+v"(xa), "+v"(xb));
          const bf16x2 pv2 = {(__bf16)xa, (__bf16)xb};
          psum[NB - 1] = __builtin_amdgcn_fdot2_f32_bf16(pv2, ones, psum[NB - 1], false);
          Pw[E][NB - 1][7] = __builtin_bit_cast(uint32_t, pv2);
        }
#pragma unroll
        for (int rb = 0; rb < NB; ++rb) {
          asm volatile("" : "+v"(psum[rb]));
          l[rb] += psum[rb];
        }
        // the accumulators follow the running maximum once every MFMA of the old one has been issued
        if (pending) {
#pragma unroll
          for (int rb = 0; rb < NB; ++rb)
#pragma unroll
            for (int db = 0; db < 4; ++db) {
#pragma unroll
              for (int i = 0; i < 16; ++i) O[rb][db][i] *= alpha[rb];
              __builtin_amdgcn_sched_barrier(0);
            }
          pending = false;
        }
      };

      // ---- prologue: K(T0), V(T0), K(T0+1); scores of the first block ----
      load_slots(nslot, T0, 0);  // (T0 == tb: the piece has tiles)
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
      {
        const TileSrc sk = src_of(T0, kc_base, kn_base, kn_row16), sv = src_of(T0, vc_base, vn_base, vn_row16);
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) issue_k1(sk, 0, i);
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) issue_v1(sv, 0, i);
      }
      {
        // (like the copies inside the loop, issued whether or not the piece has a second tile: the slots loaded for a
        // tile and the source chosen for it always belong together)
        load_slots(nslot, T0 + 1, 1);
        const TileSrc sk = src_of(T0 + 1, kc_base, kn_base, kn_row16);
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) issue_k1(sk, 1, i);
      }
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];  // slots of tile T0 + 1 for its V copy
      load_slots(nslot, T0 + 2, 2);
      build_mask(T0, 0);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      {
        // scores of block 0 (unpipelined)
#pragma unroll
        for (int rb = 0; rb < NB; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) S[0][rb][i] = 0.f;
        bf16x8 kf[3];
        rdk(kf[0], 0, 0);
        rdk(kf[1], 0, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < 8; ++f) {
          if (f + 2 < 8) { rdk(kf[(f + 2) % 3], 0, f + 2); lds_wait<2>(kf[f % 3]); }
          else if (f + 1 < 8) lds_wait<1>(kf[f % 3]);
          else lds_wait<0>(kf[f % 3]);
#pragma unroll
          for (int rb = 0; rb < NB; ++rb)
            S[0][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[f % 3], Q[rb][f], S[0][rb], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // ---- the tiles of the piece: one loop, one form of the iteration (two steps) ----
      for (int t = T0; t < T1; ++t) {
        const int par = (t - T0) & 1;
        const bool has_next = t + 1 < T1;
        // the slots of tile t + 3 are fetched first, while no copy is in flight
        load_slots(nnext, t + 3);
        if (has_next) build_mask(t + 1, par ^ 1);
        const bool active = t >= Tc;
        const int a0 = active ? (t - Tc) * kKT : 0;
        int nvalid = active ? Sa - a0 : ctx_total - t * kKT;
        const bool generic = nvalid < kKT || (active && p.mask_mode != PDLLM_MASK_FULL);
        nvalid = nvalid < kKT ? nvalid : kKT;
        int lim[NB];
        const uint32_t* mrow[NB];
#pragma unroll
        for (int rb = 0; rb < NB; ++rb) { lim[rb] = kKT; mrow[rb] = nullptr; }
        if (generic) {
#pragma unroll
          for (int rb = 0; rb < NB; ++rb) {
            lim[rb] = nvalid;
            if (active && p.mask_mode == PDLLM_MASK_CAUSAL) {
              const int cl = srow[rb] - a0 + 1;
              lim[rb] = cl < lim[rb] ? cl : lim[rb];
            }
            int tl = srow[rb] - tq_first;
            tl = tl < 0 ? 0 : (tl >= kMaxTok ? kMaxTok - 1 : tl);
            if (active && p.mask_mode == PDLLM_MASK_DENSE) mrow[rb] = &s_maskbits[par][tl][0];
          }
        }
        // ring buffers: K(t) and V(t) sit in buffer (t - T0) % 3 (= k_ring here), K(t+1) in the next one; the copy
        // of V(t+1) goes into the next one, that of K(t+2) into the one after
        const int ring1 = k_ring + 1 >= kRing ? k_ring + 1 - kRing : k_ring + 1;
        const int ring2 = ring1 + 1 >= kRing ? ring1 + 1 - kRing : ring1 + 1;
        // The copies are issued whether or not the piece has a tile t + 1 / t + 2: their ring buffers are free, their
        // slots name valid rows, and what lands there is never read (cheaper than a branch around every instruction).
        const TileSrc src_v = src_of(t + 1, vc_base, vn_base, vn_row16);
        const TileSrc src_k = src_of(t + 2, kc_base, kn_base, kn_row16);
        auto dma_a = [&](int f) __attribute__((always_inline)) {
          if (f < kDmaGroups) issue_v1(src_v, ring1, f);
          else if (f < 2 * kDmaGroups) issue_k1(src_k, ring2, f - kDmaGroups);
        };
        auto no_dma = [&](int) __attribute__((always_inline)) {};
        // step of the tile's first block: QK of its second block (same K tile), PV of the last block of tile t - 1
        // (for the first tile: zero probabilities against the first V tile itself)
        step(std::integral_constant<int, 0>{}, generic, lim, mrow, dma_a);
        // K: on to tile t + 1; V: on to tile t (in the first iteration va is there already)
        {
          const int kn = k_ring + 1 == kRing ? 0 : k_ring + 1;
          const int dk = (kn - k_ring) * kTileBytes;
          k_ring = kn;
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) ka[ks] += dk;
          if (t > T0) {
            const int vn = v_ring + 1 == kRing ? 0 : v_ring + 1;
            const int dv = (vn - v_ring) * kTileBytes;
            v_ring = vn;
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
              for (int db = 0; db < 4; ++db) va[r][db] += dv;
          }
        }
        // step of the tile's second block: QK of the first block of tile t + 1, PV of the tile's first block
        step(std::integral_constant<int, 1>{}, generic, lim, mrow, no_dma);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): K(t+2), V(t+1) and the slots have landed
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) { nsv[i] = nslot[i]; nslot[i] = nnext[i]; }
        __syncthreads();
      }
      // ---- the last block still has to be multiplied with V (second block of tile T1 - 1, at va) ----
      {
        s16x4 vlo[2], vhi[2];
        rdv(vlo[0], 1, 0, 0); rdv(vhi[0], 1, 0, 1);
        rdv(vlo[1], 1, 1, 0); rdv(vhi[1], 1, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < 8; ++f) {
          if (f + 1 < 8) lds_wait2<2>(vlo[f & 1], vhi[f & 1]);
          else lds_wait2<0>(vlo[f & 1], vhi[f & 1]);
          const s16x4 a = vlo[f & 1], b2 = vhi[f & 1];
          const s16x8 both = {a[0], a[1], a[2], a[3], b2[0], b2[1], b2[2], b2[3]};
          const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
          const int db = f & 3, j = f >> 2;
#pragma unroll
          for (int rb = 0; rb < NB; ++rb) {
            const uint4 w = {Pw[1][rb][4 * j], Pw[1][rb][4 * j + 1], Pw[1][rb][4 * j + 2], Pw[1][rb][4 * j + 3]};
            O[rb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, __builtin_bit_cast(bf16x8, w), O[rb][db], 0, 0, 0);
          }
          if (f + 2 < 8) { rdv(vlo[f & 1], 1, f + 2, 0); rdv(vhi[f & 1], 1, f + 2, 1); }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // the output strips below reuse the K ring; every wave has left the tile loop (barrier of the last
      // iteration) and the last V reads above go to the V ring -- which the strips of eight waves reach into
      if constexpr (NW * 8192 > kVRing) __syncthreads();
    }

    // ---- epilogue ----
    auto emit = [&](int rix, int db, const f32x16& o, float mfin, float lfin) __attribute__((always_inline)) {
      if (rix < 0) return;
      const int tq = rix / G;
      const int g = rix - tq * G;
      const float inv = lfin > 0.f ? 1.f / lfin : 0.f;
      const long R = ((long)(q0 + tq) * p.Hq + kvh * G + g) * p.max_pieces + piece;
      store_partial_block(p.ws_o + R * kD, p.ws_scale + R * 4, db, he, o, inv);
      if (db == 0 && he == 0) p.ws_lse[R] = lfin > 0.f ? mfin + __log2f(lfin) : -INFINITY;  // log2 domain
    };
    // rows of an uncut column go through an 8 KB strip of the (now free) K ring per wave, 64 columns at a time,
    // so that 8 lanes store the 128 contiguous bytes of a row; partial rows are stored directly
    auto emit_block = [&](int rix, const f32x16 (&Ob)[4], float mfin, float lfin) __attribute__((always_inline)) {
      if (!whole) {
#pragma unroll
        for (int db = 0; db < 4; ++db) emit(rix, db, Ob[db], mfin, lfin);
        return;
      }
      const float inv = lfin > 0.f ? 1.f / lfin : 0.f;
      unsigned long rowptr = 0;  // global address of this lane's row, 0 = no such row
      if (rix >= 0) {
        const int tq = rix / G;
        const int g = rix - tq * G;
        rowptr = (unsigned long)(p.out + (long)(q0 + tq) * p.o_stride + (long)(kvh * G + g) * kD);
      }
      const int ptr_lo = (int)(unsigned)rowptr, ptr_hi = (int)(unsigned)(rowptr >> 32);
      float* strip = reinterpret_cast<float*>(lds + wave * 8192);
      const int j = lane_e & 7;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int dd = 0; dd < 2; ++dd)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const f32x16& o = Ob[2 * hf + dd];
            const int c4 = 8 * dd + 2 * i4 + he;
            const float4 w = {o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv, o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv};
            *reinterpret_cast<float4*>(strip + l32e * 64 + 4 * (c4 ^ (l32e & 15))) = w;
          }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int rr = 8 * k + (lane_e >> 3);
          const unsigned long dst =
              ((unsigned long)(unsigned)__shfl(ptr_hi, rr, 64) << 32) | (unsigned)__shfl(ptr_lo, rr, 64);
          const float4 a = *reinterpret_cast<const float4*>(strip + rr * 64 + 4 * ((2 * j) ^ (rr & 15)));
          const float4 b = *reinterpret_cast<const float4*>(strip + rr * 64 + 4 * ((2 * j + 1) ^ (rr & 15)));
          uint4 w;
          w.x = pack_bf16x2(a.x, a.y); w.y = pack_bf16x2(a.z, a.w);
          w.z = pack_bf16x2(b.x, b.y); w.w = pack_bf16x2(b.z, b.w);
          if (dst != 0) *reinterpret_cast<uint4*>(dst + 2 * (64 * hf + 8 * j)) = w;
        }
      }
    };
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      l[b] = half_swap_sum(l[b]);
      emit_block(ridx[b], O[b], M[b], l[b]);
    }
    if (head_rt >= 0 || y < y_end) {
      // the next piece reuses the LDS buffers: wait for this piece's LDS accesses only, the global stores of the
      // epilogue stay in flight behind the next prologue
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
  }  // pieces
}

int launch_attn_fwd2(const AttnKParams& p, int grid, int dyn_lds, bool buf, hipStream_t stream) {
  if (buf) hipLaunchKernelGGL((attn_fwd2_kernel<8, 1, true>), dim3((unsigned)grid), dim3(512), dyn_lds, stream, p);
  else hipLaunchKernelGGL((attn_fwd2_kernel<8, 1, false>), dim3((unsigned)grid), dim3(512), dyn_lds, stream, p);
  return launch_status();
}

}  // namespace pdllm

