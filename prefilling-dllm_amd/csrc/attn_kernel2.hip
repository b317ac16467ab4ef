// Sparse-prefix attention for gfx950, wide form: a workgroup of 4 wavefronts owns 256 rows, every wave two
// 32-row blocks.  Each K fragment (and each V^T fragment) a wave reads from LDS feeds two MFMAs, one per row
// block, which halves the LDS operand traffic per MFMA against one block per wave -- at one block per wave
// every MFMA needs a fresh 1 KB fragment, which is the whole LDS bandwidth of a compute unit.  The price is the
// register file: two sets of Q fragments, accumulators and scores need more than 256 registers per lane, so a
// compute unit holds one such workgroup (one wave per SIMD, up to 512 registers) and all overlap of matrix,
// vector and LDS work is arranged inside the wave: while the vector unit turns the scores of tile t into
// probabilities, the matrix unit computes the scores of tile t + 1.
//
// Same work decomposition, data layout in LDS, slot table, masks, partial results and epilogue as
// attn_fwd_kernel (attn_kernel.hip); bf16 caches only.  Replaces the same reference code:
// layers/attention/attention_v4.py:336-397, layers/attention/ops/prefix_prefill.py:25-230.

#include <type_traits>

#include "attn_common.h"

namespace pdllm {

template <int N, typename T>
__device__ __forceinline__ void lds_wait_pin2(T& x, float& a0, float& a1, float& b0, float& b1, float& pa, float& pb,
                                              const T& keep) {
  asm volatile("s_waitcnt lgkmcnt(%7)"
               : "+v"(x), "+v"(a0), "+v"(a1), "+v"(b0), "+v"(b1), "+v"(pa), "+v"(pb)
               : "n"(N), "v"(keep)
               : "memory");
}

#ifdef ATTN_PROBE
__device__ unsigned long long g_probe[8 * 1024];
#define PROBE_T(i) { const unsigned long long now_ = __builtin_amdgcn_s_memtime(); pr_acc[i] += now_ - pr_last; pr_last = now_; }
#else
#define PROBE_T(i)
#endif

template <bool BUF>
__global__ __launch_bounds__(256, 1) void attn_fwd2_kernel(const AttnKParams p) {
#ifdef ATTN_PROBE
  unsigned long long pr_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  unsigned long long pr_last = __builtin_amdgcn_s_memtime();
  const unsigned long long pr_start = pr_last;
#endif
  constexpr int NW = 4;                // wavefronts per workgroup
  constexpr int NB = 2;                // row blocks per wave
  constexpr int J = NW * NB;           // row blocks per workgroup
  constexpr int kDmaGroups = 16 / NW;  // a tile is 16 groups of 4 rows; a wave copies this many of them

  __shared__ __attribute__((aligned(1024))) char lds[kMainBytes];
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

  // LDS addresses of this lane's operand fragments in buffer 0 (K: 128-bit reads of row l32 of a key block;
  // V: transposing 64-bit reads); they move to the other buffer after every tile
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
        va[r][db] = lds_base + keyrow * kRowBytes + ((cg ^ swz(keyrow)) << 4) + ((i16 & 1) << 3);
      }
    }
  }

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

    const int q0 = p.q_start_loc[req];
    const int Sq = p.q_start_loc[req + 1] - q0;
    if (q0 < 0 || Sq <= 0 || (long)q0 + Sq > p.n_tokens || Sq > p.max_q_len) continue;
    const int rows = Sq * G;
    const int row0 = row_tile * 32 * J;
    if (row0 >= rows) continue;
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int l32e = lane_e & 31;
    const int he = lane_e >> 5;

    const int* tbl = p.slot_table != nullptr ? p.slot_table + (long)req * p.slot_stride : nullptr;
    int ctx_total = tbl != nullptr ? tbl[p.slot_stride - 1] : 0;
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
    const int lane_row = 4 * wave + (lane >> 4);
    const int lane_ch = (lane & 15) ^ swz(lane_row);
    const unsigned cache_row16 = (unsigned)((p.cache_token_stride * 2) >> 4);  // 16-byte units
    const unsigned kn_row16 = (unsigned)((p.kn_stride * 2) >> 4);
    const unsigned vn_row16 = (unsigned)((p.vn_stride * 2) >> 4);
    int nslot[kDmaGroups];  // slots of the next K tile
    int nsv[kDmaGroups];    // slots of the next V tile
    auto load_slots_ctx = [&](int t) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) nslot[i] = tbl[t * kKT + 4 * NW * i + lane_row];
    };
    auto load_slots_new = [&](int t) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) nslot[i] = (t - Tc) * kKT + 4 * NW * i + lane_row;
    };
    auto load_slots = [&](int t) __attribute__((always_inline)) {
      if (t < Tc) {
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) nslot[i] = tbl[t * kKT + 4 * NW * i + lane_row];
      } else {
        const int a0 = (t - Tc) * kKT;
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) {
          const int a = a0 + 4 * NW * i + lane_row;
          nslot[i] = a < Sa ? a : a0;  // padding rows copy the first (always valid) row; they are masked
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
    // src_tag: 0 = decide by the tile number, 1 = the tile comes from the cache, 2 = from the new rows
    auto issue_k1 = [&](int t, int buf, int i, auto src_tag) __attribute__((always_inline)) {
      constexpr int SRC = decltype(src_tag)::value;
      const bool ctx = SRC == 1 || (SRC == 0 && t < Tc);
      copy_row(ctx ? kc_base : kn_base, ctx ? cache_row16 : kn_row16, nslot[i],
               lds + buf * kBufBytes + wave * 1024 + i * (NW * 1024));
    };
    auto issue_v1 = [&](int t, int buf, int i, auto src_tag) __attribute__((always_inline)) {
      constexpr int SRC = decltype(src_tag)::value;
      const bool ctx = SRC == 1 || (SRC == 0 && t < Tc);
      copy_row(ctx ? vc_base : vn_base, ctx ? cache_row16 : vn_row16, nsv[i],
               lds + buf * kBufBytes + kTileBytes + wave * 1024 + i * (NW * 1024));
    };
    auto rdk = [&](bf16x8& dst, int stp) __attribute__((always_inline)) {
      if ((stp >> 3) == 0) lds_read_b128<0>(dst, ka[stp & 7]);
      else lds_read_b128<32 * kRowBytes>(dst, ka[stp & 7]);
    };
    auto rdv = [&](s16x4& dst, int stp, int r) __attribute__((always_inline)) {
      constexpr int base = kTileBytes;
      const int db = stp & 3, kj = stp >> 2;
      if (kj == 0) lds_read_tr16_b64<base>(dst, va[r][db]);
      else if (kj == 1) lds_read_tr16_b64<base + 16 * kRowBytes>(dst, va[r][db]);
      else if (kj == 2) lds_read_tr16_b64<base + 32 * kRowBytes>(dst, va[r][db]);
      else lds_read_tr16_b64<base + 48 * kRowBytes>(dst, va[r][db]);
    };
    constexpr int PF = 3, NS = 16;  // K fragments read ahead; MFMA steps of a phase

    if (T0 < T1) {
      typedef __attribute__((ext_vector_type(8))) short s16x8;
      int flip = kBufBytes;  // ka: buffer 1 -> 0 -> 1 ..., va: buffer 0 -> 1 -> 0 ...

      // One iteration: softmax of tile t (raw scores in Sc) interleaved with QK of tile t + 1, then PV of tile t.
      // PAR = buffer of V(t); K(t+1) sits in the other buffer.  MODE 1 / 2: tiles t .. t + 3 are whole tiles of
      // the prefix / of the active block inside this piece and tile t needs no mask for any row.
      auto iter = [&](int t, int PAR, f32x16 (&Sc)[NB][2], auto steady_tag) __attribute__((always_inline)) {
        constexpr int MODE = decltype(steady_tag)::value;
        constexpr bool STEADY = MODE != 0;
        const bool has_next = STEADY || t + 1 < T1;
        const bool k_on = STEADY || t + 2 < T1;
        PROBE_T(0)
        if (!STEADY && has_next) build_mask(t + 1, PAR ^ 1);

        const bool active = !STEADY && t >= Tc;
        const int a0 = active ? (t - Tc) * kKT : 0;
        int nvalid = STEADY ? kKT : active ? Sa - a0 : ctx_total - t * kKT;
        const bool generic = !STEADY && (nvalid < kKT || (active && p.mask_mode != PDLLM_MASK_FULL));
        nvalid = nvalid < kKT ? nvalid : kKT;
        // ---- masks, row maxima, lazy rescale (vector unit only) ----
        if (generic) {
#pragma unroll
          for (int rb = 0; rb < NB; ++rb) {
            int lim = nvalid;
            if (active && p.mask_mode == PDLLM_MASK_CAUSAL) {
              const int cl = srow[rb] - a0 + 1;
              lim = cl < lim ? cl : lim;
            }
            int tl = srow[rb] - tq_first;
            tl = tl < 0 ? 0 : (tl >= kMaxTok ? kMaxTok - 1 : tl);
            const uint32_t* mrow =
                (active && p.mask_mode == PDLLM_MASK_DENSE) ? &s_maskbits[PAR][tl][0] : nullptr;
            if (mrow != nullptr || __builtin_amdgcn_ballot_w64(lim < kKT) != 0) {
#pragma unroll
              for (int b = 0; b < 2; ++b) {
                const int lb = lim - 32 * b;
                uint32_t W = lb >= 32 ? 0xffffffffu : (lb <= 0 ? 0u : ((1u << lb) - 1u));
                if (mrow != nullptr) W &= mrow[b];
                W >>= 4 * h;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                  constexpr uint32_t one = 1u;
                  const uint32_t bit = one << (8 * (i >> 2) + (i & 3));
                  Sc[rb][b][i] = (W & bit) ? Sc[rb][b][i] : -INFINITY;
                }
              }
            }
          }
        }
        float mx[NB];
        bool need = false;
#pragma unroll
        for (int rb = 0; rb < NB; ++rb) {
          float m0 = fmaxf(Sc[rb][0][0], Sc[rb][0][1]);
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = (b == 0 ? 2 : 0); i < 16; i += 2) m0 = fmaxf(fmaxf(m0, Sc[rb][b][i]), Sc[rb][b][i + 1]);
          mx[rb] = half_swap_max(m0) * c;  // log2 units
          need = need || mx[rb] > M[rb] + kRescaleSlack;
        }
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
#pragma unroll
          for (int rb = 0; rb < NB; ++rb) {
            const float Mn = fmaxf(M[rb], mx[rb]);
            const float alpha = (Mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(M[rb] - Mn);
            M[rb] = Mn;
            l[rb] *= alpha;
#pragma unroll
            for (int db = 0; db < 4; ++db) {
#pragma unroll
              for (int i = 0; i < 16; ++i) O[rb][db][i] *= alpha;
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
        PROBE_T(1)
        // ---- exponentials of tile t, two per row block and step, between the MFMAs of QK(t+1) ----
        float negM[NB];
#pragma unroll
        for (int rb = 0; rb < NB; ++rb) negM[rb] = (M[rb] == -INFINITY) ? 0.f : -M[rb];
        f32x16 Sn[NB][2];
#pragma unroll
        for (int rb = 0; rb < NB; ++rb)
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) Sn[rb][b][i] = 0.f;
        bf16x8 P[NB][2][2];
        const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
        float psum[NB] = {0.f, 0.f};
        auto exp_pair = [&](int rb, int stp) __attribute__((always_inline)) {
          const int b = stp >> 3, i = 2 * (stp & 7);
          const bf16x2 pr = {(__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(Sc[rb][b][i], c, negM[rb])),
                             (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(Sc[rb][b][i + 1], c, negM[rb]))};
          psum[rb] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, psum[rb], false);
          P[rb][b][i >> 3][i & 7] = pr[0];
          P[rb][b][i >> 3][(i & 7) + 1] = pr[1];
        };
        if (has_next) {
          bf16x8 kf[PF];
#pragma unroll
          for (int i = 0; i < PF; ++i) rdk(kf[i], i);
          bf16x8 used = kf[0];  // fragment of the MFMAs issued in the step before
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int stp = 0; stp < NS; ++stp) {
            const int kb = stp >> 3, ks = stp & 7, e = 2 * ks;
            {
              float a0s = Sc[0][kb][e], a1s = Sc[0][kb][e + 1], b0s = Sc[1][kb][e], b1s = Sc[1][kb][e + 1];
              const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;
              if (young == 2) lds_wait_pin2<2>(kf[stp % PF], a0s, a1s, b0s, b1s, psum[0], psum[1], used);
              else if (young == 1) lds_wait_pin2<1>(kf[stp % PF], a0s, a1s, b0s, b1s, psum[0], psum[1], used);
              else lds_wait_pin2<0>(kf[stp % PF], a0s, a1s, b0s, b1s, psum[0], psum[1], used);
              used = kf[stp % PF];
              Sc[0][kb][e] = a0s; Sc[0][kb][e + 1] = a1s; Sc[1][kb][e] = b0s; Sc[1][kb][e + 1] = b1s;
            }
            if (ks == 7) {
              // the block's exponentials are all issued: its registers take the finished scores
              exp_pair(0, stp);
              exp_pair(1, stp);
              Sc[0][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], Q[0][7], Sn[0][kb], 0, 0, 0);
              Sc[1][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], Q[1][7], Sn[1][kb], 0, 0, 0);
            } else {
              Sn[0][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], Q[0][ks], Sn[0][kb], 0, 0, 0);
              Sn[1][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], Q[1][ks], Sn[1][kb], 0, 0, 0);
              exp_pair(0, stp);
              exp_pair(1, stp);
            }
            if (stp + PF < NS) rdk(kf[stp % PF], stp + PF);
            if ((stp & 1) == 1 && (ks >> 1) < kDmaGroups) {
              if (stp < 8) issue_v1(t + 1, PAR ^ 1, ks >> 1, steady_tag);
              else if (k_on) issue_k1(t + 2, PAR, ks >> 1, steady_tag);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
#pragma unroll
          for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
          if (MODE == 1) load_slots_ctx(t + 3);
          else if (MODE == 2) load_slots_new(t + 3);
          else if (t + 3 < T1) load_slots(t + 3);
        } else {
#pragma unroll
          for (int stp = 0; stp < NS; ++stp) {
            exp_pair(0, stp);
            exp_pair(1, stp);
          }
        }
        l[0] += psum[0];
        l[1] += psum[1];
        __builtin_amdgcn_sched_barrier(0);
        PROBE_T(2)
        // ---- PV of tile t: every V^T fragment feeds both row blocks ----
        {
          s16x4 lo[2], hi[2];
          rdv(lo[0], 0, 0); rdv(hi[0], 0, 1);
          rdv(lo[1], 1, 0); rdv(hi[1], 1, 1);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int stp = 0; stp < NS; ++stp) {
            const int db = stp & 3, kj = stp >> 2;
            if (stp + 1 < NS) lds_wait2<2>(lo[stp & 1], hi[stp & 1]);
            else lds_wait2<0>(lo[stp & 1], hi[stp & 1]);
            const s16x4 a = lo[stp & 1], b2 = hi[stp & 1];
            const s16x8 both = {a[0], a[1], a[2], a[3], b2[0], b2[1], b2[2], b2[3]};
            const bf16x8 vf = __builtin_bit_cast(bf16x8, both);
            O[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, P[0][kj >> 1][kj & 1], O[0][db], 0, 0, 0);
            O[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, P[1][kj >> 1][kj & 1], O[1][db], 0, 0, 0);
            if (stp + 2 < NS) { rdv(lo[stp & 1], stp + 2, 0); rdv(hi[stp & 1], stp + 2, 1); }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        PROBE_T(3)
        // the next tile reads the other buffers
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) ka[ks] -= flip;
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int db = 0; db < 4; ++db) va[r][db] += flip;
        flip = -flip;
#ifndef EXP_NOWAIT
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): K(t+2), V(t+1) and the slots have landed
#endif
        PROBE_T(4)
        __syncthreads();
        PROBE_T(5)
      };

      // ---- prologue: K(T0), V(T0); then K(T0+1) while QK(T0) runs unpipelined ----
      f32x16 SX[NB][2];
      load_slots(T0);
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) issue_k1(T0, 0, i, std::integral_constant<int, 0>{});
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) issue_v1(T0, 0, i, std::integral_constant<int, 0>{});
      if (T0 + 1 < T1) load_slots(T0 + 1);
      build_mask(T0, 0);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (T0 + 1 < T1) {
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) issue_k1(T0 + 1, 1, i, std::integral_constant<int, 0>{});
      }
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
      if (T0 + 2 < T1) load_slots(T0 + 2);
#pragma unroll
      for (int rb = 0; rb < NB; ++rb)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = 0; i < 16; ++i) SX[rb][b][i] = 0.f;
      {
        bf16x8 kf[PF];
#pragma unroll
        for (int i = 0; i < PF; ++i) rdk(kf[i], i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int stp = 0; stp < NS; ++stp) {
          const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;
          if (young == 2) lds_wait<2>(kf[stp % PF]);
          else if (young == 1) lds_wait<1>(kf[stp % PF]);
          else lds_wait<0>(kf[stp % PF]);
          SX[0][stp >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], Q[0][stp & 7], SX[0][stp >> 3], 0, 0, 0);
          SX[1][stp >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], Q[1][stp & 7], SX[1][stp >> 3], 0, 0, 0);
          if (stp + PF < NS) rdk(kf[stp % PF], stp + PF);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // from here on ka reads K(t+1) in buffer 1 and va reads V(t) in buffer 0
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) ka[ks] += kBufBytes;
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      {
        using Generic = std::integral_constant<int, 0>;
        const int whole_ctx = ctx_total / kKT;  // tiles of the prefix without a ragged end
        const int ctx_end = (T1 < whole_ctx ? T1 : whole_ctx) - 3;
        // active tiles that are whole and visible to every row of this row group
        int open_tiles = Sa / kKT;
        if (p.mask_mode == PDLLM_MASK_CAUSAL) open_tiles = (tq_first + 1) / kKT < open_tiles ? (tq_first + 1) / kKT : open_tiles;
        if (p.mask_mode == PDLLM_MASK_DENSE) open_tiles = 0;
        int new_end = Tc + Sa / kKT - 3;
        new_end = new_end < T1 - 3 ? new_end : T1 - 3;
        new_end = new_end < Tc + open_tiles ? new_end : Tc + open_tiles;
        int t = T0;
        for (; t < ctx_end; ++t) iter(t, (t - T0) & 1, SX, std::integral_constant<int, 1>{});
        for (; t < T1 && t < Tc; ++t) iter(t, (t - T0) & 1, SX, Generic{});
        for (; t < new_end; ++t) iter(t, (t - T0) & 1, SX, std::integral_constant<int, 2>{});
        for (; t < T1; ++t) iter(t, (t - T0) & 1, SX, Generic{});
      }
      // leave ka / va pointing at buffer 0 for the next piece
      if (flip > 0) {
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) ka[ks] -= kBufBytes;
      } else {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int db = 0; db < 4; ++db) va[r][db] -= kBufBytes;
      }
    }

    // ---- epilogue ----
    auto emit = [&](int rix, int db, const f32x16& o, float mfin, float lfin) __attribute__((always_inline)) {
      if (rix < 0) return;
      const int tq = rix / G;
      const int g = rix - tq * G;
      const float inv = lfin > 0.f ? 1.f / lfin : 0.f;
      const long R = ((long)(q0 + tq) * p.Hq + kvh * G + g) * p.max_pieces + piece;
      float* wp = p.ws_o + R * kD + 32 * db + 4 * he;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        float4 w = {o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv, o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv};
        *reinterpret_cast<float4*>(wp + 8 * i4) = w;
      }
      if (db == 0 && he == 0) p.ws_lse[R] = lfin > 0.f ? mfin + __log2f(lfin) : -INFINITY;  // log2 domain
    };
    // rows of an uncut column go through an 8 KB strip of the (now free) tile buffers per wave, 64 columns at a
    // time, so that 8 lanes store the 128 contiguous bytes of a row; partial rows are stored directly
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
#ifdef ATTN_PROBE
  PROBE_T(6)
  if ((threadIdx.x & 63) == 0 && blockIdx.x < 128) {
    unsigned long long* o = g_probe + (blockIdx.x * 4 + (threadIdx.x >> 6)) * 8;
    for (int i = 0; i < 7; ++i) o[i] = pr_acc[i];
    o[7] = pr_last - pr_start;
  }
#endif
}

int launch_attn_fwd2(const AttnKParams& p, int grid, int dyn_lds, bool buf, hipStream_t stream) {
  if (buf) hipLaunchKernelGGL((attn_fwd2_kernel<true>), dim3((unsigned)grid), dim3(256), dyn_lds, stream, p);
  else hipLaunchKernelGGL((attn_fwd2_kernel<false>), dim3((unsigned)grid), dim3(256), dyn_lds, stream, p);
  return launch_status();
}

}  // namespace pdllm

#ifdef ATTN_PROBE
extern "C" int pdllm_debug_probe(unsigned long long* host_out) {
  return hipMemcpyFromSymbol(host_out, HIP_SYMBOL(pdllm::g_probe), sizeof(unsigned long long) * 8 * 1024) == hipSuccess ? 0 : -1;
}
#endif
