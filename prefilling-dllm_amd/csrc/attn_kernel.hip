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
//   ("slot B") are shared: J=6 -> blocks 4,5, each split between two waves that take one
//   32-key block of every tile; J=5 -> block 4 split over all four waves, two of them on even
//   tiles and two on odd tiles; J=8 -> a workgroup of 8 wavefronts, one block each.  J=1,2 have only shared
//   blocks (intra-workgroup split-KV for short active blocks).  Shared blocks are merged
//   through LDS with a log-sum-exp reduction.  An optional split over workgroups writes fp32
//   partials + LSE to a workspace that attn_merge_kernel reduces.
//   The tile buffers take 64 KB of LDS and a wave at most 256 registers, so two workgroups
//   share a CU: while one waits for the matrix unit the other runs its softmax.
//
// Per 64-key tile
//   K and V rows are copied HBM -> LDS without passing through registers (16 bytes per lane:
//   buffer_load ... lds with 32-bit offsets when every tensor is below 4 GiB, global_load_lds
//   otherwise); the row addresses come from the slot table that attn_slot_table_kernel builds
//   from the page table and the chunk ranges once per step, read two to three tiles ahead.
//   Rows are 256 bytes = 16 chunks; chunk c of row r is stored at position
//   c ^ swz(r) (attn_common.h), which makes the 128-bit K operand reads and the transposing
//   ds_read_b64_tr_b16 V operand reads bank-conflict free.
//   S^T = K Q^T and O^T += V^T P^T use v_mfma_f32_32x32x16_bf16; in the S^T accumulator
//   layout a lane holds 16 keys of one query, so softmax statistics are lane-local plus
//   one half-wave exchange, and P^T feeds the second MFMA straight from registers.
//   The S^T accumulators hold the raw fp32 dot products (first MFMA of a block starts from a zero
//   operand); the softmax scale is applied in fp32 as one fused multiply-add per score,
//   p = 2^(sm_scale * log2(e) * s - M), like the reference scales its fp32 dot product.  The
//   running maximum M is only advanced (and O rescaled) when a tile exceeds it by more than 2^8,
//   which removes most rescale work without changing the result.
//   fp8 e4m3 pages are dequantised (x * scale[page]) in registers while staging.
//   The tile loops exist in a general form and in "steady" forms for runs of whole, unmasked
//   tiles from one source, in which the mask, end-of-piece and copy-source decisions are
//   compile-time constants (a third fewer instructions per tile).

#include <cstdio>
#include <type_traits>

#include "attn_common.h"

namespace pdllm {

int launch_attn_fwd2(const AttnKParams& p, int grid, int dyn_lds, bool buf, hipStream_t stream);  // attn_kernel2.hip
// attn_prefill.hip: resident workgroups that walk a stream of tiles through all their columns (large prefills)
bool prefill_stream_plan(const pdllm_attn_desc* d, int cus, int* grid, int* team);
int launch_prefill_stream(const pdllm_attn_desc* d, int grid, int team, hipStream_t stream);

int kv_store_launch(const void* key, const void* value, void* k_cache, void* v_cache,
                    const int32_t* slot_mapping, int64_t n_tokens, int64_t row_elems,
                    int64_t key_stride, int64_t value_stride, int64_t n_slots, hipStream_t stream);

// Softmax update of one row block over NKB key blocks of 32 keys.  S holds the raw dot products
// q.k (fp32, the accumulators start at zero) in the S^T accumulator layout: element i of a lane is key
// 8*(i/4) + 4*h + i%4 of the block.  The softmax scale is applied here in fp32, as the reference
// scales the fp32 dot product: p = 2^(c * s - M) with c = sm_scale * log2(e) > 0 and the running
// maximum M kept in log2 units.
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
  float mx = fmaxf(S[0][0], S[0][1]);
#pragma unroll
  for (int b = 0; b < NKB; ++b)
#pragma unroll
    for (int i = (b == 0 ? 2 : 0); i < 16; i += 2) mx = fmaxf(fmaxf(mx, S[b][i]), S[b][i + 1]);
  mx = half_swap_max(mx) * c;  // log2 units; -inf (nothing visible) stays -inf
  // advance the reference maximum only when some row of the wave needs it (M = -inf: M + slack = -inf)
  const bool need = mx > M + kRescaleSlack;
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
  // p = 2^(c s - M) rounded to bf16; the row sum is taken over the rounded values, the same ones the
  // second MFMA multiplies with V
  const float negM = (M == -INFINITY) ? 0.f : -M;
  const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
  float psum = 0.f;
#pragma unroll
  for (int b = 0; b < NKB; ++b) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const bf16x2 pr = {(__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[b][8 * j + e], c, negM)),
                           (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[b][8 * j + e + 1], c, negM))};
        psum = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, psum, false);
        P[b][j][e] = pr[0];
        P[b][j][e + 1] = pr[1];
      }
  }
  l += psum;
}

// BUF (software-pipelined variants only): the K/V copies are buffer loads with a 32-bit byte offset per
// lane; the host selects it when every source tensor is smaller than 4 GiB.
// SPEC (fp8 pages): J waves with one row block each run the software-pipelined loop on bf16 tiles that three more
// waves write: they fetch the fp8 rows two tiles ahead, dequantise them and store them into LDS in the layout the
// direct copies produce.
template <int KV_FP8, int J, bool BUF = false, bool SPEC = false>
__global__ __launch_bounds__(SPEC ? 64 * (J + 3) : J == 8 ? 512 : 256, (SPEC || (KV_FP8 && J > 4)) ? 1 : 2) void attn_fwd_kernel(const AttnKParams p) {
  static_assert(!SPEC || (KV_FP8 && !BUF && J >= 4 && J <= 5), "producer waves serve fp8 pages only");
  constexpr int NW = SPEC ? J + 3 : J == 8 ? 8 : 4;  // wavefronts per workgroup
  constexpr int kDmaGroups = SPEC ? 1 : 16 / NW;      // a tile is 16 groups of 4 rows; a wave copies this many of them
  constexpr bool HAS_A = J >= 4;
  constexpr bool HAS_B = !SPEC && J != 4 && J != 8;
  constexpr int GS = (J == 1 || J == 5) ? 4 : (J == 2 || J == 6) ? 2 : 1;  // waves sharing a B block
  constexpr bool QB_LDS = !SPEC && (J == 5 || J == 6);  // Q of the shared block(s) lives in LDS, not in registers

  __shared__ __attribute__((aligned(1024))) char lds[kMainBytes];
  // SPEC: staging area of the three producer waves -- per wave three times six groups of 8 fp8 rows and two rows of
  // page scales (K and V), and four rows of slots, all filled by direct-to-LDS copies
  constexpr int kLead = 2;  // steps between the request of a tile's rows and their use
  constexpr int kRing = kLead + 1;
  constexpr int kStTile = 6 * 1024, kStScales = kRing * kStTile, kStSlots = kStScales + kRing * 512, kStBytes = kStSlots + 8 * 256;
  __shared__ __attribute__((aligned(1024))) char stage[SPEC ? 3 * kStBytes : 16];
  __shared__ float s_ml[4][2][32];
  // dynamic part: Q fragments of the shared blocks (QB_LDS), then the dense-mask bit rows
  // [2][kMaxTok][kNKB] of an active tile (one bit per key; only with PDLLM_MASK_DENSE)
  extern __shared__ __attribute__((aligned(16))) char dyn_lds[];
  constexpr int kQbBytes = QB_LDS ? (J - 4) * 8192 : 0;
  uint32_t (*s_maskbits)[kMaxTok][kNKB] = reinterpret_cast<uint32_t (*)[kMaxTok][kNKB]>(dyn_lds + kQbBytes);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int h = lane >> 5;

  const int G = p.G;
  const float c = p.scale_log2;
  const unsigned lds_base = (unsigned)(size_t)lds;  // LDS address of the tile buffers

  // per-lane LDS operand offsets (bytes inside a tile)
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

  // LDS addresses of this lane's operand fragments in buffer 0 (pipelined loop: the buffer and
  // key-block offsets are instruction immediates)
  unsigned ka[8], va[2][4];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) ka[ks] = lds_base + koff[ks];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int db = 0; db < 4; ++db) va[r][db] = lds_base + voff[r][db];

  // this workgroup's span of the tile line; it may cover the end of one column and the start of
  // the next, each part ("piece") is an attention pass of its own
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  int col0 = 0;      // first column of the line this workgroup works on
  int head_rt = -1;  // >= 0: this workgroup takes the head of that column of its set and nothing else
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
  const int tail_len = p.t_lin - p.head;  // positions of a column after its head
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
    // (the divisions run on the vector unit: bring the results back to scalar registers)
    tb = __builtin_amdgcn_readfirstlane(tb);
    te = tb + (y_end - y) < p.t_lin ? tb + (y_end - y) : p.t_lin;
    y += te - tb;
  }
  const int col = __builtin_amdgcn_readfirstlane(col0 + rt_lin);
  // The head of a column is its piece 0.  A later piece starts at a workgroup boundary, so its
  // number is the count of boundaries since the start of the column's tail.
  const int piece = __builtin_amdgcn_readfirstlane(tb < p.head ? 0 : (p.head > 0 ? 1 : 0) + (tb - p.head + p.span - 1) / p.span);
  const bool whole = tb == 0 && te == p.t_lin;  // the only piece: write the result, not a partial
  // causal: the row groups that see the most keys are dispatched first, the short ones fill the tail
  const int row_tile = p.mask_mode == PDLLM_MASK_CAUSAL ? p.row_tiles - 1 - col % p.row_tiles : col % p.row_tiles;
  const int kvh = (col / p.row_tiles) % p.Hkv;
  const int req = col / (p.row_tiles * p.Hkv);

  const int q0 = p.q_start_loc[req];
  const int Sq = p.q_start_loc[req + 1] - q0;
  if (q0 < 0 || Sq <= 0 || (long)q0 + Sq > p.n_tokens || Sq > p.max_q_len) continue;
  const int rows = Sq * G;
  const int row0 = row_tile * 32 * J;
  if (row0 >= rows) continue;
  // lane coordinates for the prologue and epilogue of a piece, made opaque per piece so that the
  // address arithmetic built on them is not hoisted out of the piece loop (it would stay live in
  // registers through the tile loop)
  int lane_e = lane;
  asm volatile("" : "+v"(lane_e));
  const int l32e = lane_e & 31;
  const int he = lane_e >> 5;

  // visible prefix keys of this request: count and slots come from the slot table
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

  if constexpr (SPEC) {
    if (wave >= J) {
    // ---- producer waves (SPEC) ----
    // Tile u of a piece lives in buffer (u - T0) & 1, for K as for V.  A tile is eight groups of 8 rows for K and
    // eight for V: wave J takes groups 0-5 of K, wave J + 1 groups 0-5 of V, wave J + 2 groups 6, 7 of both.
    // Everything a producer fetches goes into its staging area by direct-to-LDS copies, so nothing in flight
    // sits in registers: the slots of tile u + 3 (one per lane), then, with the slots of tile u + 2 read back,
    // its page scales and its fp8 rows (lane l: 16 values of row 8 g + l / 8).  Then it reads tile u, requested
    // two steps ago, dequantises it and stores it in the layout the bf16 copies produce.
    // The waits count memory operations, so every step issues the same number, for tiles past the end of the
    // prefix with the last prefix tile's addresses (never read).  Tiles of the active block are bf16 and are
    // copied straight into the tile buffer in the step that would have written them.
    // (The launcher has checked that slots and strides fit 24-bit multiplies and the caches 32-bit offsets.)
    auto lds_copy4 = [&](const void* src, char* dst) __attribute__((always_inline)) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)dst, 4, 0, 0);
    };
    auto lds_copy16 = [&](const void* src, char* dst) __attribute__((always_inline)) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };
    auto run_producer = [&](auto pw_tag) __attribute__((always_inline)) {
      constexpr int PW = decltype(pw_tag)::value;
      constexpr int NPL = PW == 2 ? 4 : 6;  // places: (tensor, group of 8 rows)
      constexpr int NSC = PW == 2 ? 2 : 1;  // scale rows: K, V or both
      constexpr int NF = NSC + NPL;         // copies of one tile's scales and rows
      auto place_is_k = [](int j) { return PW == 0 || (PW == 2 && j < 2); };
      auto place_group = [](int j) { return PW < 2 ? j : 6 + (j & 1); };
      const bool pfetch = T0 < Tc;  // this piece has prefix tiles
      int pu = T0;                  // the tile (of K's numbering) of the next step
      int pset = 0;                 // (pu - T0) % kRing: staging tile of its rows
      const unsigned st_base = (unsigned)(size_t)stage + PW * kStBytes;
      char* const st_ptr = stage + PW * kStBytes;
      // (lane coordinates made opaque per piece: as loop invariants of the kernel the addresses built on them would
      // be spilled, and a reload waits for every copy in flight)
      int lane_p = lane;
      asm volatile("" : "+v"(lane_p));
      const int p_row = lane_p >> 3, p_f = lane_p & 7;
      const char* pk_cache = static_cast<const char*>(p.k_cache) + (long)kvh * p.cache_head_stride + 16 * p_f;
      const char* pv_cache = static_cast<const char*>(p.v_cache) + (long)kvh * p.cache_head_stride + 16 * p_f;
      const float* pk_scale = p.k_scale + (long)kvh * p.scale_head_stride;
      const float* pv_scale = p.v_scale + (long)kvh * p.scale_head_stride;
      const unsigned tstride = (unsigned)p.cache_token_stride, sstride = (unsigned)p.scale_page_stride * 4u;
      auto prod_slots = [&](int v) __attribute__((always_inline)) {  // request the slots of tile v
        const int vv = v < Tc ? v : Tc - 1;
        lds_copy4(tbl + (long)vv * kKT + lane_p, st_ptr + kStSlots + ((v - T0) & 7) * 256);
      };
      // The third producer follows K's schedule, which runs one tile ahead of V's (iteration t of the other
      // waves needs K(t+2) and V(t+1)): in the step of tile w its V places hold tile w - 1, in the first two
      // steps T0.
      auto v_tile = [&](int w) __attribute__((always_inline)) { return PW == 2 && w > T0 ? w - 1 : w; };
      // request scales and rows for the step of tile w; the slots have landed.  set = (w - T0) % kRing
      auto prod_fetch = [&](int w, int set) __attribute__((always_inline)) {
        const unsigned sbk = st_base + kStSlots + ((w - T0) & 7) * 256;
        const unsigned sbv = st_base + kStSlots + ((v_tile(w) - T0) & 7) * 256;
        int sl[NPL], so[NSC];
#pragma unroll
        for (int i = 0; i < NSC; ++i)
          asm volatile("ds_read_b32 %0, %1" : "=v"(so[i]) : "v"((i == 0 && PW != 1 ? sbk : sbv) + 4 * lane_p) : "memory");
#pragma unroll
        for (int j = 0; j < NPL; ++j)
          asm volatile("ds_read_b32 %0, %1" : "=v"(sl[j]) : "v"((place_is_k(j) ? sbk : sbv) + 4 * (8 * place_group(j) + p_row)) : "memory");
        if constexpr (PW == 2)
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sl[0]), "+v"(sl[1]), "+v"(sl[2]), "+v"(sl[3]), "+v"(so[0]), "+v"(so[1]) : : "memory");
        else
          asm volatile("s_waitcnt lgkmcnt(0)"
                       : "+v"(sl[0]), "+v"(sl[1]), "+v"(sl[2]), "+v"(sl[3]), "+v"(sl[4]), "+v"(sl[5]), "+v"(so[0])
                       :
                       : "memory");
#pragma unroll
        for (int i = 0; i < NSC; ++i) {
          const float* sp = (i == 0 && PW != 1) ? pk_scale : pv_scale;
          lds_copy4(reinterpret_cast<const char*>(sp) + __umul24((unsigned)(so[i] >> p.page_shift), sstride),
                    st_ptr + kStScales + set * 512 + i * 256);
        }
#pragma unroll
        for (int j = 0; j < NPL; ++j)
          lds_copy16((place_is_k(j) ? pk_cache : pv_cache) + __umul24((unsigned)sl[j], tstride),
                     st_ptr + set * kStTile + j * 1024);
      };
      // dequantise and store what was fetched for the step of tile w
      auto prod_write = [&](int w, int set) __attribute__((always_inline)) {
        const int wv = v_tile(w);
        const int lim = T1 < Tc ? T1 : Tc;  // prefix tiles of this piece end here
        if (w < lim || wv < lim) {
          typedef unsigned u32v4 __attribute__((ext_vector_type(4)));
          u32v4 d[NPL];
          float sc[NPL];
          const unsigned db = st_base + set * kStTile + 16 * lane_p, scb = st_base + kStScales + set * 512 + 4 * p_row;
#pragma unroll
          for (int j = 0; j < NPL; ++j) {
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(d[j]) : "v"(db), "n"(j * 1024) : "memory");
            // (scale row 0 is K's for the first and the third producer, V's for the second; row 1 is V's)
            if (place_is_k(j) || PW == 1)
              asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(sc[j]) : "v"(scb), "n"(32 * place_group(j)) : "memory");
            else
              asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(sc[j]) : "v"(scb), "n"(256 + 32 * place_group(j)) : "memory");
          }
          if constexpr (PW == 2)
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]), "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3])
                         :
                         : "memory");
          else
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]), "+v"(d[4]), "+v"(d[5]),
                           "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]), "+v"(sc[4]), "+v"(sc[5])
                         :
                         : "memory");
#pragma unroll
          for (int j = 0; j < NPL; ++j) {
            const int x = place_is_k(j) ? w : wv;
            if (x >= lim) continue;
            const int r16 = 8 * (j & 1) + p_row;  // row & 15: every place's group has the parity of the place
            const unsigned r = lds_base + ((x - T0) & 1) * kBufBytes + (place_is_k(j) ? 0 : kTileBytes) +
                               (8 * place_group(j) + p_row) * kRowBytes;
            const uint4 lo = dequant_fp8x8(d[j].x, d[j].y, sc[j]), hi = dequant_fp8x8(d[j].z, d[j].w, sc[j]);
            const u32v4 lov = {lo.x, lo.y, lo.z, lo.w}, hiv = {hi.x, hi.y, hi.z, hi.w};
            asm volatile("ds_write_b128 %0, %1" : : "v"(r + (((2 * p_f) ^ swz(r16)) << 4)), "v"(lov) : "memory");
            asm volatile("ds_write_b128 %0, %1" : : "v"(r + (((2 * p_f + 1) ^ swz(r16)) << 4)), "v"(hiv) : "memory");
          }
        }
        if (PW < 2 && w >= Tc && w < T1) {
          const __bf16* nb = PW == 0 ? p.k_new + (long)q0 * p.kn_stride : p.v_new + (long)q0 * p.vn_stride;
          const long nstride = PW == 0 ? p.kn_stride : p.vn_stride;
          const int a0 = (w - Tc) * kKT;
          char* tp = lds + ((w - T0) & 1) * kBufBytes + (PW == 0 ? 0 : kTileBytes);
#pragma unroll
          for (int gg = 0; gg < 16; ++gg) {
            const int row = 4 * gg + (lane_p >> 4);
            const int a = a0 + row < Sa ? a0 + row : a0;  // padding rows copy a valid row; they are masked
            const int ch = (lane_p & 15) ^ swz(row);
            lds_copy16(nb + a * nstride + kvh * kD + 8 * ch, tp + gg * 1024);
          }
          asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // the copies have landed
        }
      };
      if (pfetch) {
#pragma unroll
        for (int i = 0; i <= kLead; ++i) prod_slots(pu + i);
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#pragma unroll
        for (int i = 0; i < kLead; ++i) prod_fetch(pu + i, i);
      }
      // Step 0 writes tile T0 into buffer 0; step 1, not for the V producer, K(T0 + 1) into buffer 1 while the
      // other waves compute the first scores; step 2 + i belongs to iteration T0 + i of the other waves and
      // writes K(T0 + i + 2) or V(T0 + i + 1).  One barrier per step, as many as the other waves pass.
      // Memory operations in issue order: ... slots(u+2), rows(u+1) | slots(u+3), rows(u+2), "rows" being the
      // NF copies of scales and rows: the slots of tile u + 2 have landed when at most the NF operations of
      // rows(u+1) are outstanding, the rows of tile u when at most the kLead (NF + 1) issued after them are.
      const int nsteps = T1 - T0 + 2;
      for (int i = 0; i < nsteps; ++i) {
        if (i != 1 || PW != 1) {
          if (pfetch) {
            asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NF) : "memory");
            prod_slots(pu + kLead + 1);
            prod_fetch(pu + kLead, pset == 0 ? kLead : pset - 1);
            asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kLead * (NF + 1)) : "memory");
          }
          prod_write(pu, pset);
          ++pu;
          pset = pset == kLead ? 0 : pset + 1;
        }
        // (waits for this wave's LDS stores only: what it has requested for later tiles stays in flight)
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
        __builtin_amdgcn_s_barrier();
      }
    };

      if (T0 < T1) {
        if (wave == J) run_producer(std::integral_constant<int, 0>{});
        else if (wave == J + 1) run_producer(std::integral_constant<int, 1>{});
        else run_producer(std::integral_constant<int, 2>{});
      }
      if (head_rt >= 0 || y < y_end) {  // (the barrier between two pieces, as at the end of this loop)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
      }
      continue;
    }
  }

  // ---- row blocks of this wave ----
  const int blkA = wave;
  const int gi = wave & (GS - 1);  // index of this wave among the GS waves sharing its B block
  int blkB = -1;
  if (J == 1) blkB = 0;
  else if (J == 2) blkB = wave >> 1;
  else if (J == 5) blkB = 4;
  else if (J == 6) blkB = 4 + (wave >> 1);
  const int kbB = gi & 1;       // key block of a tile this wave handles for a shared block
  const int parB = (gi >> 1) ^ (row_tile & 1);  // GS == 4: tiles of this parity only

  // ---- Q fragments (B operand of S^T = K Q^T), rows of this lane, scaled to log2 units ----
  bf16x8 QA[8], QB[8];
  int srowA = 0, srowB = 0, ridxA = -1, ridxB = -1;
  auto load_q = [&](int blk, bf16x8 (&Q)[8], int& srow, int& ridx) __attribute__((always_inline)) {
    const int r = row0 + 32 * blk + l32e;
    const bool valid = blk >= 0 && r < rows && (!SPEC || blk < J);
    const int rr = valid ? r : 0;
    const int tq = rr / G;
    const int g = rr - tq * G;
    srow = tq;
    ridx = valid ? r : -1;
    const __bf16* qp = p.q + (long)(q0 + tq) * p.q_stride + (long)(kvh * G + g) * kD + 8 * he;
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
  if (HAS_B) load_q(blkB, QB, srowB, ridxB);
  // shared block with a slot A next to it: park its fragments in LDS as [block][ks][lane] x 16 B
  // (every wave of the group holds the same values; the first one writes)
  const int qb_off = QB_LDS ? (blkB - 4) * 8192 + lane * 16 : 0;
  const int qb_off_e = QB_LDS ? (blkB - 4) * 8192 + lane_e * 16 : 0;
  if (QB_LDS && gi == 0) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) *reinterpret_cast<bf16x8*>(dyn_lds + qb_off_e + ks * 1024) = QB[ks];
  }

  f32x16 OA[4], OB[4];
  float MA = -INFINITY, MB = -INFINITY, lA = 0.f, lB = 0.f;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { OA[db][i] = 0.f; OB[db][i] = 0.f; }

  // dense mask of active tile t -> bit rows in LDS (built one tile ahead, like the slot table)
  const uint8_t* mask_base = p.mask != nullptr ? p.mask + (long)q0 * p.mask_stride + q0 : nullptr;
  const int tq_first = row0 / G;
  int ntok = ((row0 + 32 * J < rows ? row0 + 32 * J : rows) - 1) / G - tq_first + 1;
  ntok = ntok < kMaxTok ? ntok : kMaxTok;
  auto build_mask = [&](int t, int par) __attribute__((always_inline)) {
    if (p.mask_mode != PDLLM_MASK_DENSE || t < Tc) return;
    if (SPEC && wave >= J) return;  // (the producer waves never get here)
    const int a0 = (t - Tc) * kKT;
    for (int idx = tid; idx < ntok * kNKB; idx += (SPEC ? J : NW) * 64) {
      const int tok = idx / kNKB, w = idx % kNKB;
      const uint8_t* mp = mask_base + (long)(tq_first + tok) * p.mask_stride + a0 + 32 * w;
      uint32_t bits = 0;
      for (int j = 0; j < 32; ++j)
        if (a0 + 32 * w + j < Sq && mp[j] != 0) bits |= 1u << j;
      s_maskbits[par][tok][w] = bits;
    }
  };

  // fp8 staging registers (only used by the fp8 instantiations)
  uint2 st_k[kDmaGroups], st_v[kDmaGroups];
  float st_ks[kDmaGroups], st_vs[kDmaGroups];

  // Copy of tile t into buffer `buf`: this wave moves rows 4*NW*i + 4*wave + lane/16 for
  // i < kDmaGroups, one instruction for K and one for V each.  The chunk a lane fetches,
  // (lane & 15) ^ swz(row), does not depend on i because the swizzle has period 16.
  // The source rows are cache slots read from the slot table (prefix tiles) or rows of the
  // active block; they are fetched into registers one tile before the copy is issued.
  const int lane_row = 4 * wave + (lane >> 4);
  const int lane_ch = (lane & 15) ^ swz(lane_row);
  const long cache_lane_off = ((long)kvh * p.cache_head_stride + 8 * lane_ch) * (KV_FP8 ? 1 : 2);
  const char* kc_lane = static_cast<const char*>(p.k_cache) + cache_lane_off;
  const char* vc_lane = static_cast<const char*>(p.v_cache) + cache_lane_off;
  const char* kn_lane = reinterpret_cast<const char*>(p.k_new + (long)q0 * p.kn_stride + kvh * kD + 8 * lane_ch);
  const char* vn_lane = reinterpret_cast<const char*>(p.v_new + (long)q0 * p.vn_stride + kvh * kD + 8 * lane_ch);
  const unsigned cache_row16 = (unsigned)((p.cache_token_stride * (KV_FP8 ? 1 : 2)) >> 4);  // 16-byte units
  const unsigned kn_row16 = (unsigned)((p.kn_stride * 2) >> 4);
  const unsigned vn_row16 = (unsigned)((p.vn_stride * 2) >> 4);
  int nslot[kDmaGroups];
  // the same for a tile known to be a whole tile of the prefix / of the active block
  // (uniform 64-bit base + 32-bit lane offset + immediate: no vector address arithmetic per tile)
  const unsigned lane_row_b = (unsigned)lane_row * 4u;
  auto load_slots_ctx = [&](int t) __attribute__((always_inline)) {
    const char* tile_tbl = reinterpret_cast<const char*>(tbl + (long)t * kKT);
#pragma unroll
    for (int i = 0; i < kDmaGroups; ++i)
      nslot[i] = *reinterpret_cast<const int*>(tile_tbl + (unsigned long)lane_row_b + 16 * NW * i);
  };
  // (rows past the active block -- a ragged last tile, or a tile past the end of the piece that is copied
  // but never read -- repeat the last row: always a valid address)
  auto load_slots_new = [&](int t) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kDmaGroups; ++i) {
      const int a = (t - Tc) * kKT + 4 * NW * i + lane_row;
      nslot[i] = a < Sa ? a : Sa - 1;
    }
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
  // The whole copy of a tile is issued in one burst at the start of the tile before (handing the
  // copy instructions out between the MFMAs measured slower).
  // (known_ctx: the tile is known to be a tile of the prefix)
  auto issue_tile = [&](int t, int buf, auto known_ctx) __attribute__((always_inline)) {
    const bool ctx = decltype(known_ctx)::value || t < Tc;
    const char* kb = ctx ? kc_lane : kn_lane;
    const char* vb = ctx ? vc_lane : vn_lane;
    const unsigned kr = ctx ? cache_row16 : kn_row16;
    const unsigned vr = ctx ? cache_row16 : vn_row16;
    char* dst = lds + buf * kBufBytes + wave * 1024;
    if (KV_FP8 && ctx) {
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) {
        st_k[i] = *reinterpret_cast<const uint2*>(kb + ((unsigned long)((unsigned)nslot[i] * kr) << 4));
        st_v[i] = *reinterpret_cast<const uint2*>(vb + ((unsigned long)((unsigned)nslot[i] * vr) << 4));
        const long so = (long)(nslot[i] >> p.page_shift) * p.scale_page_stride + (long)kvh * p.scale_head_stride;
        st_ks[i] = p.k_scale[so];
        st_vs[i] = p.v_scale[so];
      }
    } else {
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) {
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(kb + ((unsigned long)((unsigned)nslot[i] * kr) << 4)),
            (__attribute__((address_space(3))) void*)(dst + i * (NW * 1024)), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(vb + ((unsigned long)((unsigned)nslot[i] * vr) << 4)),
            (__attribute__((address_space(3))) void*)(dst + i * (NW * 1024) + kTileBytes), 16, 0, 0);
      }
    }
  };
  // fp8: dequantise the staged rows into the LDS tile (same layout the direct copies produce)
  auto finish_tile = [&](int t, int buf, auto known_ctx) __attribute__((always_inline)) {
    if (KV_FP8 && (decltype(known_ctx)::value || t < Tc)) {
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) {
        char* kdst = lds + buf * kBufBytes + (i * NW + wave) * 1024 + lane * 16;
        *reinterpret_cast<uint4*>(kdst) = dequant_fp8x8(st_k[i].x, st_k[i].y, st_ks[i]);
        *reinterpret_cast<uint4*>(kdst + kTileBytes) = dequant_fp8x8(st_v[i].x, st_v[i].y, st_vs[i]);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct-to-LDS copies have landed
  };

  // ---- one pass: row block(s) x NKB key blocks of the tile in LDS ----
  // Operand reads run two steps ahead of the MFMAs; the scheduling barriers keep that order.
  auto pass = [&](bool generic, auto nkb_tag, auto fora_tag, int kb_first, int bufoff,
                  int nvalid, bool active, int a0, int par) __attribute__((always_inline)) {
    constexpr int NKB = decltype(nkb_tag)::value;
    constexpr bool forA = decltype(fora_tag)::value;
    constexpr bool QLDS = QB_LDS && !forA;
    const int kbase_bytes = bufoff + kb_first * 32 * kRowBytes;
    const int vbase_bytes = kbase_bytes + kTileBytes;
    bf16x8 (&Q1)[8] = forA ? QA : QB;
    f32x16 (&O1)[4] = forA ? OA : OB;
    float& M1 = forA ? MA : MB;
    float& l1 = forA ? lA : lB;
    const int srow1 = forA ? srowA : srowB;

    f32x16 S1[NKB];
#pragma unroll
    for (int b = 0; b < NKB; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) S1[b][i] = 0.f;
    if constexpr (!QLDS) {
      constexpr int PF = 4;  // operand reads run PF steps ahead of the MFMAs (LDS latency ~ 3-4 MFMAs)
      constexpr int NS = 8 * NKB;
      unsigned ka[8];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) ka[ks] = lds_base + koff[ks] + kbase_bytes;
      auto rdk = [&](bf16x8& dst, int stp) __attribute__((always_inline)) {
        if ((stp >> 3) == 0) lds_read_b128<0>(dst, ka[stp & 7]);
        else lds_read_b128<32 * kRowBytes>(dst, ka[stp & 7]);
      };
      bf16x8 kf[PF];
#pragma unroll
      for (int i = 0; i < PF; ++i) rdk(kf[i], i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int stp = 0; stp < NS; ++stp) {
        const int kb = stp >> 3, ks = stp & 7;
        const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;  // reads issued after this step's
        if (young == 3) lds_wait<3>(kf[stp % PF]);
        else if (young == 2) lds_wait<2>(kf[stp % PF]);
        else if (young == 1) lds_wait<1>(kf[stp % PF]);
        else lds_wait<0>(kf[stp % PF]);
        const bf16x8 cur = kf[stp % PF];
        S1[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur, Q1[ks], S1[kb], 0, 0, 0);
        if (stp + PF < NS) rdk(kf[stp % PF], stp + PF);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      // shared block next to a slot A: K and Q fragments both come from LDS (compiler-managed reads)
      auto ldk = [&](int stp) __attribute__((always_inline)) {
        const int kb = stp >> 3, ks = stp & 7;
        return *reinterpret_cast<const bf16x8*>(lds + koff[ks] + kbase_bytes + kb * 32 * kRowBytes);
      };
      auto ldq = [&](int stp) __attribute__((always_inline)) {
        return *reinterpret_cast<const bf16x8*>(dyn_lds + qb_off + (stp & 7) * 1024);
      };
      constexpr int PF = 4;
      bf16x8 kf[PF], qf[PF];
#pragma unroll
      for (int i = 0; i < PF; ++i) { kf[i] = ldk(i); qf[i] = ldq(i); }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int stp = 0; stp < 8 * NKB; ++stp) {
        const int kb = stp >> 3;
        S1[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], qf[stp % PF], S1[kb], 0, 0, 0);
        if (stp + PF < 8 * NKB) { kf[stp % PF] = ldk(stp + PF); qf[stp % PF] = ldq(stp + PF); }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    bf16x8 P1[NKB][2];
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
    __builtin_amdgcn_sched_barrier(0);
    {
      typedef __attribute__((ext_vector_type(8))) short s16x8;
      constexpr int NS = 8 * NKB;
      // step = (kj, db): V^T fragment of keys 16 kj .. +16 of the pass, columns 32 db .. +32
      unsigned va[2][4];
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int db = 0; db < 4; ++db) va[r][db] = lds_base + voff[r][db] + vbase_bytes;
      auto rdv = [&](s16x4& dst, int stp, int r) __attribute__((always_inline)) {
        const int db = stp & 3, kj = stp >> 2;
        if (kj == 0) lds_read_tr16_b64<0>(dst, va[r][db]);
        else if (kj == 1) lds_read_tr16_b64<16 * kRowBytes>(dst, va[r][db]);
        else if (kj == 2) lds_read_tr16_b64<32 * kRowBytes>(dst, va[r][db]);
        else lds_read_tr16_b64<48 * kRowBytes>(dst, va[r][db]);
      };
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
        O1[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, P1[kj >> 1][kj & 1], O1[db], 0, 0, 0);
        if (stp + 2 < NS) { rdv(lo[stp & 1], stp + 2, 0); rdv(hi[stp & 1], stp + 2, 1); }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // steady_tag: tiles t .. t + 2 are whole tiles of the prefix inside this piece (nothing to mask, copies from the
  // cache, no end-of-piece cases): the same code with those decisions made at compile time
  auto compute = [&](bool generic, int t, int buf, bool has_next, auto steady_tag) __attribute__((always_inline)) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    const int bufoff = buf * kBufBytes;
    const bool active = !STEADY && t >= Tc;
    const int a0 = active ? (t - Tc) * kKT : 0;
    int nvalid = STEADY ? kKT : active ? Sa - a0 : ctx_total - t * kKT;
    nvalid = nvalid < kKT ? nvalid : kKT;
    using N1 = std::integral_constant<int, 1>;
    using NT = std::integral_constant<int, kNKB>;
    if (has_next) issue_tile(t + 1, buf ^ 1, steady_tag);
    if (STEADY) load_slots_ctx(t + 2);
    else if (t + 2 < T1) load_slots(t + 2);
    if (HAS_A) pass(generic, NT{}, std::true_type{}, 0, bufoff, nvalid, active, a0, buf);
    if (HAS_B) {
      if (GS == 2 || ((t & 1) == parB))
        pass(generic, N1{}, std::false_type{}, kbB, bufoff, nvalid, active, a0, buf);
    }
  };

  auto step = [&](int t, auto steady_tag) __attribute__((always_inline)) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    const int rel = t - T0;
    const int buf = rel & 1;
    if (!STEADY && t + 1 < T1) build_mask(t + 1, buf ^ 1);
    const bool active = !STEADY && t >= Tc;
    const int a0 = active ? (t - Tc) * kKT : 0;
    const int nv = STEADY ? kKT : active ? Sa - a0 : ctx_total - t * kKT;
    const bool generic = !STEADY && (nv < kKT || (active && p.mask_mode != PDLLM_MASK_FULL));
    compute(generic, t, buf, STEADY || t + 1 < T1, steady_tag);
    if (STEADY || t + 1 < T1) finish_tile(t + 1, buf ^ 1, steady_tag);
    __syncthreads();
  };

  // ------------------------------------------------------------------------------------------
  // Software-pipelined tile loop (one own row block per wave, bf16 cache).  While the vector
  // unit turns the scores of tile t into probabilities, the matrix unit already computes the
  // scores of tile t + 1: each step issues one MFMA of QK(t+1) and the exponentials of two
  // elements of tile t.  K therefore runs one tile ahead of V in the buffers: iteration t
  // reads K(t+1) and V(t) and copies K(t+2) and V(t+1).  The last MFMA of a key block writes
  // into the registers the finished exponentials have just released, so the new scores are in
  // place for the next iteration without moves.  Every QK step and every PV step is one asm
  // statement (attn_common.h: qk_step, pv_step): its order is fixed, the MFMA comes first and
  // nothing is inserted between its parts.  Between the PV steps runs the row maximum of tile
  // t + 1, so that an iteration over an unmasked tile starts with its maximum known.
  // ------------------------------------------------------------------------------------------
  constexpr bool PIPELINED = ((J == 4 || J == 8) && !KV_FP8) || SPEC;
  if constexpr (PIPELINED) {
    if (T0 < T1) {
      typedef __attribute__((ext_vector_type(8))) short s16x8;
      int nsv[kDmaGroups];  // slots of the next V tile (nslot holds those of the next K tile)
      // source of a row = uniform base + 16 B * (slot * row pitch + chunk of this lane)
      const char* kc_base = static_cast<const char*>(p.k_cache) + (long)kvh * p.cache_head_stride * 2;
      const char* vc_base = static_cast<const char*>(p.v_cache) + (long)kvh * p.cache_head_stride * 2;
      const char* kn_base = reinterpret_cast<const char*>(p.k_new + (long)q0 * p.kn_stride + kvh * kD);
      const char* vn_base = reinterpret_cast<const char*>(p.v_new + (long)q0 * p.vn_stride + kvh * kD);
      // BUF: a buffer load with the LDS bit (resource descriptor made from the uniform base, 32-bit byte
      // offset per lane from one 24-bit multiply-add) costs the issuing wave about 15 clk, the
      // flat-address form 60 and more.
      const unsigned lane_b16 = (unsigned)lane_ch << 4;
      // LDS address of this wave's part of buffer 0; made opaque once per iteration so that the copy destinations
      // are one scalar add each (as loop invariants they would be sixteen spilled scalars in the unrolled loops)
      unsigned wave_lds = lds_base + wave * 1024;
      auto copy_row = [&](const char* base, unsigned row16, int slot, unsigned dst_off) __attribute__((always_inline)) {
        auto* dst = (__attribute__((address_space(3))) char*)(size_t)(wave_lds + dst_off);
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
      // src_tag: 0 = decide by the tile number, 1 = the tile is known to come from the cache, 2 = from the new rows
      auto issue_k1 = [&](int t, int buf, int i, auto src_tag) __attribute__((always_inline)) {
        constexpr int SRC = decltype(src_tag)::value;
        const bool ctx = SRC == 1 || (SRC == 0 && t < Tc);
        copy_row(ctx ? kc_base : kn_base, ctx ? cache_row16 : kn_row16, nslot[i],
                 (unsigned)(buf * kBufBytes + i * (NW * 1024)));
      };
      auto issue_v1 = [&](int t, int buf, int i, auto src_tag) __attribute__((always_inline)) {
        constexpr int SRC = decltype(src_tag)::value;
        const bool ctx = SRC == 1 || (SRC == 0 && t < Tc);
        copy_row(ctx ? vc_base : vn_base, ctx ? cache_row16 : vn_row16, nsv[i],
                 (unsigned)(buf * kBufBytes + kTileBytes + i * (NW * 1024)));
      };
      auto issue_k = [&](int t, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) issue_k1(t, buf, i, std::integral_constant<int, 0>{});
      };
      auto issue_v = [&](int t, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) issue_v1(t, buf, i, std::integral_constant<int, 0>{});
      };
      // K fragment read of QK step stp / V^T fragment read of PV step stp; ka and va point into the
      // buffer in use and move to the other one after every tile
      // (par_tag: -1 = as described; 0 / 1 = an iteration of known buffer parity in a loop unrolled by two,
      // where ka and va stay on buffer 0 and the buffer is part of the immediate offset)
      auto rdkp = [&](bf16x8& dst, int stp, auto par_tag) __attribute__((always_inline)) {
        constexpr int boff = decltype(par_tag)::value == 0 ? kBufBytes : 0;  // K(t+1) of an even iteration: buffer 1
        if ((stp >> 3) == 0) lds_read_b128<boff>(dst, ka[stp & 7]);
        else lds_read_b128<boff + 32 * kRowBytes>(dst, ka[stp & 7]);
      };
      auto rdk = [&](bf16x8& dst, int stp) __attribute__((always_inline)) { rdkp(dst, stp, std::integral_constant<int, -1>{}); };
      auto rdv = [&](s16x4& dst, int stp, int r, auto par_tag) __attribute__((always_inline)) {
        constexpr int base = kTileBytes + (decltype(par_tag)::value == 1 ? kBufBytes : 0);  // V(t) of an odd iteration: buffer 1
        const int db = stp & 3, kj = stp >> 2;
        if (kj == 0) lds_read_tr16_b64<base>(dst, va[r][db]);
        else if (kj == 1) lds_read_tr16_b64<base + 16 * kRowBytes>(dst, va[r][db]);
        else if (kj == 2) lds_read_tr16_b64<base + 32 * kRowBytes>(dst, va[r][db]);
        else lds_read_tr16_b64<base + 48 * kRowBytes>(dst, va[r][db]);
      };
      constexpr int PF = BUF ? 2 : 3, NS = 16;  // K fragments read ahead (what the register budget allows)
      auto wait_k = [&](bf16x8& x, int stp) __attribute__((always_inline)) {
        const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;
        if (young == 3) lds_wait<3>(x);
        else if (young == 2) lds_wait<2>(x);
        else if (young == 1) lds_wait<1>(x);
        else lds_wait<0>(x);
      };

      // one iteration: softmax of tile t (scores in Sc) interleaved with QK of tile t + 1 (into Sn),
      // then PV of tile t.  PAR = buffer of V(t); K(t+1) sits in the other buffer.
      int flip = kBufBytes;  // ka: buffer 1 -> 0 -> 1 ..., va: buffer 0 -> 1 -> 0 ...
      float mx_carry = 0.f;  // unmasked row maximum (log2 units) of the scores the next iteration starts with
      // steady (mode 1 / 2): tiles t .. t + 3 are whole tiles of the prefix / of the active block, lie inside this
      // piece, and tile t needs no mask for any row -- every copy comes from one tensor, nothing to mask, no
      // end-of-piece cases (the same code with those decisions made at compile time)
      auto iter = [&](int t, int par_rt, f32x16 (&Sc)[2], auto steady_tag, auto par_tag) __attribute__((always_inline)) {
        constexpr int PARC = decltype(par_tag)::value;
        const int PAR = PARC >= 0 ? PARC : par_rt;
        asm volatile("" : "+s"(wave_lds));
        constexpr int MODE = decltype(steady_tag)::value;
        constexpr bool STEADY = MODE != 0;
        const bool has_next = STEADY || t + 1 < T1;
        // The copies of V(t+1) (slots in nsv) and K(t+2) (slots in nslot) are handed out one per
        // second step of the QK loop below: a burst would block the wave on the memory pipeline.
        const bool k_on = STEADY || t + 2 < T1;
        if (!STEADY && has_next) build_mask(t + 1, PAR ^ 1);

        const bool active = !STEADY && t >= Tc;
        const int a0 = active ? (t - Tc) * kKT : 0;
        int nvalid = STEADY ? kKT : active ? Sa - a0 : ctx_total - t * kKT;
        const bool generic = !STEADY && (nvalid < kKT || (active && p.mask_mode != PDLLM_MASK_FULL));
        nvalid = nvalid < kKT ? nvalid : kKT;
        // ---- masks, row maximum, lazy rescale (vector unit only) ----
        if (generic) {
          int lim = nvalid;
          if (active && p.mask_mode == PDLLM_MASK_CAUSAL) { const int cl = srowA - a0 + 1; lim = cl < lim ? cl : lim; }
          int tl = srowA - tq_first;
          tl = tl < 0 ? 0 : (tl >= kMaxTok ? kMaxTok - 1 : tl);
          const uint32_t* mrow = (active && p.mask_mode == PDLLM_MASK_DENSE) ? &s_maskbits[PAR][tl][0] : nullptr;
          // a causal tile that lies below the diagonal for every row of this wave needs no mask
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
                Sc[b][i] = (W & bit) ? Sc[b][i] : -INFINITY;
              }
            }
          }
        }
        // A steady tile has no mask: its row maximum was taken from the finished scores during the PV
        // phase of the iteration before (or the prologue), where the vector unit idles under the MFMAs.
        float mx;
        if constexpr (STEADY) {
          mx = mx_carry;
        } else {
          mx = fmaxf(Sc[0][0], Sc[0][1]);
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = (b == 0 ? 2 : 0); i < 16; i += 2) mx = fmaxf(fmaxf(mx, Sc[b][i]), Sc[b][i + 1]);
          mx = half_swap_max(mx) * c;  // log2 units
        }
        const bool need = mx > MA + kRescaleSlack;
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
          const float Mn = fmaxf(MA, mx);
          const float alpha = (Mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(MA - Mn);
          MA = Mn;
          lA *= alpha;
#pragma unroll
          for (int db = 0; db < 4; ++db) {
#pragma unroll
            for (int i = 0; i < 16; ++i) OA[db][i] *= alpha;
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        // ---- exponentials of tile t, two per step, between the MFMAs of QK(t+1) ----
        float negM = (MA == -INFINITY) ? 0.f : -MA;
        f32x16 Sn[2];
        typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
        u32x4 PW[2][2];  // probabilities of tile t, two bf16 per word: the B operands of PV
        const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
        float psum = 0.f;
        if (has_next) {
          bf16x8 kf[PF];
#pragma unroll
          for (int i = 0; i < PF; ++i) rdkp(kf[i], i, par_tag);
          bf16x8 used = kf[0];  // fragment of the MFMA issued in the step before
          // arguments of the first pair of exponentials; every step forms those of the next one
          float t0 = __builtin_fmaf(Sc[0][0], c, negM), t1 = __builtin_fmaf(Sc[0][1], c, negM);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int stp = 0; stp < NS; ++stp) {
            const int b = stp >> 3;
            const int nb = (stp + 1) >> 3, ni = 2 * ((stp + 1) & 7);  // the next step's pair of scores
            const float s2 = stp + 1 < NS ? Sc[nb & 1][ni] : 0.f, s3 = stp + 1 < NS ? Sc[nb & 1][ni + 1] : 0.f;
            float u0 = 0.f, u1 = 0.f;
            unsigned pw;
            constexpr int kLast = NS - 1;
            const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;
            // (one statement per step: wait for the K fragment, MFMA, exponentials, next arguments, pack, row sum;
            // the last MFMA of a key block writes into the registers of the scores the block has used up)
#define PDLLM_QK_STEP(KIND, ACC, DST)                                                                                 \
  do {                                                                                                                \
    if (young == 2) qk_step<2, KIND>(ACC, DST, kf[stp % PF], QA[stp & 7], t0, t1, s2, s3, c, negM, u0, u1, pw, psum, used);      \
    else if (young == 1) qk_step<1, KIND>(ACC, DST, kf[stp % PF], QA[stp & 7], t0, t1, s2, s3, c, negM, u0, u1, pw, psum, used); \
    else qk_step<0, KIND>(ACC, DST, kf[stp % PF], QA[stp & 7], t0, t1, s2, s3, c, negM, u0, u1, pw, psum, used);                 \
  } while (0)
            if (stp == kLast) PDLLM_QK_STEP(3, Sn[b], Sc[b]);
            else if ((stp & 7) == 7) PDLLM_QK_STEP(2, Sn[b], Sc[b]);
            else if ((stp & 7) == 0) PDLLM_QK_STEP(0, Sn[b], Sn[b]);
            else PDLLM_QK_STEP(1, Sn[b], Sn[b]);
#undef PDLLM_QK_STEP
            used = kf[stp % PF];
            PW[b][(stp & 7) >> 2][stp & 3] = pw;
            t0 = u0;
            t1 = u1;
            if (stp + PF < NS) rdkp(kf[stp % PF], stp + PF, par_tag);
            if constexpr (!SPEC) {
              if ((stp & 1) == 1 && ((stp & 7) >> 1) < kDmaGroups) {
                if (stp < 8) issue_v1(t + 1, PAR ^ 1, (stp & 7) >> 1, steady_tag);
                else if (k_on) issue_k1(t + 2, PAR, (stp & 7) >> 1, steady_tag);
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          if constexpr (!SPEC) {
#pragma unroll
            for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
            if (MODE == 1) load_slots_ctx(t + 3);
            else if (MODE == 2) load_slots_new(t + 3);
            else if (t + 3 < T1) load_slots(t + 3);
          }
        } else {
#pragma unroll
          for (int stp = 0; stp < NS; ++stp) {
            const int b = stp >> 3, i = 2 * (stp & 7);
            const bf16x2 pr = {(__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(Sc[b][i], c, negM)),
                               (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(Sc[b][i + 1], c, negM))};
            psum = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, psum, false);
            PW[b][(stp & 7) >> 2][stp & 3] = __builtin_bit_cast(unsigned, pr);
          }
        }
        lA += psum;
        __builtin_amdgcn_sched_barrier(0);
        // ---- PV of tile t ----
        {
          // V^T fragments of step stp in staging operand stp & 1 (attn_common.h: pv_step); the offset of a
          // fragment inside the tile: key block kj = stp >> 2 (16 keys each), buffer by the parity tag
          constexpr int vbase = kTileBytes + (PARC == 1 ? kBufBytes : 0);
          bf16x8 stg0, stg1;
          float mnext = 0.f;
          pv_read<0, vbase>(stg0, va[0][0], va[1][0]);
          pv_read<1, vbase>(stg1, va[0][1], va[1][1]);
          __builtin_amdgcn_sched_barrier(0);
#define PDLLM_PV_STEP(STP)                                                                                             \
  do {                                                                                                                 \
    constexpr int stp = STP, db = stp & 3, kj = stp >> 2, nx = stp + 2;                                                 \
    constexpr int off = nx < NS ? vbase + (nx >> 2) * 16 * kRowBytes : -1;                                              \
    if constexpr ((stp & 1) == 0)                                                                                       \
      pv_step<0, (stp + 1 < NS ? 2 : 0), off>(OA[db], stg0, PW[kj >> 1][kj & 1], va[0][nx & 3], va[1][nx & 3], mnext);  \
    else                                                                                                                \
      pv_step<1, (stp + 1 < NS ? 2 : 0), off>(OA[db], stg1, PW[kj >> 1][kj & 1], va[0][nx & 3], va[1][nx & 3], mnext);  \
    /* unmasked row maximum of the scores of tile t + 1 (Sc holds them since the QK steps), one instruction      */  \
    /* between two steps; without a next tile the value is not used                                              */  \
    mnext = stp == 0 ? fmaxf(Sc[0][0], Sc[0][1])                                                                        \
                     : fmaxf(fmaxf(mnext, Sc[stp >> 3][2 * (stp & 7)]), Sc[stp >> 3][2 * (stp & 7) + 1]);               \
    __builtin_amdgcn_sched_barrier(0);                                                                                  \
  } while (0)
          PDLLM_PV_STEP(0); PDLLM_PV_STEP(1); PDLLM_PV_STEP(2); PDLLM_PV_STEP(3);
          PDLLM_PV_STEP(4); PDLLM_PV_STEP(5); PDLLM_PV_STEP(6); PDLLM_PV_STEP(7);
          PDLLM_PV_STEP(8); PDLLM_PV_STEP(9); PDLLM_PV_STEP(10); PDLLM_PV_STEP(11);
          PDLLM_PV_STEP(12); PDLLM_PV_STEP(13); PDLLM_PV_STEP(14); PDLLM_PV_STEP(15);
#undef PDLLM_PV_STEP
          mx_carry = half_swap_max(mnext) * c;
        }
        if constexpr (PARC < 0) {
          // the next tile reads the other buffers
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) ka[ks] -= flip;
#pragma unroll
          for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int db = 0; db < 4; ++db) va[r][db] += flip;
          flip = -flip;
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): K(t+2), V(t+1) and the slots have landed
        __syncthreads();
      };

      // ---- prologue: K(T0), V(T0); then K(T0+1) while QK(T0) runs unpipelined ----
      f32x16 SX[2];
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) SX[b][i] = 0.f;
      if constexpr (!SPEC) {
        load_slots(T0);
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
        issue_k(T0, 0);
        issue_v(T0, 0);
        if (T0 + 1 < T1) load_slots(T0 + 1);
      }
      build_mask(T0, 0);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if constexpr (!SPEC) {
        if (T0 + 1 < T1) issue_k(T0 + 1, 1);
#pragma unroll
        for (int i = 0; i < kDmaGroups; ++i) nsv[i] = nslot[i];
        if (T0 + 2 < T1) load_slots(T0 + 2);
      }
      {
        bf16x8 kf[PF];
#pragma unroll
        for (int i = 0; i < PF; ++i) rdk(kf[i], i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int stp = 0; stp < NS; ++stp) {
          wait_k(kf[stp % PF], stp);
          SX[stp >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], QA[stp & 7], SX[stp >> 3], 0, 0, 0);
          if (stp + PF < NS) rdk(kf[stp % PF], stp + PF);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      {
        float m0 = fmaxf(SX[0][0], SX[0][1]);
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = (b == 0 ? 2 : 0); i < 16; i += 2) m0 = fmaxf(fmaxf(m0, SX[b][i]), SX[b][i + 1]);
        mx_carry = half_swap_max(m0) * c;
      }
      // from here on ka reads K(t+1) in buffer 1 and va reads V(t) in buffer 0
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) ka[ks] += kBufBytes;
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      {
        using Generic = std::integral_constant<int, 0>;
        // The steady forms need a tile t that is whole and unmasked and a tile t + 1 inside the piece.  Their copies
        // (V(t+1), K(t+2)) and slots (t+3) are issued unconditionally: past the end of the piece they land in free
        // buffers and are never read, but they must come from the tensor the form assumes -- prefix tiles up to
        // t + 3 for the first form (table entries exist for whole_ctx tiles), clamped rows for the second.
        const int whole_ctx = ctx_total / kKT;  // tiles of the prefix without a ragged end
        const int ctx_end = T1 - 1 < whole_ctx - 3 ? T1 - 1 : whole_ctx - 3;
        // active tiles that are whole and visible to every row of this row group
        int open_tiles = Sa / kKT;
        if (p.mask_mode == PDLLM_MASK_CAUSAL) open_tiles = (tq_first + 1) / kKT < open_tiles ? (tq_first + 1) / kKT : open_tiles;
        if (p.mask_mode == PDLLM_MASK_DENSE) open_tiles = 0;
        const int new_end = T1 - 1 < Tc + open_tiles ? T1 - 1 : Tc + open_tiles;
        int t = T0;
        using AnyPar = std::integral_constant<int, -1>;
        using Even = std::integral_constant<int, 0>;
        using Odd = std::integral_constant<int, 1>;
        if constexpr (BUF) {  // (the wide-address form keeps the one general loop: it has no registers to spare)
          // Each steady form runs unrolled by two from an even iteration on (t - T0 even: ka on buffer 1, va on
          // buffer 0): the buffers are then immediate offsets from ka moved to buffer 0, nothing toggles and
          // the scores of the two tiles alternate between two register sets without moves.
          auto pairs = [&](int end, auto steady_tag) __attribute__((always_inline)) {
            if (((t - T0) & 1) && t < end) { iter(t, 1, SX, steady_tag, AnyPar{}); ++t; }
            if (t + 1 < end) {
#pragma unroll
              for (int ks = 0; ks < 8; ++ks) ka[ks] -= kBufBytes;
              for (; t + 1 < end; t += 2) {
                iter(t, 0, SX, steady_tag, Even{});
                iter(t + 1, 1, SX, steady_tag, Odd{});
              }
#pragma unroll
              for (int ks = 0; ks < 8; ++ks) ka[ks] += kBufBytes;
            }
            for (; t < end; ++t) iter(t, (t - T0) & 1, SX, steady_tag, AnyPar{});
          };
          pairs(ctx_end, std::integral_constant<int, 1>{});
          for (; t < T1 && t < Tc; ++t) iter(t, (t - T0) & 1, SX, Generic{}, AnyPar{});
          pairs(new_end, std::integral_constant<int, 2>{});
        }
        for (; t < T1; ++t) iter(t, (t - T0) & 1, SX, Generic{}, AnyPar{});
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
  } else
  if (T0 < T1) {
    load_slots(T0);
    issue_tile(T0, 0, std::false_type{});  // waits for the slots it uses
    if (T0 + 1 < T1) load_slots(T0 + 1);
    build_mask(T0, 0);
    finish_tile(T0, 0, std::false_type{});
    __syncthreads();
    const int whole_ctx = ctx_total / kKT;  // tiles of the prefix without a ragged end
    const int steady_end = (T1 < whole_ctx ? T1 : whole_ctx) - 2;
    int t = T0;
    for (; t < steady_end; ++t) step(t, std::true_type{});
    for (; t < T1; ++t) step(t, std::false_type{});
  }

  // ---- epilogue ----
  auto emit = [&](int ridx, int db, const f32x16& o, float mfin, float lfin) __attribute__((always_inline)) {
    if (ridx < 0) return;
    const int tq = ridx / G;
    const int g = ridx - tq * G;
    const float inv = lfin > 0.f ? 1.f / lfin : 0.f;
    if (whole) {
      __bf16* op = p.out + (long)(q0 + tq) * p.o_stride + (long)(kvh * G + g) * kD + 32 * db + 4 * he;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        uint2 w;
        w.x = pack_bf16x2(o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv);
        w.y = pack_bf16x2(o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv);
        *reinterpret_cast<uint2*>(op + 8 * i4) = w;
      }
    } else {
      const long R = ((long)(q0 + tq) * p.Hq + kvh * G + g) * p.max_pieces + piece;
      store_partial_block(p.ws_o + R * kD, p.ws_scale + R * 4, db, he, o, inv);
      if (db == 0 && he == 0) p.ws_lse[R] = lfin > 0.f ? mfin + __log2f(lfin) : -INFINITY;  // log2 domain
    }
  };

  // A block of output rows (the column's only piece): the rows go through an 8 KB strip of the (now free) tile
  // buffers, 64 columns at a time, so that 8 lanes store the 128 contiguous bytes of a row instead of 16-byte
  // pieces of 32 different rows (2 % on a causal prefill layer).  The strip holds [32 rows][16 float4], float4
  // column c of row r at c ^ (r & 15).  Partial rows keep the direct stores (the detour costs 1 % at 32 rows).
  auto emit_block = [&](int ridx, const f32x16 (&O)[4], float mfin, float lfin) __attribute__((always_inline)) {
    if (!whole) {
#pragma unroll
      for (int db = 0; db < 4; ++db) emit(ridx, db, O[db], mfin, lfin);
      return;
    }
    const float inv = lfin > 0.f ? 1.f / lfin : 0.f;
    unsigned long rowptr = 0;  // global address of this lane's row, 0 = no such row
    if (ridx >= 0) {
      const int tq = ridx / G;
      const int g = ridx - tq * G;
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
          const f32x16& o = O[2 * hf + dd];
          const int c4 = 8 * dd + 2 * i4 + he;
          const float4 w = {o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv, o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv};
          *reinterpret_cast<float4*>(strip + l32e * 64 + 4 * (c4 ^ (l32e & 15))) = w;
        }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int rr = 8 * k + (lane_e >> 3);
        const unsigned long dst = ((unsigned long)(unsigned)__shfl(ptr_hi, rr, 64) << 32) | (unsigned)__shfl(ptr_lo, rr, 64);
        const float4 a = *reinterpret_cast<const float4*>(strip + rr * 64 + 4 * ((2 * j) ^ (rr & 15)));
        const float4 b = *reinterpret_cast<const float4*>(strip + rr * 64 + 4 * ((2 * j + 1) ^ (rr & 15)));
        uint4 w;
        w.x = pack_bf16x2(a.x, a.y); w.y = pack_bf16x2(a.z, a.w);
        w.z = pack_bf16x2(b.x, b.y); w.w = pack_bf16x2(b.z, b.w);
        if (dst != 0) *reinterpret_cast<uint4*>(dst + 2 * (64 * hf + 8 * j)) = w;
      }
    }
  };

  if (HAS_A) {
    lA = half_swap_sum(lA);
    emit_block(ridxA, OA, MA, lA);
  }
  if (HAS_B) {
    lB = half_swap_sum(lB);
    if (GS == 1) {
      emit_block(ridxB, OB, MB, lB);
    } else {
      // merge the GS partial results of a shared block through LDS (the tile buffers are free now);
      // element (d, row) of a partial lives at [d][row ^ (d & 31)], conflict-free both ways
      float* part = reinterpret_cast<float*>(lds) + wave * (kPartBytes / 4);
      if (HAS_A) __syncthreads();  // the partial of this wave lies over the strips two other waves just used
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int d = 32 * db + 8 * (i >> 2) + 4 * he + (i & 3);
          part[d * 32 + (l32e ^ (d & 31))] = OB[db][i];
        }
      if (he == 0) {
        s_ml[wave][0][l32e] = MB;
        s_ml[wave][1][l32e] = lB;
      }
      __syncthreads();
      const int wbase = wave - gi;
      float M = -INFINITY;
#pragma unroll
      for (int w = 0; w < GS; ++w) M = fmaxf(M, s_ml[wbase + w][0][l32e]);
      const float Muse = (M == -INFINITY) ? 0.f : M;
      float wgt[GS];
      float L = 0.f;
#pragma unroll
      for (int w = 0; w < GS; ++w) {
        wgt[w] = __builtin_amdgcn_exp2f(s_ml[wbase + w][0][l32e] - Muse);
        L += wgt[w] * s_ml[wbase + w][1][l32e];
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
            const int d = 32 * db + 8 * (i >> 2) + 4 * he + (i & 3);
            acc[i] += wgt[w] * pw[d * 32 + (l32e ^ (d & 31))];
          }
        }
        emit(ridxB, db, acc, M, L);
      }
    }
  }
  if (head_rt >= 0 || y < y_end) {
    // the next piece reuses the LDS buffers: wait for this piece's LDS reads only -- the global stores of the
    // epilogue stay in flight behind the next prologue (a full barrier would wait for their acknowledgement)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  }
  }  // pieces
}

// Slot table: for request r and v < count(r), table[r][v] = page * page_size + offset of the v-th
// visible prefix key (ranges in order, each mapped through the page table); entries up to the
// next multiple of the tile size repeat a valid slot (they are loaded but masked);
// table[r][stride - 1] = count(r).
// A page-table entry outside [0, n_pages) names no page: its keys are left out, as the reference skips such
// entries (layers/attention/ops/kv_cache_kernels.py:208), and count(r) is the number of keys that remain, at most
// max_ctx_len of them.  (A request whose ranges touch more than kMaxSegments pages keeps the older behaviour:
// such entries are clamped into the cache.)
constexpr int kMaxSegments = 2048;  // (range, page) pieces of one request's visible prefix

__global__ __launch_bounds__(256) void attn_slot_table_kernel(const AttnKParams p, int* __restrict__ table) {
  __shared__ int s_cum[kMaxRanges + 1];      // visible keys before range i, invalid pages included
  __shared__ int s_start[kMaxRanges];
  __shared__ int s_len[kMaxRanges];
  __shared__ int s_seg0[kMaxRanges + 1];     // pieces before range i
  __shared__ int s_gone[kMaxSegments];       // keys left out before piece s (exclusive prefix of the invalid pieces' lengths)
  __shared__ int s_wave[4];
  __shared__ int s_total_gone;
  const int tid = threadIdx.x;
  const int req = blockIdx.y;
  const int r0 = p.range_ptr[req];
  int nr = p.range_ptr[req + 1] - r0;
  nr = nr < 0 ? 0 : (nr > kMaxRanges ? kMaxRanges : nr);
  if (tid < nr) {
    const int len = p.range_len[r0 + tid];
    s_len[tid] = len > 0 ? len : 0;
    s_start[tid] = p.range_start[r0 + tid];
  }
  __syncthreads();
  if (tid == 0) {
    int cc = 0, ss = 0;
    for (int i = 0; i < nr; ++i) {
      s_cum[i] = cc;
      s_seg0[i] = ss;
      cc += s_len[i];
      if (s_len[i] > 0) ss += ((s_start[i] + s_len[i] - 1) >> p.page_shift) - (s_start[i] >> p.page_shift) + 1;
    }
    s_cum[nr] = cc;
    s_seg0[nr] = ss;
    s_total_gone = 0;
  }
  __syncthreads();
  const int all = s_cum[nr] < p.max_ctx_len ? s_cum[nr] : p.max_ctx_len;  // keys of the ranges, capped
  const int n_seg = s_seg0[nr];
  const bool compact = n_seg <= kMaxSegments;
  const int page_mask = (1 << p.page_shift) - 1;
  auto page_of = [&](int tok) {
    int pi = tok >> p.page_shift;
    pi = pi < 0 ? 0 : (pi >= p.bt_stride ? p.bt_stride - 1 : pi);
    return p.block_table[(long)req * p.bt_stride + pi];
  };
  // ---- which pieces name no page, and how many keys are left out before each piece ----
  bool any_gone = false;
  if (compact) {
    bool mine_gone = false;
    for (int sg = tid; sg < n_seg; sg += 256) {
      int rp = 0;
      while (rp + 1 < nr && sg >= s_seg0[rp + 1]) ++rp;
      const int pg = (s_start[rp] >> p.page_shift) + (sg - s_seg0[rp]);
      const int t0 = pg << p.page_shift, t1 = t0 + page_mask + 1;
      const int a = t0 > s_start[rp] ? t0 : s_start[rp];
      const int b = t1 < s_start[rp] + s_len[rp] ? t1 : s_start[rp] + s_len[rp];
      int v0 = s_cum[rp] + (a - s_start[rp]), v1 = s_cum[rp] + (b - s_start[rp]);
      v0 = v0 < all ? v0 : all;
      v1 = v1 < all ? v1 : all;
      const int page = page_of(a);
      const int gone = (v1 > v0 && (page < 0 || page >= p.n_pages)) ? v1 - v0 : 0;
      s_gone[sg] = gone;
      mine_gone |= gone != 0;
    }
    any_gone = __syncthreads_or(mine_gone);
    if (any_gone) {
      // exclusive prefix over the pieces, in place: a thread owns `per` consecutive pieces
      const int per = (n_seg + 255) / 256;
      const int s0 = tid * per < n_seg ? tid * per : n_seg;
      const int s1 = s0 + per < n_seg ? s0 + per : n_seg;
      int sum = 0;
      for (int sg = s0; sg < s1; ++sg) sum += s_gone[sg];
      int incl = sum;
      const int lane = tid & 63, wv = tid >> 6;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int x = __shfl_up(incl, o, 64);
        if (lane >= o) incl += x;
      }
      if (lane == 63) s_wave[wv] = incl;
      __syncthreads();
      int before = incl - sum;
      for (int w = 0; w < wv; ++w) before += s_wave[w];
      for (int sg = s0; sg < s1; ++sg) {
        const int g = s_gone[sg];
        s_gone[sg] = before;
        before += g;
      }
      if (tid == 255) s_total_gone = before;
      __syncthreads();
    }
  }
  const int count = all - (any_gone ? s_total_gone : 0);
  int* row = table + (long)req * p.slot_stride;
  if (blockIdx.x == 0 && tid == 0) row[p.slot_stride - 1] = count;
  const int padded = (count + kKT - 1) / kKT * kKT;
  const int v = blockIdx.x * 256 + tid;   // a key of the ranges (before anything is left out)
  if (v >= all) return;
  int rp = 0;
  while (rp + 1 < nr && v >= s_cum[rp + 1]) ++rp;
  const int tok = s_start[rp] + (v - s_cum[rp]);
  int page = page_of(tok);
  int at = v;
  if (any_gone) {
    if (page < 0 || page >= p.n_pages) return;     // left out
    const int sg = s_seg0[rp] + (tok >> p.page_shift) - (s_start[rp] >> p.page_shift);
    at = v - s_gone[sg];
  } else {
    page = page < 0 ? 0 : (page >= p.n_pages ? p.n_pages - 1 : page);
  }
  const int slot = (page << p.page_shift) + (tok & page_mask);
  row[at] = slot;
  if (at == count - 1)
    for (int o = count; o < padded; ++o) row[o] = slot;   // the ragged end of the last tile: a valid slot, masked
}

// Reduce the partial results of the columns that were cut into several pieces: one wave per
// (token, q-head) row.  Rows of a column with a single piece were written directly.
struct MergeParams {
  const uint16_t* ws_o;  // fp16 partial rows, see store_partial_block
  const float* ws_lse;
  const float* ws_scale;
  __bf16* out;
  const int* q_start_loc;
  long o_stride, n_tokens;
  int n_req, max_q_len, Hq, Hkv, rows_per_group, row_tiles, t_lin, span, max_pieces, reversed, head;
  // paged store of the active rows (bf16, unified layout) by the first store_blocks workgroups of the launch (they
  // start first and their round trip to memory overlaps the merge); store_blocks == 0: no store
  int store_blocks;
  const int* store_slots;
  const uint4* k_new;
  const uint4* v_new;
  uint4* k_cache;
  uint4* v_cache;
  long kn_stride16, vn_stride16, n_slots;  // strides in 16-byte units
};

__global__ __launch_bounds__(256) void attn_merge_kernel(const MergeParams m) {
  if ((int)blockIdx.x < m.store_blocks) {
    // store_kvcache of the active rows: one 16-byte chunk of a K row and of a V row per thread
    const int cpr = m.Hkv * (kD / 8);  // chunks per token row
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    const long tok = idx / cpr;
    const int ch = (int)(idx - tok * cpr);
    if (tok >= m.n_tokens) return;
    const long slot = m.store_slots[tok];
    if (slot < 0 || slot >= m.n_slots) return;
    const uint4 kv = m.k_new[tok * m.kn_stride16 + ch];
    const uint4 vv = m.v_new[tok * m.vn_stride16 + ch];
    m.k_cache[slot * cpr + ch] = kv;
    m.v_cache[slot * cpr + ch] = vv;
    return;
  }
  // 16 lanes per row (8 columns = 16 bytes of a partial row each), 16 rows per workgroup
  const int l = threadIdx.x & 15;
  const long row = (long)((int)blockIdx.x - m.store_blocks) * 16 + (threadIdx.x >> 4);
  const long per_req = (long)m.max_q_len * m.Hq;
  if (row >= per_req * m.n_req) return;
  const int req = (int)(row / per_req);
  const int rem = (int)(row - (long)req * per_req);
  const int tq = rem / m.Hq;
  const int head = rem - tq * m.Hq;
  const int q0 = m.q_start_loc[req];
  const int Sq = m.q_start_loc[req + 1] - q0;
  if (q0 < 0 || tq >= Sq || (long)q0 + Sq > m.n_tokens || Sq > m.max_q_len) return;
  const int G = m.Hq / m.Hkv;
  const int kvh = head / G;
  const int rt = (tq * G + (head - kvh * G)) / m.rows_per_group;
  const int col = (req * m.Hkv + kvh) * m.row_tiles + (m.reversed ? m.row_tiles - 1 - rt : rt);
  const int tail_len = m.t_lin - m.head;
  const int tail_at = (m.head > 0 ? col % m.row_tiles : col) * tail_len;  // on the line the column's tail lies on
  const int np = (m.head > 0 ? 1 : 0) + (tail_at + tail_len - 1) / m.span - tail_at / m.span + 1;
  if (np == 1) return;
  const long R = ((long)(q0 + tq) * m.Hq + head) * m.max_pieces;
  // Four pieces at a time: their log-sum-exps and partial rows are fetched together (one round trip), then
  // folded into the running maximum.  A piece without keys has lse = -inf and weight 0; what its row holds is
  // never used.
  float M = -INFINITY, L = 0.f;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < np; s0 += 4) {
    float lse[4], sc[4];
    uint4 o[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool on = s0 + u < np;
      lse[u] = on ? m.ws_lse[R + s0 + u] : -INFINITY;
      sc[u] = on ? m.ws_scale[(R + s0 + u) * 4 + (l >> 2)] : 0.f;
      o[u] = on ? *reinterpret_cast<const uint4*>(m.ws_o + (R + s0 + u) * kD + 8 * l) : uint4{0u, 0u, 0u, 0u};
    }
    const float Mn = fmaxf(fmaxf(M, fmaxf(lse[0], lse[1])), fmaxf(lse[2], lse[3]));
    if (Mn == -INFINITY) continue;
    const float r = M == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(M - Mn);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= r;
    L *= r;
    M = Mn;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float w = lse[u] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(lse[u] - M);
      if (w > 0.f) {
        const unsigned words[4] = {o[u].x, o[u].y, o[u].z, o[u].w};
        const float ws = w * sc[u];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const f16x2 h2 = __builtin_bit_cast(f16x2, words[e]);
          acc[2 * e] += ws * (float)h2[0];
          acc[2 * e + 1] += ws * (float)h2[1];
        }
        L += w;
      }
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  uint4 packed;
  packed.x = pack_bf16x2(acc[0] * inv, acc[1] * inv);
  packed.y = pack_bf16x2(acc[2] * inv, acc[3] * inv);
  packed.z = pack_bf16x2(acc[4] * inv, acc[5] * inv);
  packed.w = pack_bf16x2(acc[6] * inv, acc[7] * inv);
  *reinterpret_cast<uint4*>(m.out + (long)(q0 + tq) * m.o_stride + (long)head * kD + 8 * l) = packed;
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct AttnPlan {
  int J;
  int row_tiles;
  int t_lin;       // positions per column on the tile line
  int span;        // tiles per workgroup
  int n_lin;       // columns * t_lin
  int max_pieces;  // most pieces a column is cut into
  int grid;        // workgroups
  int head;        // tiles of a column taken by a workgroup of its own at the start of its set (0: one line over all columns)
  int wg_set;      // workgroups per set when head > 0
};

static int ilog2_exact(int v) {
  if (v <= 0 || (v & (v - 1))) return -1;
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

// ints per request of the slot table: the keys padded to whole tiles, one spare tile, the count
static int64_t slot_table_stride_for(const pdllm_attn_desc* d) {
  return ((int64_t)d->max_ctx_len + kKT - 1) / kKT * kKT + kKT;
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
  if (!prefill && d->active_slot_mapping != nullptr) {
    // the store writes whole token rows of a contiguous unified cache
    if (!d->k_cache || !d->v_cache) return PDLLM_ERR_NULL;
    if (d->kv_dtype != PDLLM_KV_BF16 && d->kv_dtype != PDLLM_KV_FP8_E4M3) return PDLLM_ERR_DTYPE;
    if (d->kv_dtype == PDLLM_KV_FP8_E4M3 && (!d->k_scale || !d->v_scale)) return PDLLM_ERR_NULL;
    if (ilog2_exact(d->page_size) < 0 || d->n_pages <= 0) return PDLLM_ERR_SHAPE;
    if (d->cache_head_stride != kD || d->cache_token_stride != hk ||
        d->cache_page_stride != hk * d->page_size)
      return PDLLM_ERR_STRIDE;
    // the store kernels write 16 bytes per lane (8 per lane of fp8 bytes), with or without a visible prefix
    const uintptr_t salign = d->kv_dtype == PDLLM_KV_FP8_E4M3 ? 8 : 16;
    if (((uintptr_t)d->k_cache | (uintptr_t)d->v_cache) % salign) return PDLLM_ERR_STRIDE;
    if ((uintptr_t)d->active_slot_mapping % 4) return PDLLM_ERR_STRIDE;
  }
  if (has_cache && d->slot_table != nullptr) {
    if (d->slot_table_stride < slot_table_stride_for(d) || ((uintptr_t)d->slot_table % 4)) return PDLLM_ERR_STRIDE;
  }
  if (!(d->sm_scale > 0.f) || !(d->sm_scale < 1e30f)) return PDLLM_ERR_SHAPE;  // the row maximum is taken before scaling
  if (d->num_splits < 0 || d->num_splits > 16 || d->tiles_per_workgroup < 0) return PDLLM_ERR_SHAPE;
  if (d->rows_per_group != 0) {
    const int j = d->rows_per_group / 32;
    if (d->rows_per_group % 32 || !(j == 1 || j == 2 || j == 4 || j == 5 || j == 6 || j == 8)) return PDLLM_ERR_SHAPE;
  }
  return PDLLM_OK;
}

// Bytes of dynamic LDS of attn_fwd_kernel<*, J>: Q fragments of the shared blocks next to a
// slot A, then the bit rows of a dense mask.
static int dyn_lds_bytes(int J, int mask_mode) {
  int b = (J == 5 || J == 6) ? (J - 4) * 8192 : 0;
  if (mask_mode == PDLLM_MASK_DENSE) b += 2 * kMaxTok * kNKB * 4;
  return b;
}

// Pick the row-group size J and the span (tiles per workgroup) by a small cost model.
// All tiles of all columns (request, KV head, row group) lie on one line of n_cols * t_lin
// positions; workgroup g takes positions [g * span, (g + 1) * span).  span = t_lin gives one
// workgroup per column; a smaller span that does not divide t_lin lets pieces of two columns
// share a workgroup, which balances any shape over the CUs at the price of partial rows in the workspace.
// Unit of time: one wave doing one 32-row block of one 64-key tile on a CU of its own.  A
// workgroup alone on a CU spends (fixed + blocks per wave) per tile; two workgroups sharing a CU
// (at most 4 row blocks, LDS footprint <= 80 KB) overlap matrix and vector work and take kPair of the
// serial time.  The most loaded CU sets the makespan.
// Compute units of the current device (the planner balances over them); 256, an MI355X, when no device can be
// asked -- sizes and plans can be queried on a machine without a GPU.
static int compute_units() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

#ifndef PDLLM_FP8_PRODUCERS
#define PDLLM_FP8_PRODUCERS 1
#endif
// 32-bit copy offsets: a tensor the copies read is smaller than 4 GiB and its rows and row indices fit the 24-bit
// multiply
static bool small_tensor(int64_t rows, int64_t row_bytes) {
  return rows < (1l << 24) && row_bytes < (1l << 24) && rows * row_bytes < (1l << 32) - 4096;
}

// fp8 pages, five row blocks: the kernel with producer waves addresses caches and scales with 32-bit offsets
static bool fp8_producers_fit(const pdllm_attn_desc* d) {
  return small_tensor(d->n_pages * (int64_t)d->page_size, d->cache_token_stride) &&
         small_tensor(d->n_pages, d->scale_page_stride * 4);
}

static AttnPlan compute_plan(const pdllm_attn_desc* d, bool prefill) {
  const int G = d->num_q_heads / d->num_kv_heads;
  const long rows = (long)d->max_q_len * G;
  const long nblk = (rows + 31) / 32;
  const long ctx = prefill ? 0 : d->max_ctx_len;
  const long T = (ctx + kKT - 1) / kKT + (d->max_q_len + kKT - 1) / kKT;
  const long units = (long)d->n_req * d->num_kv_heads;
  const bool fp8 = !prefill && d->k_cache != nullptr && d->max_ctx_len > 0 && d->kv_dtype == PDLLM_KV_FP8_E4M3;
  const bool producers = fp8 && PDLLM_FP8_PRODUCERS && fp8_producers_fit(d);
  const int cus = compute_units();
  // kPiece: what a piece costs outside its tile loop (three round trips to memory before the first MFMA, the
  // last PV, the partial rows): about 3.2 tiles of a 4-wave workgroup
  constexpr double kFixed = 0.35, kPair = 0.65, kPiece = 4.3, kWide = 1.45;
  constexpr int kStaticLds = 66 * 1024;
  static const int js[] = {1, 2, 4, 5, 6, 8};
  static const double upw[] = {0.45, 0.75, 1.0, 1.25, 1.5, 1.0};
  AttnPlan best = {4, 1, (int)T, (int)T, (int)T, 1, 1, 0, 0};
  double best_cost = 1e300;
  for (int ji = 0; ji < 6; ++ji) {
    const int J = js[ji];
    if (d->rows_per_group && d->rows_per_group != 32 * J) continue;
    // 5 and 6 row blocks need more than 256 registers (one workgroup per CU): on request, and for an fp8
    // cache (which has no 8-block kernel) when they hold all rows of a (request, KV head) in one column
    // where 4 blocks would leave a second, mostly empty one (160 rows of an MHA layer: 250-265 us against 362).
    // Five blocks with producer waves are a candidate for any fp8 shape of five blocks or more: per row block
    // and tile they take 0.92 of what a pair of 4-block workgroups takes (8 x 1120 rows over 4096 keys, GQA 28/4:
    // 116 against 122 us; 4 x 640 rows over 16400 keys, GQA 32/8: 227 against 237 us).
    // -- where groups of five do not leave more empty row blocks than groups of four (7 blocks of a 32-row decode
    // with GQA 28/4 are 5 + 2 against 4 + 3: 43.6 against 40.0 us).
    const bool fives_fill = (nblk + 4) / 5 * 5 <= (nblk + 3) / 4 * 4;
    if (!d->rows_per_group && (J == 5 || J == 6) &&
        !(fp8 && nblk > 4 && (nblk <= J || (J == 5 && producers && fives_fill))))
      continue;
    const double units_per_wave = (J == 5 && producers) ? 0.66 : upw[ji];
    if (J == 8 && fp8) continue;  // the 8-wave workgroup has no room for the fp8 staging registers
    if (J == 8 && prefill && !d->rows_per_group) continue;  // coarser causal staircase: measured slower
    const long row_tiles = (nblk + J - 1) / J;
    const long cols = units * row_tiles;
    const bool two = (!fp8 || J <= 4) && J != 8 && kStaticLds + dyn_lds_bytes(J, d->mask_mode) <= 80 * 1024;
    const long slots = (long)cus * (two ? 2 : 1);
    // candidate spans: whole columns, columns cut into 2..16 equal parts, and the balanced cut
    for (int cand = 0; cand <= 20; ++cand) {
      long t_lin = T, span, head = 0, wg_set = 0;
      double set_load = 0.0;
      if (cand == 0) {
        span = T;
      } else if (cand <= 15) {
        const int S = cand + 1;
        if (S > T) break;
        span = (T + S - 1) / S;
        t_lin = span * S;  // aligned: pieces never cross a column
      } else if (cand == 16) {
        if (prefill) continue;
        span = (cols * T + slots - 1) / slots;
        if (span >= T || span < 2) continue;
      } else if (cand == 17) {
        if (prefill) continue;
        span = (cols * T + 2 * slots - 1) / (2 * slots);
        if (span >= T || span < 4) continue;
      } else if (cand == 18) {
        if (d->tiles_per_workgroup <= 0) continue;
        span = d->tiles_per_workgroup < T ? d->tiles_per_workgroup : T;
      } else {
        // the balanced cut, set by set: k workgroups per (request, KV head), the first row_tiles of
        // them side by side over the same leading tiles of their columns
        if (prefill || row_tiles < 2) continue;
        const long k = (cand == 19 ? slots : 2 * slots) / units;
        if (k <= row_tiles) continue;
        // A head workgroup handles one piece of `head` tiles; the others cut the rest of the set's columns into
        // spans and handle two or three pieces each.  The head is made `extra` tiles longer than a span; which
        // `extra` gives the shortest longest workgroup depends on where the cuts fall in the columns (a cut that
        // coincides with the end of a column saves a piece), so the candidates are laid out and compared.
        const double tile_cost = kFixed + units_per_wave, piece_cost = kPiece;
        double best_load = 1e300;
        long best_span = 0, best_head = 0;
        for (long extra = 0; extra <= 12; ++extra) {
          const long sp = (row_tiles * (T - extra) + k - 1) / k;
          const long hd = sp + extra;
          if (hd >= T || sp < 4) continue;
          const long tail_len = T - hd, tail_total = row_tiles * tail_len;
          double load = (double)hd * tile_cost + piece_cost;
          for (long a = 0; a < tail_total; a += sp) {
            const long b = a + sp < tail_total ? a + sp : tail_total;
            const long n_pieces = (b - 1) / tail_len - a / tail_len + 1;
            const double l = (double)(b - a) * tile_cost + piece_cost * (double)n_pieces;
            load = l > load ? l : load;
          }
          if (load < best_load) { best_load = load; best_span = sp; best_head = hd; }
        }
        if (best_span == 0) continue;
        span = best_span;
        head = best_head;
        wg_set = k;
        set_load = best_load;
      }
      if (d->tiles_per_workgroup > 0) {
        if (cand != 18) continue;
      } else if (d->num_splits) {
        if (cand == 0 ? d->num_splits != 1 : (cand > 15 || d->num_splits != cand + 1)) continue;
      } else if (prefill && cand != 0) {
        continue;
      }
      const long n_lin = head > 0 ? row_tiles * (t_lin - head) : cols * t_lin;
      if (n_lin >= (1l << 30)) continue;
      const long grid = head > 0 ? units * wg_set : (n_lin + span - 1) / span;
      const long n = (grid + cus - 1) / cus;  // workgroups on the most loaded CU
      // an 8-wave workgroup behaves like a co-resident pair that shares its tiles
      const double serial = J == 8 ? (double)n * kWide : two ? (double)(n / 2) * 2.0 * kPair + (double)(n % 2) : (double)n;
      const bool cut = span < t_lin;
      long pieces = cut ? (t_lin + span - 1) / span + (t_lin % span ? 1 : 0) : 1;
      if (head > 0) {
        pieces = 0;
        for (long r = 0; r < row_tiles; ++r) {
          const long a = r * (t_lin - head);
          const long np = 1 + (a + t_lin - head - 1) / span - a / span + 1;
          pieces = np > pieces ? np : pieces;
        }
      }
      // the most loaded workgroup: its tiles and its pieces (two where the cuts do not respect the columns)
      const double wg_load = head > 0 ? set_load
                                      : (double)span * (kFixed + units_per_wave) + kPiece * (cut && t_lin % span ? 2.0 : 1.0);
      double cost = serial * wg_load + 1.0;
      if (cut) {
        // partial rows written and read back (~4 MB per unit of time), plus the merge launch
        const double avg_pieces = (double)t_lin / (double)span + (t_lin % span ? 1.0 : 0.0);
        const double part_bytes = (double)units * rows * avg_pieces * (kD * 2 + 4 + 16) * 2.0;
        cost += part_bytes / 4.0e6 + 4.0 + 0.3 * avg_pieces;  // (the merge folds a row's pieces one after the other)
      }
      if (head > 0) cost *= 0.97;  // the set's workgroups share their tiles in L2: less traffic for the same cut
      if (cost < best_cost) {
        best_cost = cost;
        best.J = J;
        best.row_tiles = (int)row_tiles;
        best.t_lin = (int)t_lin;
        best.span = (int)span;
        best.n_lin = (int)n_lin;
        best.max_pieces = (int)pieces;
        best.grid = (int)grid;
        best.head = (int)head;
        best.wg_set = (int)wg_set;
      }
    }
  }
  if (best_cost == 1e300) {
    // the forced values fit no candidate (e.g. a split of a prefill): one workgroup per column, J = 4
    const long row_tiles = (nblk + 3) / 4;
    best = {4, (int)row_tiles, (int)T, (int)T, (int)(units * row_tiles * T), 1, (int)(units * row_tiles), 0, 0};
  }
  return best;
}

// The plan depends on a handful of descriptor fields; every launch asks for it, and laying out the candidates costs
// several microseconds of host time -- as much as a small launch runs on the GPU.  Each host thread remembers the last
// few plans it computed.
static AttnPlan make_plan(const pdllm_attn_desc* d, bool prefill) {
  struct Key {
    int64_t n_req;
    int32_t hq, hkv, q_len, ctx, kv_dtype, mask_mode, rows, splits, tiles, cus;
    bool prefill, has_cache;
    bool operator==(const Key& o) const {
      return n_req == o.n_req && hq == o.hq && hkv == o.hkv && q_len == o.q_len && ctx == o.ctx && kv_dtype == o.kv_dtype &&
             mask_mode == o.mask_mode && rows == o.rows && splits == o.splits && tiles == o.tiles && cus == o.cus &&
             prefill == o.prefill && has_cache == o.has_cache;
    }
  };
  struct Entry { Key key; AttnPlan plan; bool used; };
  static thread_local Entry cache[8] = {};
  static thread_local int next = 0;
  const Key key = {d->n_req, d->num_q_heads, d->num_kv_heads, d->max_q_len, d->max_ctx_len, d->kv_dtype, d->mask_mode,
                   d->rows_per_group, d->num_splits, d->tiles_per_workgroup, compute_units(), prefill, d->k_cache != nullptr};
  for (const Entry& e : cache)
    if (e.used && e.key == key) return e.plan;
  Entry& e = cache[next];
  next = (next + 1) & 7;
  e.key = key;
  e.plan = compute_plan(d, prefill);
  e.used = true;
  return e.plan;
}

static bool needs_own_table(const pdllm_attn_desc* d, bool prefill) {
  return !prefill && d->k_cache != nullptr && d->max_ctx_len > 0 && d->slot_table == nullptr;
}

// split-KV partials first, then (when the caller passed no slot table) the table
static int64_t partial_bytes_for(const pdllm_attn_desc* d, int max_pieces) {
  if (max_pieces <= 1) return 0;
  const int64_t rows = d->n_tokens * d->num_q_heads;
  return rows * max_pieces * (int64_t)(kD * 2 + 4 + 16);  // fp16 row, log-sum-exp, four scales
}
static int64_t ws_bytes_for(const pdllm_attn_desc* d, int max_pieces, bool prefill) {
  int64_t b = partial_bytes_for(d, max_pieces);
  if (needs_own_table(d, prefill)) b += (int64_t)d->n_req * slot_table_stride_for(d) * 4;
  return b;
}

static void fill_table_params(const pdllm_attn_desc* d, AttnKParams& p) {
  p.block_table = d->block_table;
  p.range_ptr = d->range_ptr;
  p.range_start = d->range_start;
  p.range_len = d->range_len;
  p.bt_stride = d->bt_stride;
  p.n_pages = (int)d->n_pages;
  p.page_shift = ilog2_exact(d->page_size);
  p.max_ctx_len = d->max_ctx_len;
  p.max_ranges = d->max_ranges;
}

static int launch_slot_table(const AttnKParams& p, int n_req, int* table, hipStream_t stream) {
  const int padded = (p.max_ctx_len + kKT - 1) / kKT * kKT;
  const dim3 grid((unsigned)((padded + 255) / 256), (unsigned)n_req);
  hipLaunchKernelGGL(attn_slot_table_kernel, grid, dim3(256), 0, stream, p, table);
  return launch_status();
}

static int launch_attn(const pdllm_attn_desc* d, bool prefill, hipStream_t stream) {
  int st = validate_desc(d, prefill);
  if (st != PDLLM_OK) return st;
  if (prefill) {
    int grid = 0, team = 0;
    if (prefill_stream_plan(d, compute_units(), &grid, &team)) return launch_prefill_stream(d, grid, team, stream);
  }
  const AttnPlan plan = make_plan(d, prefill);
  const int64_t need = ws_bytes_for(d, plan.max_pieces, prefill);
  if (need > 0 && (!d->workspace || d->workspace_bytes < need)) return PDLLM_ERR_WORKSPACE;
  if (need > 0 && ((uintptr_t)d->workspace % 16)) return PDLLM_ERR_STRIDE;

  AttnKParams p = {};
  p.q = static_cast<const __bf16*>(d->q);
  p.k_new = static_cast<const __bf16*>(d->k_new);
  p.v_new = static_cast<const __bf16*>(d->v_new);
  p.out = static_cast<__bf16*>(d->out);
  const bool has_cache = !prefill && d->k_cache != nullptr && d->max_ctx_len > 0;
  p.k_cache = has_cache ? d->k_cache : nullptr;
  p.v_cache = has_cache ? d->v_cache : nullptr;
  p.k_scale = d->k_scale;
  p.v_scale = d->v_scale;
  p.q_start_loc = d->q_start_loc;
  p.mask = d->mask_mode == PDLLM_MASK_DENSE ? d->mask : nullptr;
  const int64_t rows = d->n_tokens * d->num_q_heads;
  p.ws_o = plan.max_pieces > 1 ? static_cast<uint16_t*>(d->workspace) : nullptr;
  p.ws_lse = p.ws_o ? reinterpret_cast<float*>(p.ws_o + rows * plan.max_pieces * kD) : nullptr;
  p.ws_scale = p.ws_o ? p.ws_lse + rows * plan.max_pieces : nullptr;
  if (has_cache) {
    fill_table_params(d, p);
    p.slot_stride = d->slot_table ? d->slot_table_stride : slot_table_stride_for(d);
    if (d->slot_table) {
      p.slot_table = d->slot_table;
    } else {
      int* table = reinterpret_cast<int*>(static_cast<char*>(d->workspace) + partial_bytes_for(d, plan.max_pieces));
      st = launch_slot_table(p, d->n_req, table, stream);
      if (st != PDLLM_OK) return st;
      p.slot_table = table;
    }
  }
  p.q_stride = d->q_stride; p.kn_stride = d->kn_stride; p.vn_stride = d->vn_stride; p.o_stride = d->o_stride;
  p.cache_page_stride = d->cache_page_stride;
  p.cache_token_stride = d->cache_token_stride;
  p.cache_head_stride = d->cache_head_stride;
  p.mask_stride = d->mask_stride;
  p.n_tokens = d->n_tokens;
  p.scale_page_stride = d->scale_page_stride;
  p.scale_head_stride = d->scale_head_stride;
  p.n_req = d->n_req; p.Hq = d->num_q_heads; p.Hkv = d->num_kv_heads; p.G = d->num_q_heads / d->num_kv_heads;
  p.mask_mode = d->mask_mode;
  p.J = plan.J;
  p.row_tiles = plan.row_tiles;
  p.t_lin = plan.t_lin;
  p.span = plan.span;
  p.n_lin = plan.n_lin;
  p.max_pieces = plan.max_pieces;
  p.head = plan.head;
  p.wg_set = plan.wg_set;
  p.max_q_len = d->max_q_len;
  p.scale_log2 = d->sm_scale * 1.4426950408889634f;

  if (plan.grid <= 0) return PDLLM_ERR_SHAPE;

  const bool fp8 = has_cache && d->kv_dtype == PDLLM_KV_FP8_E4M3;
  const int dyn = dyn_lds_bytes(plan.J, d->mask_mode);
  const dim3 grid((unsigned)plan.grid), block(plan.J == 8 && fp8 ? 512 : kThreads);
  const auto small = small_tensor;
  const bool buf = !fp8 && (plan.J == 4 || plan.J == 8) && small(d->n_tokens, d->kn_stride * 2) &&
                   small(d->n_tokens, d->vn_stride * 2) &&
                   (!has_cache || small(d->n_pages * (int64_t)d->page_size, d->cache_token_stride * 2));
#define PDLLM_LAUNCH(JJ)                                                                              \
  do {                                                                                                \
    if (fp8) hipLaunchKernelGGL((attn_fwd_kernel<1, JJ>), grid, block, dyn, stream, p);               \
    else hipLaunchKernelGGL((attn_fwd_kernel<0, JJ>), grid, block, dyn, stream, p);                   \
  } while (0)
  switch (plan.J) {
    case 1: PDLLM_LAUNCH(1); break;
    case 2: PDLLM_LAUNCH(2); break;
    case 4:
      if (buf) hipLaunchKernelGGL((attn_fwd_kernel<0, 4, true>), grid, block, dyn, stream, p);
      else PDLLM_LAUNCH(4);
      break;
    case 5:
      if (fp8 && PDLLM_FP8_PRODUCERS && fp8_producers_fit(d))  // (no Q fragments in LDS: only the mask rows are dynamic)
        hipLaunchKernelGGL((attn_fwd_kernel<1, 5, false, true>), grid, dim3(64 * 8), dyn_lds_bytes(4, d->mask_mode), stream, p);
      else PDLLM_LAUNCH(5);
      break;
    case 6: PDLLM_LAUNCH(6); break;
    case 8:
      if (fp8) PDLLM_LAUNCH(8);
      else if (launch_attn_fwd2(p, plan.grid, dyn, buf, stream) != PDLLM_OK) return PDLLM_ERR_LAUNCH;
      break;
    default: return PDLLM_ERR_SHAPE;
  }
#undef PDLLM_LAUNCH
  st = launch_status();
  if (st != PDLLM_OK) return st;
  // Paged store of the active rows (the reference stores them in front of the attention, attention_v4.py:328-331;
  // the slots lie behind the visible prefix, so the order within the call does not matter).  With a merge launch
  // the copy rides in that launch -- a kernel of its own between two attention launches costs more than the
  // copy -- otherwise, and for fp8 pages, it is the store kernel.
  const bool store = !prefill && d->active_slot_mapping != nullptr;
  const bool store_in_merge = store && plan.max_pieces > 1 && d->kv_dtype == PDLLM_KV_BF16;
  if (store && !store_in_merge) {
    const int64_t row = (int64_t)d->num_kv_heads * d->head_dim;
    const int64_t n_slots = d->n_pages * (int64_t)d->page_size;
    if (d->kv_dtype == PDLLM_KV_BF16)
      st = kv_store_launch(d->k_new, d->v_new, const_cast<void*>(d->k_cache), const_cast<void*>(d->v_cache),
                           d->active_slot_mapping, d->n_tokens, row, d->kn_stride, d->vn_stride, n_slots, stream);
    else
      st = pdllm_kv_store_fp8(d->k_new, d->v_new, const_cast<void*>(d->k_cache), const_cast<void*>(d->v_cache),
                              d->k_scale, d->v_scale, d->active_slot_mapping, d->n_tokens, row, d->kn_stride,
                              d->vn_stride, n_slots, d->page_size, d->head_dim, d->scale_page_stride,
                              d->scale_head_stride, stream);
    if (st != PDLLM_OK) return st;
  }
  if (plan.max_pieces > 1) {
    MergeParams m = {};
    m.ws_o = p.ws_o; m.ws_lse = p.ws_lse; m.ws_scale = p.ws_scale; m.out = p.out; m.q_start_loc = p.q_start_loc;
    m.o_stride = p.o_stride; m.n_tokens = p.n_tokens;
    m.n_req = p.n_req; m.max_q_len = p.max_q_len; m.Hq = p.Hq; m.Hkv = p.Hkv;
    m.rows_per_group = 32 * plan.J; m.row_tiles = plan.row_tiles; m.reversed = p.mask_mode == PDLLM_MASK_CAUSAL;
    m.t_lin = plan.t_lin; m.span = plan.span; m.max_pieces = plan.max_pieces; m.head = plan.head;
    const long mrows = (long)d->n_req * d->max_q_len * d->num_q_heads;
    const int merge_blocks = (int)((mrows + 15) / 16);  // 16 rows per workgroup
    if (store_in_merge) {
      m.store_slots = d->active_slot_mapping;
      m.k_new = static_cast<const uint4*>(d->k_new);
      m.v_new = static_cast<const uint4*>(d->v_new);
      m.k_cache = static_cast<uint4*>(const_cast<void*>(d->k_cache));
      m.v_cache = static_cast<uint4*>(const_cast<void*>(d->v_cache));
      m.kn_stride16 = d->kn_stride / 8;
      m.vn_stride16 = d->vn_stride / 8;
      m.n_slots = d->n_pages * (int64_t)d->page_size;
      const long chunks = d->n_tokens * d->num_kv_heads * (kD / 8);
      m.store_blocks = (int)((chunks + 255) / 256);
    }
    hipLaunchKernelGGL(attn_merge_kernel, dim3((unsigned)(merge_blocks + m.store_blocks)), dim3(256), 0, stream, m);
    st = launch_status();
  }
  return st;
}

}  // namespace pdllm

extern "C" int64_t pdllm_attn_workspace_bytes(const pdllm_attn_desc* desc) {
  const int st = pdllm::validate_desc(desc, false);
  if (st != PDLLM_OK) return st;
  return pdllm::ws_bytes_for(desc, pdllm::make_plan(desc, false).max_pieces, false);
}

extern "C" int64_t pdllm_attn_slot_table_stride(const pdllm_attn_desc* desc) {
  if (!desc) return PDLLM_ERR_NULL;
  if (desc->max_ctx_len < 0) return PDLLM_ERR_SHAPE;
  return pdllm::slot_table_stride_for(desc);
}

extern "C" int pdllm_attn_build_slot_table(const pdllm_attn_desc* desc, int32_t* table, int64_t table_stride,
                                           pdllm_stream_t stream) {
  if (!desc || !table) return PDLLM_ERR_NULL;
  if (!desc->block_table || !desc->range_ptr || !desc->range_start || !desc->range_len) return PDLLM_ERR_NULL;
  if (desc->n_req <= 0 || desc->max_ctx_len <= 0 || desc->bt_stride <= 0) return PDLLM_ERR_SHAPE;
  if (pdllm::ilog2_exact(desc->page_size) < 0) return PDLLM_ERR_SHAPE;
  if (desc->n_pages <= 0 || desc->n_pages * (int64_t)desc->page_size >= (1ll << 31)) return PDLLM_ERR_SHAPE;
  if (desc->max_ranges < 0 || desc->max_ranges > pdllm::kMaxRanges) return PDLLM_ERR_UNSUPPORTED;
  if (table_stride < pdllm::slot_table_stride_for(desc) || ((uintptr_t)table % 4)) return PDLLM_ERR_STRIDE;
  pdllm::AttnKParams p = {};
  pdllm::fill_table_params(desc, p);
  p.slot_stride = table_stride;
  return pdllm::launch_slot_table(p, desc->n_req, table, static_cast<hipStream_t>(stream));
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

extern "C" int pdllm_attn_plan_describe(const pdllm_attn_desc* desc, int32_t prefill, char* text, int32_t text_bytes) {
  const int st = pdllm::validate_desc(desc, prefill != 0);
  if (st != PDLLM_OK) return st;
  if (text == nullptr || text_bytes <= 0) return PDLLM_ERR_NULL;
  if (prefill) {
    int grid = 0, team = 0;
    if (pdllm::prefill_stream_plan(desc, pdllm::compute_units(), &grid, &team)) {
      const int n = snprintf(text, (size_t)text_bytes, "attn_prefill_stream_kernel kv=bf16 row_blocks=4 grid=%d team=%d", grid, team);
      return n > 0 && n < text_bytes ? PDLLM_OK : PDLLM_ERR_SHAPE;
    }
  }
  const pdllm::AttnPlan plan = pdllm::make_plan(desc, prefill != 0);
  const bool fp8 = !prefill && desc->k_cache != nullptr && desc->max_ctx_len > 0 && desc->kv_dtype == PDLLM_KV_FP8_E4M3;
  const char* kernel = plan.J == 8 && !fp8 ? "attn_fwd2_kernel" : "attn_fwd_kernel";
  // (the bytes of a partial row are part of the text: traffic figures taken for one format do not describe another)
  const int n = snprintf(text, (size_t)text_bytes,
                         "%s kv=%s row_blocks=%d grid=%d span=%d head=%d set=%d tiles=%d pieces=%d partial_row_bytes=%d",
                         kernel, fp8 ? "fp8" : "bf16", plan.J, plan.grid, plan.span, plan.head, plan.wg_set,
                         plan.t_lin, plan.max_pieces, plan.max_pieces > 1 ? pdllm::kD * 2 + 4 + 16 : 0);
  return n > 0 && n < text_bytes ? PDLLM_OK : PDLLM_ERR_SHAPE;
}

extern "C" int pdllm_attn_plan(const pdllm_attn_desc* desc, int32_t prefill, int32_t* rows_per_group,
                               int32_t* num_splits) {
  const int st = pdllm::validate_desc(desc, prefill != 0);
  if (st != PDLLM_OK) return st;
  const pdllm::AttnPlan plan = pdllm::make_plan(desc, prefill != 0);
  if (rows_per_group) *rows_per_group = 32 * plan.J;
  if (num_splits) *num_splits = (plan.t_lin + plan.span - 1) / plan.span;
  return PDLLM_OK;
}
