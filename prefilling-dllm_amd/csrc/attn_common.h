// Shared pieces of the attention kernels for gfx950: tile geometry, the kernel parameter block, and the
// hand-issued LDS operand reads with their explicit wait counts.
#pragma once

#include "pdllm_common.h"

namespace pdllm {

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int kD = 128;          // head dim
constexpr int kKT = 64;          // keys per tile
constexpr int kNKB = kKT / 32;   // 32-key blocks per tile
constexpr int kThreads = 256;    // 4 wavefronts (8 for the 256-row group)
constexpr int kRowBytes = 256;   // one K or V row in LDS
constexpr int kTileBytes = kKT * kRowBytes;      // 16384
constexpr int kBufBytes = 2 * kTileBytes;        // K tile + V tile
constexpr int kMainBytes = 2 * kBufBytes;        // double buffered: 65536
constexpr int kPartBytes = kD * 32 * 4;          // LDS partial of a shared row block: [d][row ^ (d & 31)] fp32
constexpr int kMaxRanges = 128;
constexpr int kMaxTok = 264;                     // query tokens a row group of 256 rows can touch (+ slack)
constexpr float kRescaleSlack = 8.f;             // log2 units
static_assert(4 * kPartBytes <= kMainBytes, "partials must fit the tile buffers");
static_assert(kNKB == 2, "the shared-block schedule assumes two key blocks per tile");

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
  const int* slot_table;  // [n_req, slot_stride]: cache slot of every visible prefix key; last entry = key count
  long slot_stride;
  const uint8_t* mask;
  uint16_t* ws_o;    // partial rows, fp16 with one power-of-two scale per 32 columns (store_partial_block)
  float* ws_lse;     // log-sum-exp of a partial row, log2 units
  float* ws_scale;   // [row][4] scales of the partial rows
  long q_stride, kn_stride, vn_stride, o_stride;
  long cache_page_stride, cache_token_stride, cache_head_stride;
  long mask_stride;
  long n_tokens;
  int n_pages;
  int bt_stride;
  int scale_page_stride, scale_head_stride;
  int n_req, Hq, Hkv, G;
  int page_shift;
  int max_ctx_len;
  int max_ranges;
  int mask_mode;
  int J;
  int row_tiles;
  // work decomposition: the tiles of all columns (request, KV head, row group) form one line of
  // n_cols * t_lin positions that is cut into spans of `span` tiles, one per workgroup
  int t_lin;       // positions per column (>= the largest tile count of a column)
  int span;        // tiles per workgroup
  int n_lin;       // length of the line
  int max_pieces;  // partial results per row in the workspace
  // head == 0: one line over all columns (n_lin = columns * t_lin).  head > 0: the row_tiles columns of
  // one (request, KV head), which read the same K/V tiles, form a set of wg_set workgroups: the first
  // row_tiles of them take the first `head` tiles of one column each, side by side over the same
  // tiles, which they share in L2; the others cut the line of the columns' remaining t_lin - head
  // tiles (n_lin = row_tiles * (t_lin - head) positions) into spans.
  int head;
  int wg_set;
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
// Partial results of a column that is cut into pieces: a row of 128 normalised values is stored as fp16 with one
// power-of-two scale per block of 32 columns -- half the bytes of fp32, rounded (to nearest) at 2^-12 .. 2^-11 of the
// block's largest element, whatever the magnitude of V.  A lane pair (l, l ^ 32) holds the 32 columns of a block: `o`
// are this lane's 16 values (columns 32 db + 8 i + 4 he + 0..3 for i = 0..3), inv = 1 / (sum of the row's weights).
// The block's largest |value| is scaled into [2^14, 2^15).
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_partial_block(uint16_t* row16, float* scale4, int db, int he, const f32x16& o,
                                                    float inv) {
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(o[i]));
  amax = half_swap_max(amax) * inv;
  unsigned ef = (__float_as_uint(amax) >> 23) & 0xffu;  // biased exponent of the largest element
  ef = ef < 15u ? 15u : (ef > 254u ? 254u : ef);
  const float up = __uint_as_float((268u - ef) << 23);  // 2^(14 - E)
  // this lane's values as packed fp16: word 2 i + k = columns 8 i + 4 he + 2 k, + 1
  unsigned w[8];
#pragma unroll
  for (int i4 = 0; i4 < 4; ++i4) {
    const f16x2 a = {(_Float16)(o[4 * i4 + 0] * inv * up), (_Float16)(o[4 * i4 + 1] * inv * up)};
    const f16x2 b = {(_Float16)(o[4 * i4 + 2] * inv * up), (_Float16)(o[4 * i4 + 3] * inv * up)};
    w[2 * i4] = __builtin_bit_cast(unsigned, a);
    w[2 * i4 + 1] = __builtin_bit_cast(unsigned, b);
  }
  // Of the 16 columns 16 j .. 16 j + 15 the lower lane holds 0-3 and 8-11, the upper one 4-7 and 12-15: after
  // exchanging the lower lane's second group with the upper lane's first, each lane stores 16 contiguous bytes
  // (the cost of these stores is their number, not their bytes).
  uint16_t* wp = row16 + 32 * db + 8 * he;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const auto x = __builtin_amdgcn_permlane32_swap(w[4 * j], w[4 * j + 2], false, false);
    const auto y = __builtin_amdgcn_permlane32_swap(w[4 * j + 1], w[4 * j + 3], false, false);
    const uint4 q = {x[0], y[0], x[1], y[1]};
    *reinterpret_cast<uint4*>(wp + 16 * j) = q;
  }
  if (he == 0) scale4[db] = __uint_as_float((ef - 14u) << 23);  // 2^(E - 14)
}

// Position swizzle of the 16 chunks (16 bytes each) of a 256-byte row: chunk c of row r sits at c ^ swz(r).  Any
// bijection of the low four row bits keeps the 128-bit K reads (16 consecutive rows, one chunk) and the copies
// (whole rows) free of bank conflicts.  The transposing 64-bit V reads touch, per group of 32 lanes, four rows
// (row bits 0-1) and four neighbouring chunks of each (chunk bits 0-1): row bits 0-1 therefore go to chunk bits
// 2-3, so that the four rows use four different quarters of the 64 banks.  (With the row bits merely rotated the
// rows collided in pairs and every V read took two passes: measured 2x on the LDS read rate.)
__device__ __forceinline__ int swz(int row) {
  const int r = row & 15;
  return ((r & 3) << 2) | (((r >> 2) & 1) << 1) | (r >> 3);
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

// LDS operand reads of the MFMA loops are issued and awaited by hand.  The compiler would make
// every LDS read wait for the direct-to-LDS copies of the next tile that are in flight (it
// cannot tell that they go to the other buffer), which serialises copy and compute.  The asm
// reads are invisible to its wait-count bookkeeping, so each consumer waits explicitly:
// lds_wait<N>(x) blocks until at most N younger LDS operations are outstanding and ties the
// wait to the registers x that the operation filled.
template <int OFF>
__device__ __forceinline__ void lds_read_b128(bf16x8& dst, unsigned addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_read_tr16_b64(s16x4& dst, unsigned addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int N, typename T>
__device__ __forceinline__ void lds_wait(T& x) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N) : "memory");
}
// the same, and also a fence for two values of the vector pipeline: work that produces them
// stays before this point, work that consumes them after it (pins the interleaving of softmax
// arithmetic with the MFMAs, which the compiler would otherwise gather in one place)
// `keep` is only named as an input: it holds the fragment the MFMA of the step before is still
// reading, and naming it here keeps the register allocator from handing those registers to the
// vector instructions in between (a write to a source of a running MFMA stalls the wave until
// the MFMA has finished, which would serialise the two pipelines).
template <int N, typename T>
__device__ __forceinline__ void lds_wait_pin(T& x, float& a, float& b, const T& keep) {
  asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(x), "+v"(a), "+v"(b) : "n"(N), "v"(keep) : "memory");
}
template <int N, typename T>
__device__ __forceinline__ void lds_wait2(T& x, T& y) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N) : "memory");
}
// the same, and a fence for one value of the vector pipeline (see lds_wait_pin)
template <int N, typename T>
__device__ __forceinline__ void lds_wait2_pin(T& x, T& y, float& a) {
  asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(x), "+v"(y), "+v"(a) : "n"(N) : "memory");
}

// One QK step of the software-pipelined loop as a single statement, so that its order is fixed and no wait state is
// spent between the parts: wait for the K fragment, the MFMA of the next tile's scores, the exponentials of this
// step's two scores (their arguments t0, t1 were formed a step earlier), the arguments u0, u1 of the next step's
// pair, then the pack of the two probabilities into one word and its contribution to the row sum.  Two vector
// instructions lie between an exponential and the instruction that reads it (a transcendental result needs one).
// KIND 0: first MFMA of a key block (starts from zero), 1: accumulates in place, 2 and 3: last MFMA of the block: it
// writes `dst` (the registers of the scores this block has used up; every argument taken from them was formed
// before this step) from the accumulator `acc`.  `keep` names the fragment the MFMA of the step before still reads.
template <int N, int KIND>
__device__ __forceinline__ void qk_step(f32x16& acc, f32x16& dst, const bf16x8& kf, const bf16x8& q, float& t0, float& t1,
                                        float s2, float s3, float c, float negm, float& u0, float& u1, unsigned& pw,
                                        float& psum, const bf16x8& keep) {
  if constexpr (KIND == 0) {
    asm volatile(
        "s_waitcnt lgkmcnt(%[n])\n"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[kf], %[q], 0\n"
        "v_exp_f32 %[t0], %[t0]\n"
        "v_exp_f32 %[t1], %[t1]\n"
        "v_fma_f32 %[u0], %[s2], %[c], %[nm]\n"
        "v_fma_f32 %[u1], %[s3], %[c], %[nm]\n"
        "v_cvt_pk_bf16_f32 %[pw], %[t0], %[t1]\n"
        "v_dot2c_f32_bf16 %[ps], 0x3f803f80, %[pw]\n"
        : [acc] "=&v"(acc), [t0] "+v"(t0), [t1] "+v"(t1), [u0] "=&v"(u0), [u1] "=&v"(u1), [pw] "=&v"(pw), [ps] "+v"(psum)
        : [kf] "v"(kf), [q] "v"(q), [s2] "v"(s2), [s3] "v"(s3), [c] "s"(c), [nm] "v"(negm), [n] "n"(N), "v"(keep)
        : "memory");
  } else if constexpr (KIND == 1) {
    asm volatile(
        "s_waitcnt lgkmcnt(%[n])\n"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[kf], %[q], %[acc]\n"
        "v_exp_f32 %[t0], %[t0]\n"
        "v_exp_f32 %[t1], %[t1]\n"
        "v_fma_f32 %[u0], %[s2], %[c], %[nm]\n"
        "v_fma_f32 %[u1], %[s3], %[c], %[nm]\n"
        "v_cvt_pk_bf16_f32 %[pw], %[t0], %[t1]\n"
        "v_dot2c_f32_bf16 %[ps], 0x3f803f80, %[pw]\n"
        : [acc] "+v"(acc), [t0] "+v"(t0), [t1] "+v"(t1), [u0] "=&v"(u0), [u1] "=&v"(u1), [pw] "=&v"(pw), [ps] "+v"(psum)
        : [kf] "v"(kf), [q] "v"(q), [s2] "v"(s2), [s3] "v"(s3), [c] "s"(c), [nm] "v"(negm), [n] "n"(N), "v"(keep)
        : "memory");
  } else if constexpr (KIND == 3) {  // the last step of a tile: no next pair; the MFMA separates the exponentials from the pack
    asm volatile(
        "s_waitcnt lgkmcnt(%[n])\n"
        "v_exp_f32 %[t0], %[t0]\n"
        "v_exp_f32 %[t1], %[t1]\n"
        "v_mfma_f32_32x32x16_bf16 %[dst], %[kf], %[q], %[acc]\n"
        "v_cvt_pk_bf16_f32 %[pw], %[t0], %[t1]\n"
        "v_dot2c_f32_bf16 %[ps], 0x3f803f80, %[pw]\n"
        : [dst] "=&v"(dst), [t0] "+v"(t0), [t1] "+v"(t1), [pw] "=&v"(pw), [ps] "+v"(psum)
        : [acc] "v"(acc), [kf] "v"(kf), [q] "v"(q), [n] "n"(N), "v"(keep)
        : "memory");
  } else {
    asm volatile(
        "s_waitcnt lgkmcnt(%[n])\n"
        "v_mfma_f32_32x32x16_bf16 %[dst], %[kf], %[q], %[acc]\n"
        "v_exp_f32 %[t0], %[t0]\n"
        "v_exp_f32 %[t1], %[t1]\n"
        "v_fma_f32 %[u0], %[s2], %[c], %[nm]\n"
        "v_fma_f32 %[u1], %[s3], %[c], %[nm]\n"
        "v_cvt_pk_bf16_f32 %[pw], %[t0], %[t1]\n"
        "v_dot2c_f32_bf16 %[ps], 0x3f803f80, %[pw]\n"
        : [dst] "=&v"(dst), [t0] "+v"(t0), [t1] "+v"(t1), [u0] "=&v"(u0), [u1] "=&v"(u1), [pw] "=&v"(pw), [ps] "+v"(psum)
        : [acc] "v"(acc), [kf] "v"(kf), [q] "v"(q), [s2] "v"(s2), [s3] "v"(s3), [c] "s"(c), [nm] "v"(negm), [n] "n"(N), "v"(keep)
        : "memory");
  }
}

// One PV step as a single statement: wait for the V^T fragment of this step, its MFMA, and the reads of the
// fragment two steps ahead into the registers the MFMA has just taken its operand from.  The two 64-bit transposing
// reads of a fragment have to land in the two halves of one 128-bit operand; an asm operand cannot be addressed
// by halves, so the two staging operands are pinned to fixed registers (v[248:251] and v[252:255]) and the text
// names the halves.  WHICH selects the staging operand, N the outstanding LDS operations to wait for, OFF the
// immediate offset of the reads (a negative OFF: no reads, the last two steps).  `pin` is only named: it orders
// the vector instruction that produced it in front of this statement.
template <int WHICH, int OFF>
__device__ __forceinline__ void pv_read(bf16x8& a, unsigned x, unsigned y) {
  if constexpr (WHICH == 0)
    asm volatile("ds_read_b64_tr_b16 v[248:249], %1 offset:%3\n ds_read_b64_tr_b16 v[250:251], %2 offset:%3"
                 : "={v[248:251]}"(a) : "v"(x), "v"(y), "n"(OFF) : "memory");
  else
    asm volatile("ds_read_b64_tr_b16 v[252:253], %1 offset:%3\n ds_read_b64_tr_b16 v[254:255], %2 offset:%3"
                 : "={v[252:255]}"(a) : "v"(x), "v"(y), "n"(OFF) : "memory");
}
template <int WHICH, int N, int OFF, typename P4>
__device__ __forceinline__ void pv_step(f32x16& o, bf16x8& a, const P4& p, unsigned x, unsigned y, float pin) {
  if constexpr (OFF >= 0) {
    if constexpr (WHICH == 0)
      asm volatile("s_waitcnt lgkmcnt(%6)\n v_mfma_f32_32x32x16_bf16 %0, v[248:251], %2, %0\n"
                   "ds_read_b64_tr_b16 v[248:249], %3 offset:%7\n ds_read_b64_tr_b16 v[250:251], %4 offset:%7"
                   : "+v"(o), "+{v[248:251]}"(a) : "v"(p), "v"(x), "v"(y), "v"(pin), "n"(N), "n"(OFF) : "memory");
    else
      asm volatile("s_waitcnt lgkmcnt(%6)\n v_mfma_f32_32x32x16_bf16 %0, v[252:255], %2, %0\n"
                   "ds_read_b64_tr_b16 v[252:253], %3 offset:%7\n ds_read_b64_tr_b16 v[254:255], %4 offset:%7"
                   : "+v"(o), "+{v[252:255]}"(a) : "v"(p), "v"(x), "v"(y), "v"(pin), "n"(N), "n"(OFF) : "memory");
  } else {
    if constexpr (WHICH == 0)
      asm volatile("s_waitcnt lgkmcnt(%4)\n v_mfma_f32_32x32x16_bf16 %0, v[248:251], %2, %0"
                   : "+v"(o), "+{v[248:251]}"(a) : "v"(p), "v"(pin), "n"(N) : "memory");
    else
      asm volatile("s_waitcnt lgkmcnt(%4)\n v_mfma_f32_32x32x16_bf16 %0, v[252:255], %2, %0"
                   : "+v"(o), "+{v[252:255]}"(a) : "v"(p), "v"(pin), "n"(N) : "memory");
  }
}

}  // namespace pdllm
