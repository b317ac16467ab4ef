// Block-diagonal chunk prefill attention for gfx950 (MI355X), stream form.
//
// Replaces the prefill branch of the reference's attention layer for a packed batch of independent chunks
// (layers/attention/attention_v4.py:336-367 with the block-diagonal mask of utils/context.py:73-84, causal or
// full inside a chunk) when the batch is large enough to keep every compute unit busy with resident
// workgroups; attn_fwd_kernel (attn_kernel.hip) serves every other case with one workgroup per column.
//
// Why a second kernel.  A column is one (chunk, KV head, group of 128 rows; a row is a (token, q-head of the GQA
// group) pair).  Under a causal mask a column of a 1025-token chunk has 1 to 17 tiles of 64 keys, 8.7 on
// average, and a workgroup that handles one column spends a third of its life before its first MFMA (three
// dependent round trips to memory, an unpipelined first QK^T) and after its last one (normalise, store, drain).
// Here 2 x (compute units) workgroups stay resident and each walks a *stream* of tiles that runs through all
// of its columns: the software pipeline of the tile loop -- scores of tile t + 1 on the matrix unit while the
// vector unit turns the scores of tile t into probabilities, K two tiles and V one tile ahead in LDS -- does not
// drain at a column boundary.  The Q fragments of the next column are loaded into the registers of the current
// ones right after their last use (the QK^T of the column's last tile runs one iteration before its softmax),
// the output rows of a finished column are normalised and stored at the start of the next iteration, behind
// the barrier, so that their stores fly under the following tiles.
//
// Schedule.  The units (chunk, KV head) are dealt to teams of `team` workgroups that sit on one XCD (they share
// the unit's K/V through its L2); inside a unit the columns, longest first under a causal mask, are dealt to
// the team's workgroups in snake order (j, 2 team - 1 - j, 2 team + j, ...), mirrored for every other unit, so
// that every workgroup gets the same number of tiles within a few per cent.  A workgroup computes the list of its
// columns once, at its start, into LDS.
//
// Tile loop, LDS layout (rows of 256 bytes, 16-byte chunks XOR-swizzled), MFMA operand layouts, the statements
// of a QK^T step and of a PV step, the lazy rescale and the fp32 softmax scale are those of attn_fwd_kernel
// (attn_common.h).

#include <type_traits>

#include "attn_common.h"

namespace pdllm {

namespace {

constexpr int kMaxPieces = 256;  // columns one workgroup can be given (the host checks)

struct PrefillParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* out;
  const int* q_start_loc;
  long q_stride, o_stride;  // elements
  unsigned kv_row_bytes;    // token pitch of k and of v (equal), bytes
  unsigned out_bytes;       // bytes from out to the end of its last row
  long n_tokens;
  int n_req, Hq, Hkv, G;
  int causal;
  int max_q_len;
  int R;        // row groups of 128 rows a unit has at most
  int team;     // workgroups per team
  int n_teams;  // grid = n_teams * team
  int n_units;  // n_req * Hkv
  float scale_log2;
};

// A column: as the workgroup's list holds it in LDS, and (in scalar registers) as the tile loop uses it
struct alignas(16) Piece {
  int q0;    // first token row of the chunk
  int Sq;    // tokens of the chunk
  int Sa;    // keys the column sees (tokens 0 .. Sa - 1 of the chunk)
  int kvh;   // KV head
  int row0;  // first row of the column inside the chunk (a row is token * G + head of the group)
  int tq0;   // token of that row
  int T;     // tiles of 64 keys; 0 = no column
  int pad;
};

}  // namespace

__global__ __launch_bounds__(256, 2) void attn_prefill_stream_kernel(const PrefillParams p) {
  constexpr int NW = 4, kDmaGroups = 4, NS = 16, PF = 2;
  __shared__ __attribute__((aligned(1024))) char lds[kMainBytes];
  __shared__ Piece s_piece[kMaxPieces];
  __shared__ int s_npieces;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int h = lane >> 5;
  const int G = p.G;
  const float c = p.scale_log2;
  const unsigned lds_base = (unsigned)(size_t)lds;

  // ---- the list of this workgroup's columns ----
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  const int team_id = wg / p.team;
  const int jw = wg - team_id * p.team;
  const int units_here = (p.n_units - team_id + p.n_teams - 1) / p.n_teams;  // units of this team
  // Causal: inside every unit the columns, longest first, go to the team's workgroups in snake order, mirrored for
  // every other unit -- long and short columns pair up and every workgroup gets the same number of tiles within a
  // few per cent.  Full mask (all columns equally long): one snake through the columns of all the team's units,
  // so that the column counts of two workgroups differ by one at most.
  const int i_max = (p.R + p.team - 1) / p.team;  // columns of a unit per workgroup at most
  const int n_cand = p.causal ? units_here * i_max : (units_here * p.R + p.team - 1) / p.team;
  if (tid == 0) s_npieces = 0;
  __syncthreads();
  if (wave == 0) {
    // 64 candidates at a time, kept in order
    int base = 0;
    for (int c0 = 0; c0 < n_cand; c0 += 64) {
      const int idx = c0 + lane;
      Piece pc = {0, 0, 0, 0, 0, 0, 0, 0};
      bool ok = false;
      if (idx < n_cand) {
        int k, pos;
        if (p.causal) {
          // candidate = (k-th unit of the team, i-th column of the workgroup in it)
          k = idx / i_max;
          const int i = idx - k * i_max;
          const int j = (k & 1) ? p.team - 1 - jw : jw;
          pos = (i & 1) ? i * p.team + (p.team - 1 - j) : i * p.team + j;
        } else {
          // candidate = round idx of the snake through units_here * R columns
          const int at = idx * p.team + ((idx & 1) ? p.team - 1 - jw : jw);
          k = at / p.R;
          pos = k < units_here ? at - k * p.R : p.R;
        }
        const int unit = team_id + k * p.n_teams;
        if (unit < p.n_units && pos < p.R) {
          const int seq = unit / p.Hkv, kvh = unit - seq * p.Hkv;
          const int r = p.causal ? p.R - 1 - pos : pos;  // causal: the columns with the most keys first
          const int q0 = p.q_start_loc[seq];
          const int Sq = p.q_start_loc[seq + 1] - q0;
          if (q0 >= 0 && Sq > 0 && (long)q0 + Sq <= p.n_tokens && Sq <= p.max_q_len) {
            const int rows = Sq * G, row0 = r * 128;
            if (row0 < rows) {
              int Sa = Sq;
              if (p.causal) {
                const int last_row = (row0 + 128 < rows ? row0 + 128 : rows) - 1;
                const int lim = last_row / G + 1;
                Sa = lim < Sq ? lim : Sq;
              }
              pc = {q0, Sq, Sa, kvh, row0, row0 / G, (Sa + kKT - 1) / kKT, 0};
              ok = true;
            }
          }
        }
      }
      const unsigned long bal = __builtin_amdgcn_ballot_w64(ok);
      const int before = __builtin_popcountl(bal & ((1ul << lane) - 1ul));
      if (ok && base + before < kMaxPieces) s_piece[base + before] = pc;
      base += __builtin_popcountl(bal);
    }
    if (lane == 0) s_npieces = base < kMaxPieces ? base : kMaxPieces;
  }
  __syncthreads();
  const int n_pieces = __builtin_amdgcn_readfirstlane(s_npieces);
  if (n_pieces == 0) return;

  // ---- per-lane LDS operand addresses (buffer 0; buffer and key block are instruction immediates) ----
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

  // ---- copies HBM -> LDS: this wave moves rows 16 i + 4 wave + lane / 16 of a tile, i < 4 ----
  const int lane_row = 4 * wave + (lane >> 4);
  const int lane_ch = (lane & 15) ^ swz(lane_row);
  const unsigned lane_b16 = (unsigned)lane_ch << 4;
  // byte offset of this lane's chunk of row lane_row behind the tile's first row (rows 16 i further go through
  // the uniform offset of the copy)
  const unsigned voff0 = (unsigned)lane_row * p.kv_row_bytes + lane_b16;
  unsigned wave_lds = lds_base + wave * 1024;
  const __amdgpu_buffer_rsrc_t k_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<__bf16*>(p.k), 0, 0xffffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<__bf16*>(p.v), 0, 0xffffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t q_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<__bf16*>(p.q), 0, 0xffffffff, 0x00020000);
  // the output's size in bytes bounds its stores: offsets of rows that do not exist lie behind it
  const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, p.out_bytes, 0x00020000);
  // copy group i of tile `tile` of column pc into LDS offset dst_off of this wave's part
  // (whole_tag: the tile is known to be a whole tile of the column)
  auto copy_group = [&](const __amdgpu_buffer_rsrc_t& rs, const Piece& pc, int tile, int i, unsigned dst_off,
                        auto whole_tag) __attribute__((always_inline)) {
    auto* dst = (__attribute__((address_space(3))) char*)(size_t)(wave_lds + dst_off);
    const unsigned head_b = (unsigned)pc.kvh * (kD * 2);
    const int a0 = tile * kKT;
    if (decltype(whole_tag)::value || a0 + kKT <= pc.Sa) {
      // a whole tile: uniform offset of the group's first row, constant lane offset
      const unsigned so = (unsigned)(pc.q0 + a0 + 16 * i) * p.kv_row_bytes + head_b;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)dst, 16, voff0, so, 0, 0);
    } else {
      // a ragged last tile: rows past the column's keys repeat its last key (they are masked)
      int a = a0 + 16 * i + lane_row;
      a = a < pc.Sa ? a : pc.Sa - 1;
      const unsigned vo = (unsigned)(pc.q0 + a) * p.kv_row_bytes + head_b + lane_b16;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)dst, 16, vo, 0, 0, 0);
    }
  };

  // ---- the columns in flight: P0 holds the tile the softmax works on, P1 and P2 follow it in the list ----
  Piece P0, P1, P2;
  int next_piece = 0;
  auto fetch_piece = [&](Piece& dst) __attribute__((always_inline)) {
    if (next_piece >= n_pieces) {
      dst.T = 0;
      return;
    }
    const int4 lo = *reinterpret_cast<const int4*>(&s_piece[next_piece]);
    const int4 hi = *(reinterpret_cast<const int4*>(&s_piece[next_piece]) + 1);
    ++next_piece;
    dst.q0 = __builtin_amdgcn_readfirstlane(lo.x);
    dst.Sq = __builtin_amdgcn_readfirstlane(lo.y);
    dst.Sa = __builtin_amdgcn_readfirstlane(lo.z);
    dst.kvh = __builtin_amdgcn_readfirstlane(lo.w);
    dst.row0 = __builtin_amdgcn_readfirstlane(hi.x);
    dst.tq0 = __builtin_amdgcn_readfirstlane(hi.y);
    dst.T = __builtin_amdgcn_readfirstlane(hi.z);
  };

  // token of this lane's row in column pc (of the column's first row for a row past the chunk's rows)
  auto row_token = [&](const Piece& pc, int lane_e) __attribute__((always_inline)) {
    const int r = pc.row0 + 32 * wave + (lane_e & 31);
    return (int)((unsigned)(r < pc.Sq * G ? r : pc.row0) / (unsigned)G);
  };
  // a lower bound of the token of this wave's first row behind the token of the column's first row
  const int wave_tok = __builtin_amdgcn_readfirstlane((int)((unsigned)(32 * wave) / (unsigned)G));

  // Q fragments (B operand of S^T = K Q^T) of column pc.  Always eight loads per lane (the wait at the end of an
  // iteration counts them): a lane whose row lies past the chunk's rows loads the column's first row instead and
  // computes a duplicate that is never stored.
  bf16x8 QA[8];
  auto q_address = [&](const Piece& pc) __attribute__((always_inline)) {
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));  // (keeps the address arithmetic next to its use)
    const int r = pc.row0 + 32 * wave + (lane_e & 31);
    const int rr = r < pc.Sq * G ? r : pc.row0;
    const int tq = rr / G;
    const int g = rr - tq * G;
    // byte offset behind p.q (the launch is made only when Q and the output lie below 4 GiB: a buffer load with a
    // 32-bit offset costs the issuing wave a fraction of a load with a 64-bit address per lane)
    return 2u * ((unsigned)(pc.q0 + tq) * (unsigned)p.q_stride + (unsigned)((pc.kvh * G + g) * kD + 8 * (lane_e >> 5)));
  };
  auto load_q = [&](const Piece& pc) __attribute__((always_inline)) {
    const unsigned qo = q_address(pc);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      QA[ks] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(q_rs, (int)qo + 32 * ks, 0, 0));
  };

  f32x16 OA[4];
  float MA = -INFINITY, lA = 0.f;
  int fresh = 1;  // the accumulators belong to a finished column: the next tile starts them from zero

  // Normalised output rows of column pc (its accumulators are complete).  The rows go through LDS, 64 columns at
  // a time, so that 8 lanes store the 128 contiguous bytes of a row instead of 8-byte pieces of 32 different rows
  // (every store instruction then touches 8 cache lines instead of 32; the scattered form cost a sixth of the
  // launch).  The strip is this wave's own part of the V region of buffer `par` -- the four 1 KB pieces its copies
  // of the V tile after the next one will overwrite: that tile's predecessor in the buffer has been consumed by every
  // wave (the caller stands behind the barrier), and only this wave writes there again, later in its own
  // program order.  Row r lies in piece r / 8 at (r % 8) * 128 bytes, its 16-byte chunk c at position
  // c ^ ((r / 2) % 8): writes and reads take the minimal number of LDS passes.
  auto emit = [&](const Piece& pc, int par) __attribute__((always_inline)) {
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int l32e = lane_e & 31, he = lane_e >> 5;
    const float lsum = half_swap_sum(lA);
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
    const int r = pc.row0 + 32 * wave + l32e;
    // byte offset of this lane's row behind p.out; a row that does not exist gets an offset past the buffer's
    // size, and the hardware drops a buffer store that lies out of range
    unsigned rowoff = 0xfffff000u;
    if (r < pc.Sq * G) {
      const int srow = row_token(pc, lane_e);
      const int g = r - srow * G;
      rowoff = 2u * ((unsigned)(pc.q0 + srow) * (unsigned)p.o_stride + (unsigned)((pc.kvh * G + g) * kD));
    }
    char* strip = lds + par * kBufBytes + kTileBytes + wave * 1024;
    char* wrow = strip + (l32e >> 3) * 4096 + (l32e & 7) * 128 + 8 * he;
    const int wsw = (l32e >> 1) & 7;
    const int j = lane_e & 7;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
      for (int dd = 0; dd < 2; ++dd)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          const f32x16& o = OA[2 * hf + dd];
          uint2 w;
          w.x = pack_bf16x2(o[4 * i4 + 0] * inv, o[4 * i4 + 1] * inv);
          w.y = pack_bf16x2(o[4 * i4 + 2] * inv, o[4 * i4 + 3] * inv);
          *reinterpret_cast<uint2*>(wrow + (((4 * dd + i4) ^ wsw) << 4)) = w;
        }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int rr = 8 * k + (lane_e >> 3);
        const unsigned dst = (unsigned)__shfl((int)rowoff, rr, 64);
        typedef unsigned u32x4s __attribute__((ext_vector_type(4)));
        const u32x4s x = *reinterpret_cast<const u32x4s*>(strip + k * 4096 + (rr & 7) * 128 + ((j ^ ((rr >> 1) & 7)) << 4));
        __builtin_amdgcn_raw_buffer_store_b128(x, o_rs, (int)(dst + 2u * (64 * hf + 8 * j)), 0, 0);
      }
    }
    MA = -INFINITY;
    lA = 0.f;
    fresh = 1;
  };

  auto rdkp = [&](bf16x8& dst, int stp, auto par_tag) __attribute__((always_inline)) {
    constexpr int boff = decltype(par_tag)::value == 0 ? kBufBytes : 0;  // K(t+1) of an even iteration: buffer 1
    if ((stp >> 3) == 0) lds_read_b128<boff>(dst, ka[stp & 7]);
    else lds_read_b128<boff + 32 * kRowBytes>(dst, ka[stp & 7]);
  };

  // ---- cold start: K and V of the first tile, then K of the second one while QK of the first runs unpipelined ----
  fetch_piece(P0);
  fetch_piece(P1);
  fetch_piece(P2);
  int ti = 0;  // tile of P0 the softmax works on
  load_q(P0);
#pragma unroll
  for (int i = 0; i < kDmaGroups; ++i) {
    copy_group(k_rs, P0, 0, i, (unsigned)(i * (NW * 1024)), std::false_type{});
    copy_group(v_rs, P0, 0, i, (unsigned)(kTileBytes + i * (NW * 1024)), std::false_type{});
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  {
    const bool same = P0.T > 1;
    if (same || P1.T > 0) {
#pragma unroll
      for (int i = 0; i < kDmaGroups; ++i) {
        if (same) copy_group(k_rs, P0, 1, i, (unsigned)(kBufBytes + i * (NW * 1024)), std::false_type{});
        else copy_group(k_rs, P1, 0, i, (unsigned)(kBufBytes + i * (NW * 1024)), std::false_type{});
      }
    }
  }
  f32x16 SX[2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int i = 0; i < 16; ++i) SX[b][i] = 0.f;
  {
    bf16x8 kf[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) rdkp(kf[i], i, std::integral_constant<int, 1>{});  // buffer 0
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int stp = 0; stp < NS; ++stp) {
      const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;
      if (young == 1) lds_wait<1>(kf[stp % PF]);
      else lds_wait<0>(kf[stp % PF]);
      SX[stp >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[stp % PF], QA[stp & 7], SX[stp >> 3], 0, 0, 0);
      if (stp + PF < NS) rdkp(kf[stp % PF], stp + PF, std::integral_constant<int, 1>{});
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float mx_carry;
  {
    float m0 = fmaxf(SX[0][0], SX[0][1]);
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = (b == 0 ? 2 : 0); i < 16; i += 2) m0 = fmaxf(fmaxf(m0, SX[b][i]), SX[b][i + 1]);
    mx_carry = half_swap_max(m0) * c;
  }
  // the second tile of the stream opens a new column (the first one has a single tile): its Q replaces the first one's
  if (P0.T == 1 && P1.T > 0) load_q(P1);
  // from here on ka reads the next tile's K (buffer 1 at an even position of the stream) and va this tile's V
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) ka[ks] += kBufBytes;
  int flip = kBufBytes;  // ka: buffer 1 -> 0 -> 1 ..., va: buffer 0 -> 1 -> 0 ...
  int par_rt = 0;        // parity of the stream position
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  // ---- one iteration: softmax of tile `ti` of P0 (scores in SX) interleaved with QK^T of the stream's next tile,
  // then PV of the tile.  The parity of the stream position is the buffer of this tile's V; the next tile's K sits
  // in the other buffer.  PARC = 0 / 1: an iteration of known parity in the loop unrolled by two, where ka and va
  // stay on buffer 0 and the buffer is part of the immediate offsets; -1: ka and va point at the buffers in use
  // and move to the other ones afterwards.  KIND says where the two following tiles of the stream lie:
  //   0  both in P0 (three or more tiles of P0 left)
  //   1  the next one is P0's last tile, the one after it P1's first: P1's Q fragments are loaded after the QK steps
  //   2  this is P0's last tile: the next one is P1's first, the one after it P1's second or P2's first (then P2's Q
  //      is loaded); P0's rows are written and the columns move up
  // plain_tag (KIND 0 only): the tile needs no mask for any wave and the tile whose K is copied is a whole one.
  auto iter = [&](auto par_tag, auto kind_tag, auto plain_tag) __attribute__((always_inline)) {
    constexpr int PARC = decltype(par_tag)::value;
    constexpr int KIND = decltype(kind_tag)::value;
    constexpr bool PLAIN = decltype(plain_tag)::value;
    const int PAR = PARC >= 0 ? PARC : par_rt;
    // (the LDS address of this wave's part, made opaque once per iteration: the copy destinations are then one
    // scalar add each instead of sixteen loop-invariant scalars)
    {
      unsigned wl = lds_base + wave * 1024;
      asm volatile("" : "+v"(wl));
      wave_lds = __builtin_amdgcn_readfirstlane(wl);
    }
    const int a0 = ti * kKT;
    const bool has_next = KIND != 2 || P1.T > 0;
    // the column whose Q fragments this iteration loads after its QK steps (if any)
    const bool q_from_p1 = KIND == 1 && P1.T > 0;
    const bool q_from_p2 = KIND == 2 && P1.T == 1 && P2.T > 0;
    // ---- mask, row maximum, lazy rescale ----
    // The tile needs a mask when it reaches past the keys of the column or, under a causal mask, past the token
    // of the wave's first row (its smallest; a lower bound of it will do); otherwise its row maximum is known
    // from the iteration before.
    const bool masked = !PLAIN && (a0 + kKT > P0.Sa || (p.causal && a0 + kKT - 1 > P0.tq0 + wave_tok));
    float mx;
    if (masked) {
      int lim = P0.Sa - a0;
      if (p.causal) { const int cl = row_token(P0, lane) - a0 + 1; lim = cl < lim ? cl : lim; }
      // element i of block b is key 32 b + 8 (i / 4) + 4 h + i % 4 of the tile: visible while that is below lim
      const int lim_h = lim - 4 * h;
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) SX[b][i] = (32 * b + 8 * (i >> 2) + (i & 3)) < lim_h ? SX[b][i] : -INFINITY;
      mx = fmaxf(SX[0][0], SX[0][1]);
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int i = (b == 0 ? 2 : 0); i < 16; i += 2) mx = fmaxf(fmaxf(mx, SX[b][i]), SX[b][i + 1]);
      mx = half_swap_max(mx) * c;
    } else {
      mx = mx_carry;
    }
    if (fresh) {
      // first tile of a column: the accumulators start from zero, the maximum from this tile's
      fresh = 0;
      MA = mx;
      lA = 0.f;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) OA[db][i] = 0.f;
    } else {
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
    }
    // ---- exponentials of the tile, two per step, between the MFMAs of the next tile's QK^T ----
    float negM = (MA == -INFINITY) ? 0.f : -MA;
    f32x16 Sn[2];
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    u32x4 PW[2][2];  // probabilities of the tile, two bf16 per word: the B operands of PV
    const bf16x2 ones = {(__bf16)1.f, (__bf16)1.f};
    float psum = 0.f;
    if (has_next) {
      // where the tile after the next one lies (its K is copied now)
      const bool k_in_p1 = KIND == 2 && P1.T > 1;
      const bool k_on = KIND == 0 || (KIND == 1 ? P1.T > 0 : (k_in_p1 || P2.T > 0));
      bf16x8 kf[PF];
#pragma unroll
      for (int i = 0; i < PF; ++i) rdkp(kf[i], i, par_tag);
      bf16x8 used = kf[0];
      float t0 = __builtin_fmaf(SX[0][0], c, negM), t1 = __builtin_fmaf(SX[0][1], c, negM);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int stp = 0; stp < NS; ++stp) {
        const int b = stp >> 3;
        const int nb = (stp + 1) >> 3, ni = 2 * ((stp + 1) & 7);
        const float s2v = stp + 1 < NS ? SX[nb & 1][ni] : 0.f, s3v = stp + 1 < NS ? SX[nb & 1][ni + 1] : 0.f;
        float u0 = 0.f, u1 = 0.f;
        unsigned pw;
        constexpr int kLast = NS - 1;
        const int young = NS - 1 - stp < PF - 1 ? NS - 1 - stp : PF - 1;
#define PDLLM_QK_STEP(KND, ACC, DST)                                                                                   \
  do {                                                                                                                 \
    if (young == 1) qk_step<1, KND>(ACC, DST, kf[stp % PF], QA[stp & 7], t0, t1, s2v, s3v, c, negM, u0, u1, pw, psum, used); \
    else qk_step<0, KND>(ACC, DST, kf[stp % PF], QA[stp & 7], t0, t1, s2v, s3v, c, negM, u0, u1, pw, psum, used);            \
  } while (0)
        if (stp == kLast) PDLLM_QK_STEP(3, Sn[b], SX[b]);
        else if ((stp & 7) == 7) PDLLM_QK_STEP(2, Sn[b], SX[b]);
        else if ((stp & 7) == 0) PDLLM_QK_STEP(0, Sn[b], Sn[b]);
        else PDLLM_QK_STEP(1, Sn[b], Sn[b]);
#undef PDLLM_QK_STEP
        used = kf[stp % PF];
        PW[b][(stp & 7) >> 2][stp & 3] = pw;
        t0 = u0;
        t1 = u1;
        if (stp + PF < NS) rdkp(kf[stp % PF], stp + PF, par_tag);
        // the copies of the next tile's V and of the K of the tile after it, one per second step (a burst would
        // block the wave on the memory pipeline)
        if ((stp & 1) == 1) {
          const int i = (stp & 7) >> 1;
          if (stp < 8) {
            const unsigned dst = (unsigned)((PAR ^ 1) * kBufBytes + kTileBytes + i * (NW * 1024));
            if (KIND == 2) copy_group(v_rs, P1, 0, i, dst, std::false_type{});
            else if (KIND == 1) copy_group(v_rs, P0, ti + 1, i, dst, std::false_type{});
            else copy_group(v_rs, P0, ti + 1, i, dst, std::true_type{});  // not the column's last tile
          } else if (k_on) {
            const unsigned dst = (unsigned)(PAR * kBufBytes + i * (NW * 1024));
            if (KIND == 0) copy_group(k_rs, P0, ti + 2, i, dst, plain_tag);
            else if (KIND == 1) copy_group(k_rs, P1, 0, i, dst, std::false_type{});
            else if (k_in_p1) copy_group(k_rs, P1, 1, i, dst, std::false_type{});
            else copy_group(k_rs, P2, 0, i, dst, std::false_type{});
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // The tile after the next one opens a new column: the scores of the old column's last tile are done, its Q
      // fragments make room for the new ones; they arrive under the PV steps below.  (Handing the eight loads
      // out over the second half of the QK steps, each behind the last use of the fragment it replaces, measured
      // slower: a load that waits for room in the address queue holds up the MFMAs behind it.)
      if (q_from_p1) load_q(P1);
      else if (q_from_p2) load_q(P2);
    } else {
#pragma unroll
      for (int stp = 0; stp < NS; ++stp) {
        const int b = stp >> 3, i = 2 * (stp & 7);
        const bf16x2 pr = {(__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(SX[b][i], c, negM)),
                           (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(SX[b][i + 1], c, negM))};
        psum = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, psum, false);
        PW[b][(stp & 7) >> 2][stp & 3] = __builtin_bit_cast(unsigned, pr);
      }
    }
    lA += psum;
    __builtin_amdgcn_sched_barrier(0);
    // ---- PV of the tile ----
    {
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
    /* unmasked row maximum of the next tile's scores (SX holds them since the QK steps) */                          \
    mnext = stp == 0 ? fmaxf(SX[0][0], SX[0][1])                                                                        \
                     : fmaxf(fmaxf(mnext, SX[stp >> 3][2 * (stp & 7)]), SX[stp >> 3][2 * (stp & 7) + 1]);               \
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
    par_rt ^= 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the copies and the next Q have landed
    __syncthreads();
    if (KIND == 2) {
      // the column is complete: its rows leave while the next tiles are computed (the stores are waited for at the
      // end of the next iteration, long after they are done), and the columns move up
      emit(P0, PAR);
      P0 = P1;
      P1 = P2;
      fetch_piece(P2);
      ti = 0;
    } else {
      ++ti;
    }
  };

  using AnyPar = std::integral_constant<int, -1>;
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;
  using K0 = std::integral_constant<int, 0>;
  using K1 = std::integral_constant<int, 1>;
  using K2 = std::integral_constant<int, 2>;
  // Per column: the tiles that have two successors in the same column (from an even position on in pairs, with
  // the buffers as immediate offsets), then its last tile but one and its last tile.  The forms follow each other
  // in sequence -- one loop that picks a form per iteration makes the register allocator spill hundreds of
  // registers.
  using Plain = std::true_type;
  using Any = std::false_type;
  while (P0.T > 0) {
    int n0 = P0.T - ti - 2;  // tiles with two successors in the column
    // those of them that need no mask for any wave and whose K copy is a whole tile: the plain form
    int np = P0.Sa / kKT - 2 - ti;
    if (p.causal) { const int um = (P0.tq0 + 1) / kKT - ti; np = um < np ? um : np; }
    np = np < n0 ? np : n0;
    if (np > 0 && par_rt == 1) { iter(AnyPar{}, K0{}, Any{}); --n0; --np; }
    if (np >= 2) {
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) ka[ks] -= kBufBytes;
      for (; np >= 2; np -= 2, n0 -= 2) {
        iter(Even{}, K0{}, Plain{});
        iter(Odd{}, K0{}, Plain{});
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) ka[ks] += kBufBytes;
    }
    for (; n0 > 0; --n0) iter(AnyPar{}, K0{}, Any{});
    if (P0.T - ti == 2) iter(AnyPar{}, K1{}, Any{});
    iter(AnyPar{}, K2{}, Any{});
  }
}

// host side -----------------------------------------------------------------------------------------------------

// The launch shape of the stream kernel for this descriptor, or grid = 0 when attn_fwd_kernel should run: the
// batch must give every team of resident workgroups a unit and every workgroup of a team a column.
bool prefill_stream_plan(const pdllm_attn_desc* d, int cus, int* grid, int* team) {
  *grid = 0;
  *team = 0;
  if (d->mask_mode != PDLLM_MASK_CAUSAL && d->mask_mode != PDLLM_MASK_FULL) return false;
  if (d->num_splits != 0 || d->tiles_per_workgroup != 0) return false;
  if (d->rows_per_group != 0 && d->rows_per_group != 128) return false;
  if (d->kn_stride != d->vn_stride) return false;
  const int64_t row_b = d->kn_stride * 2;
  if (d->n_tokens >= (1l << 24) || row_b >= (1l << 24) || d->n_tokens * row_b >= (1l << 32) - 4096) return false;
  // Q and the output are addressed with 32-bit byte offsets as well
  if (d->n_tokens * d->q_stride * 2 >= (1l << 32) - 8192 || d->n_tokens * d->o_stride * 2 >= (1l << 32) - 8192) return false;
  const int G = d->num_q_heads / d->num_kv_heads;
  const long R = ((long)d->max_q_len * G + 127) / 128;
  const long units = (long)d->n_req * d->num_kv_heads;
  if (d->num_kv_heads > 255 || R >= (1l << 22)) return false;
  const int slots = 2 * cus;
  for (int tw = 16; tw <= 64; tw *= 2) {
    const int teams = slots / tw;
    if (teams < 1 || units < teams || R < tw) continue;
    const long per_wg = ((units + teams - 1) / teams) * ((R + tw - 1) / tw) + 1;
    if (per_wg > kMaxPieces) return false;
    *grid = teams * tw;
    *team = tw;
    return true;
  }
  return false;
}

int launch_prefill_stream(const pdllm_attn_desc* d, int grid, int team, hipStream_t stream) {
  PrefillParams p = {};
  p.q = static_cast<const __bf16*>(d->q);
  p.k = static_cast<const __bf16*>(d->k_new);
  p.v = static_cast<const __bf16*>(d->v_new);
  p.out = static_cast<__bf16*>(d->out);
  p.q_start_loc = d->q_start_loc;
  p.q_stride = d->q_stride;
  p.o_stride = d->o_stride;
  p.kv_row_bytes = (unsigned)(d->kn_stride * 2);
  p.out_bytes = (unsigned)(((d->n_tokens - 1) * d->o_stride + (int64_t)d->num_q_heads * kD) * 2);
  p.n_tokens = d->n_tokens;
  p.n_req = d->n_req;
  p.Hq = d->num_q_heads;
  p.Hkv = d->num_kv_heads;
  p.G = d->num_q_heads / d->num_kv_heads;
  p.causal = d->mask_mode == PDLLM_MASK_CAUSAL;
  p.max_q_len = d->max_q_len;
  p.R = (int)(((long)d->max_q_len * p.G + 127) / 128);
  p.team = team;
  p.n_teams = grid / team;
  p.n_units = d->n_req * d->num_kv_heads;
  p.scale_log2 = d->sm_scale * 1.4426950408889634f;
  hipLaunchKernelGGL(attn_prefill_stream_kernel, dim3((unsigned)grid), dim3(256), 0, stream, p);
  return launch_status();
}

}  // namespace pdllm
