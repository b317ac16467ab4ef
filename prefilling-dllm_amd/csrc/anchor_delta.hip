// Anchor corrections of the attention output (experimental modes of the reference layer, default off).
//
// Every `stride`-th active row (the anchors) gets a second, denser attention result; the difference to the
// base result is added to the anchor's neighbours:
//   delta[a] = (dense[a] - base[a]) * scale                                  (plain)
//   delta[a] = (sel[a] - base[a]) * scale * valid[a]                         (selection replaces dense)
//   delta[a] = (dense[a] - base[a]) * scale + (sel[a] - dense[a]) * sel_scale * valid[a]   (selection added)
//   out[r]   = base[r] + sum over anchors a whose window holds r of delta[a]
// (attention_v4.py:139-166 decode, :263-293 prefill).  The reference does this with bf16 tensor operations,
// i.e. every subtraction, product and sum is rounded to bf16 and the anchors are added in ascending order; the
// kernel rounds at the same places, so equal inputs give equal bits.
#include "pdllm_common.h"

namespace pdllm {

struct AnchorParams {
  const __bf16* base;
  const __bf16* dense;
  const __bf16* sel;
  const int64_t* sel_counts;
  __bf16* out;
  const int* q_start_loc;
  long base_stride, dense_stride, sel_stride, out_stride, n_sel_rows, n_rows;
  int n_req, max_q_len, groups;  // groups = row_elems / 8
  int stride, offset, lo_reach, hi_reach;  // a row r takes anchors in [r - lo_reach, r + hi_reach]
  int sel_mode;                            // 0 none, 1 replace, 2 add
  float scale, sel_scale;
};

__device__ __forceinline__ float rbf(float x) { return (float)(__bf16)x; }

__global__ __launch_bounds__(256) void anchor_delta_add_kernel(const AnchorParams p) {
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  const long per_req = (long)p.max_q_len * p.groups;
  const int req = (int)(gid / per_req);
  if (req >= p.n_req) return;
  const long rem = gid - req * per_req;
  const int i = (int)(rem / p.groups);
  const int e = (int)(rem - (long)i * p.groups) * 8;
  const int q0 = p.q_start_loc[req];
  const int L = p.q_start_loc[req + 1] - q0;
  if (i >= L || q0 < 0 || (long)q0 + L > p.n_rows) return;  // a sequence outside the tensors is left alone
  const bf16x8 b = *reinterpret_cast<const bf16x8*>(p.base + (long)(q0 + i) * p.base_stride + e);
  float corr[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  int a_lo = i - p.lo_reach;
  a_lo = a_lo < p.offset ? p.offset : a_lo;
  // first anchor >= a_lo
  int a = p.offset + (a_lo - p.offset + p.stride - 1) / p.stride * p.stride;
  int a_hi = i + p.hi_reach;
  a_hi = a_hi < L - 1 ? a_hi : L - 1;
  for (; a <= a_hi; a += p.stride) {
    const bf16x8 ba = *reinterpret_cast<const bf16x8*>(p.base + (long)(q0 + a) * p.base_stride + e);
    bf16x8 da = ba, sa = ba;
    if (p.dense != nullptr) da = *reinterpret_cast<const bf16x8*>(p.dense + (long)(q0 + a) * p.dense_stride + e);
    float valid = 0.f;
    if (p.sel_mode != 0) {
      const bool in_range = a < p.n_sel_rows;
      if (in_range) {
        sa = *reinterpret_cast<const bf16x8*>(p.sel + (long)a * p.sel_stride + e);
        valid = (p.sel_counts == nullptr || p.sel_counts[a] > 0) ? 1.f : 0.f;
      } else {
#pragma unroll
        for (int x = 0; x < 8; ++x) sa[x] = (__bf16)0.f;  // rows past the selection read as zero and are not valid
      }
    }
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      const float bx = (float)ba[x], dx = (float)da[x], sx = (float)sa[x];
      float delta;
      if (p.sel_mode == 1) {
        delta = rbf(rbf(rbf(sx - bx) * p.scale) * valid);
      } else {
        delta = rbf(rbf(dx - bx) * p.scale);
        if (p.sel_mode == 2) delta = rbf(delta + rbf(rbf(rbf(sx - dx) * p.sel_scale) * valid));
      }
      corr[x] = rbf(corr[x] + delta);
    }
  }
  bf16x8 o;
#pragma unroll
  for (int x = 0; x < 8; ++x) o[x] = (__bf16)((float)b[x] + corr[x]);
  *reinterpret_cast<bf16x8*>(p.out + (long)(q0 + i) * p.out_stride + e) = o;
}

}  // namespace pdllm

using namespace pdllm;

extern "C" int pdllm_anchor_delta_add(const void* base, int64_t base_stride, const void* dense, int64_t dense_stride,
                                      const void* sel, int64_t sel_stride, int64_t n_sel_rows,
                                      const int64_t* sel_counts, void* out, int64_t out_stride,
                                      const int32_t* q_start_loc, int64_t n_req, int64_t max_q_len, int64_t n_rows,
                                      int64_t row_elems,
                                      int32_t stride, int32_t anchor_offset, int32_t left, int32_t right,
                                      int32_t direction, float scale, float sel_scale, int32_t sel_mode,
                                      pdllm_stream_t stream) {
  if (!base || !out || !q_start_loc) return PDLLM_ERR_NULL;
  if (sel_mode < PDLLM_ANCHOR_SEL_NONE || sel_mode > PDLLM_ANCHOR_SEL_ADD) return PDLLM_ERR_DTYPE;
  if (direction < PDLLM_ANCHOR_LEFT || direction > PDLLM_ANCHOR_BOTH) return PDLLM_ERR_DTYPE;
  if (sel_mode != PDLLM_ANCHOR_SEL_REPLACE && !dense) return PDLLM_ERR_NULL;
  if (sel_mode != PDLLM_ANCHOR_SEL_NONE && (!sel || n_sel_rows < 0)) return PDLLM_ERR_NULL;
  if (n_req < 0 || max_q_len < 0 || n_rows < 0 || row_elems <= 0 || row_elems % 8 || stride <= 0 || anchor_offset < 0 ||
      anchor_offset >= stride || left < 0 || right < 0)
    return PDLLM_ERR_SHAPE;
  if (sel_mode != PDLLM_ANCHOR_SEL_NONE && n_req > 1) return PDLLM_ERR_UNSUPPORTED;  // selection rows are per sequence
  if (base_stride < row_elems || out_stride < row_elems || (dense && dense_stride < row_elems) ||
      (sel && sel_stride < row_elems) || base_stride % 8 || out_stride % 8 || (dense && dense_stride % 8) ||
      (sel && sel_stride % 8) || ((uintptr_t)base % 16) || ((uintptr_t)out % 16) || ((uintptr_t)dense % 16) ||
      ((uintptr_t)sel % 16))
    return PDLLM_ERR_STRIDE;
  if (out == base || out == dense) return PDLLM_ERR_STRIDE;  // anchors are read after their own row is written
  if (n_req == 0 || max_q_len == 0) return PDLLM_OK;
  const int64_t threads = n_req * max_q_len * (row_elems / 8);
  if (threads >= (1ll << 31) * 256 || max_q_len >= (1ll << 31) || n_req >= (1ll << 31)) return PDLLM_ERR_SHAPE;
  AnchorParams p;
  p.base = static_cast<const __bf16*>(base);
  p.dense = static_cast<const __bf16*>(dense);
  p.sel = sel_mode != PDLLM_ANCHOR_SEL_NONE ? static_cast<const __bf16*>(sel) : nullptr;
  p.sel_counts = sel_mode != PDLLM_ANCHOR_SEL_NONE ? sel_counts : nullptr;
  p.out = static_cast<__bf16*>(out);
  p.q_start_loc = q_start_loc;
  p.base_stride = base_stride; p.dense_stride = dense_stride; p.sel_stride = sel_stride; p.out_stride = out_stride;
  p.n_sel_rows = n_sel_rows;
  p.n_rows = n_rows;
  p.n_req = (int)n_req; p.max_q_len = (int)max_q_len; p.groups = (int)(row_elems / 8);
  p.stride = stride; p.offset = anchor_offset;
  // window of anchor a: left [a - left, a], right [a, a + right], both [a - left, a + right]
  p.hi_reach = direction == PDLLM_ANCHOR_RIGHT ? 0 : left;   // anchors above the row reach down to it
  p.lo_reach = direction == PDLLM_ANCHOR_LEFT ? 0 : right;   // anchors below the row reach up to it
  p.sel_mode = sel_mode;
  p.scale = scale; p.sel_scale = sel_scale;
  hipLaunchKernelGGL(anchor_delta_add_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), p);
  return launch_status();
}
