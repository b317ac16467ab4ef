// Shared device/host helpers for the gfx950 kernels of the Prefilling-dLLM hot path.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pdllm.h"

namespace pdllm {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int kWave = 64;
constexpr int kNumXcd = 8;  // MI355X: 8 XCDs, workgroups are dealt to them round-robin

// Map the hardware workgroup id to a logical id such that consecutive logical ids
// land on the same XCD (and therefore share its L2).  Bijective for any grid size.
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
  const int xcd = bid % kNumXcd;
  const int idx = bid / kNumXcd;
  const int per = nblocks / kNumXcd;
  const int rem = nblocks % kNumXcd;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  return (uint32_t) __builtin_bit_cast(unsigned short, b);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 p = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? PDLLM_OK : PDLLM_ERR_LAUNCH;
}

}  // namespace pdllm
