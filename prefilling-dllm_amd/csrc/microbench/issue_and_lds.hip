// Microbenchmark of the two hardware facts the attention kernels are built around (gfx950, run on one MI355X):
//
//  1. what a wavefront can issue in the shadow of an MFMA: straight-line mixes of v_mfma_f32_32x32x16_bf16 with
//     the softmax arithmetic (fma, exp, cvt_pk, dot2) and the LDS operand reads of the attention loop, timed per
//     wavefront with s_memtime, for one and for two wavefronts per SIMD (256 / 512 threads per workgroup, one
//     workgroup per compute unit);
//  2. the LDS read rate of the operand fragments: 128-bit K reads and transposing 64-bit V reads with the address
//     pattern of the kernels under the row swizzle of attn_common.h, next to linear addresses and next to the
//     swizzle that merely rotates the row bits (its V reads take two passes).
//
// Build:  make -C prefilling-dllm_amd/csrc microbench      Run:  prefilling-dllm_amd/csrc/build/issue_and_lds
// Output: one line per case: average ticks of the measured block per wavefront, and per compute unit the span from
// the first wavefront's start to the last one's end (with two wavefronts per SIMD they do not start together, so
// the span, not the per-wave time, says what a SIMD gets through).  s_memtime counts shader clocks.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <vector>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

#define CLOB_ACC                                                                                                       \
  "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v113",      \
      "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127",  \
      "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141",  \
      "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", "v152", "v153", "v154", "v155",  \
      "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163"
#define CLOB_TMP                                                                                                       \
  "v60", "v61", "v62", "v63", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75",      \
      "v76", "v77", "v78", "v79", "v80", "v81", "v82", "v83"

// four independent accumulators; %0 / %1 = A / B fragments, %2 = a float, %3 / %4 = LDS addresses
#define M0 "v_mfma_f32_32x32x16_bf16 v[100:115], %0, %1, v[100:115]\n"
#define M1 "v_mfma_f32_32x32x16_bf16 v[116:131], %0, %1, v[116:131]\n"
#define M2 "v_mfma_f32_32x32x16_bf16 v[132:147], %0, %1, v[132:147]\n"
#define M3 "v_mfma_f32_32x32x16_bf16 v[148:163], %0, %1, v[148:163]\n"
#define E(a) "v_exp_f32 v" #a ", v" #a "\n"
#define F(a) "v_fma_f32 v" #a ", v" #a ", %2, %2\n"
#define CV(a, b, c) "v_cvt_pk_bf16_f32 v" #a ", v" #b ", v" #c "\n"
#define D2(a, b) "v_dot2c_f32_bf16 v" #a ", %2, v" #b "\n"
#define NOP "s_nop 0\n"
#define WT(n) "s_waitcnt lgkmcnt(" #n ")\n"
#define RDK "ds_read_b128 v[76:79], %3\n"
#define RDV "ds_read_b64_tr_b16 v[80:81], %3\n ds_read_b64_tr_b16 v[82:83], %3 offset:512\n"
#define RK(o) "ds_read_b128 v[76:79], %3 offset:" #o "\n"
#define RV(o) "ds_read_b64_tr_b16 v[80:81], %4 offset:" #o "\n"
// two row blocks per wave: one K (or V) fragment feeds two MFMAs
#define SLOT2K WT(5) M0 F(60) E(60) CV(66, 64, 65) D2(67, 66) M1 F(61) E(61) RDK
#define SLOT2V WT(4) M2 F(64) E(64) CV(62, 60, 61) D2(63, 62) M3 F(65) E(65) RDV
// one row block per wave: every MFMA has its own fragment
#define SLOT1K(M, x) WT(5) M F(x) E(x) CV(66, 64, 65) D2(67, 66) RDK
#define SLOT1V(M, x) WT(4) M F(x) E(x) RDV
#define R8(x) x x x x x x x x

enum Mode { kExp, kFma, kNop, kMfma, kMfmaExp, kMfmaFmaExp, kMfma4, kMfma7, kMfma11, kTwoBlocks, kOneBlock,
            kKLinear, kKPattern, kVLinear, kVPattern, kVRotated };

template <int MODE>
__global__ __launch_bounds__(512, 1) void bench_kernel(unsigned long long* out, float seed) {
  __shared__ char pad[100 * 1024];  // one workgroup per compute unit
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + i); b[i] = (__bf16)(seed * 2 + i); }
  const float c = seed;
  const int lane = threadIdx.x & 63, l32 = lane & 31, hh = lane >> 5, wave = threadIdx.x >> 6;
  // the row swizzle of the kernels, and the one that only rotates the low four row bits
  auto swz = [](int row) { const int r = row & 15; return ((r & 3) << 2) | (((r >> 2) & 1) << 1) | (r >> 3); };
  auto rot = [](int row) { const int r = row & 15; return ((r & 7) << 1) | (r >> 3); };
  const unsigned lbase = (unsigned)(size_t)pad;
  const unsigned lin16 = lbase + lane * 16 + wave * 2048, lin8 = lbase + lane * 8;
  const unsigned kfrag = lbase + l32 * 256 + (((2 * 3 + hh) ^ swz(l32)) << 4);  // K fragment 3 of a tile
  const int i16 = lane & 15, g4 = l32 >> 4, keyrow = 4 * hh + (i16 >> 2), cg = 4 * 1 + 2 * g4 + ((i16 & 3) >> 1);
  const unsigned vfrag = lbase + 49152 + keyrow * 256 + ((cg ^ swz(keyrow)) << 4) + ((i16 & 1) << 3);
  const unsigned vrot = lbase + 49152 + keyrow * 256 + ((cg ^ rot(keyrow)) << 4) + ((i16 & 1) << 3);
  if (seed == 12345.f) pad[threadIdx.x] = 1;
  unsigned long long t0 = 0, t1 = 0;
  for (int rep = 0; rep < 3; ++rep) {  // the last repetition is reported
    __syncthreads();
    t0 = __builtin_amdgcn_s_memtime();
#define ARGS : : "v"(a), "v"(b), "v"(c), "v"(lin16), "v"(vfrag) : CLOB_ACC, CLOB_TMP
    if constexpr (MODE == kExp) asm volatile(R8(E(60) E(61) E(62) E(63) E(64) E(65) E(66) E(67)) ARGS);
    else if constexpr (MODE == kFma) asm volatile(R8(F(60) F(61) F(62) F(63) F(64) F(65) F(66) F(67)) ARGS);
    else if constexpr (MODE == kNop) asm volatile(R8(NOP NOP NOP NOP NOP NOP NOP NOP) ARGS);
    else if constexpr (MODE == kMfma) asm volatile(R8(M0 M1 M2 M3) ARGS);
    else if constexpr (MODE == kMfmaExp) asm volatile(R8(M0 E(60) M1 E(61) M2 E(62) M3 E(63)) ARGS);
    else if constexpr (MODE == kMfmaFmaExp) asm volatile(R8(M0 F(60) E(60) M1 F(61) E(61) M2 F(62) E(62) M3 F(63) E(63)) ARGS);
    else if constexpr (MODE == kMfma4)
      asm volatile(R8(M0 F(60) F(61) F(62) F(63) M1 F(64) F(65) F(66) F(67) M2 F(68) F(69) F(70) F(71) M3 F(72) F(73) F(74) F(75)) ARGS);
    else if constexpr (MODE == kMfma7)
      asm volatile(R8(M0 F(60) F(61) F(62) F(63) F(64) F(65) F(66) M1 F(64) F(65) F(66) F(67) F(68) F(69) F(70)
                      M2 F(68) F(69) F(70) F(71) F(72) F(73) F(74) M3 F(72) F(73) F(74) F(75) F(60) F(61) F(62)) ARGS);
    else if constexpr (MODE == kMfma11)
      asm volatile(R8(M0 F(60) F(61) F(62) F(63) F(64) F(65) F(66) F(67) F(68) F(69) F(70)
                      M1 F(64) F(65) F(66) F(67) F(68) F(69) F(70) F(71) F(72) F(73) F(74)
                      M2 F(68) F(69) F(70) F(71) F(72) F(73) F(74) F(75) F(60) F(61) F(62)
                      M3 F(72) F(73) F(74) F(75) F(60) F(61) F(62) F(63) F(64) F(65) F(66)) ARGS);
    else if constexpr (MODE == kTwoBlocks) asm volatile(R8(SLOT2K SLOT2V) ARGS);
    else if constexpr (MODE == kOneBlock) asm volatile(R8(SLOT1K(M0, 60) SLOT1V(M1, 61) SLOT1K(M0, 62) SLOT1V(M2, 63)) ARGS);
#undef ARGS
#define LARGS(k, v) : : "v"(a), "v"(b), "v"(c), "v"(k), "v"(v) : "v76", "v77", "v78", "v79", "v80", "v81"
    else if constexpr (MODE == kKLinear)
      asm volatile(R8(RK(0) RK(0) RK(0) RK(0) RK(0) RK(0) RK(0) RK(0)) WT(0) LARGS(lin16, vfrag));
    else if constexpr (MODE == kKPattern)
      asm volatile(R8(RK(0) RK(8192) RK(0) RK(8192) RK(0) RK(8192) RK(0) RK(8192)) WT(0) LARGS(kfrag, vfrag));
#define V16 RV(0) RV(4096) RV(8192) RV(12288) RV(0) RV(4096) RV(8192) RV(12288) RV(0) RV(4096) RV(8192) RV(12288) RV(0) RV(4096) RV(8192) RV(12288)
    else if constexpr (MODE == kVLinear) asm volatile(R8(V16) WT(0) LARGS(kfrag, lin8));
    else if constexpr (MODE == kVPattern) asm volatile(R8(V16) WT(0) LARGS(kfrag, vfrag));
    else if constexpr (MODE == kVRotated) asm volatile(R8(V16) WT(0) LARGS(kfrag, vrot));
#undef V16
#undef LARGS
    t1 = __builtin_amdgcn_s_memtime();
  }
  if (lane == 0) {
    out[(blockIdx.x * 8 + wave) * 2] = t0;
    out[(blockIdx.x * 8 + wave) * 2 + 1] = t1;
  }
}

#define CHECK(x)                                                                       \
  do {                                                                                 \
    const hipError_t e_ = (x);                                                         \
    if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 1; } \
  } while (0)

template <int MODE>
int run(const char* what, int threads) {
  constexpr int grid = 256;
  unsigned long long* d = nullptr;
  CHECK(hipMalloc(&d, grid * 16 * sizeof(unsigned long long)));
  CHECK(hipMemset(d, 0, grid * 16 * sizeof(unsigned long long)));
  for (int i = 0; i < 2; ++i) {
    hipLaunchKernelGGL(bench_kernel<MODE>, dim3(grid), dim3(threads), 0, 0, d, 1.0f);
    CHECK(hipDeviceSynchronize());
  }
  std::vector<unsigned long long> h(grid * 16);
  CHECK(hipMemcpy(h.data(), d, h.size() * 8, hipMemcpyDeviceToHost));
  double s = 0, span = 0;
  int n = 0;
  for (int b = 0; b < grid; ++b) {
    unsigned long long first = ~0ull, last = 0;
    for (int wv = 0; wv < threads / 64; ++wv) {
      const unsigned long long t0 = h[(b * 8 + wv) * 2], t1 = h[(b * 8 + wv) * 2 + 1];
      s += (double)(t1 - t0);
      first = t0 < first ? t0 : first;
      last = t1 > last ? t1 : last;
      ++n;
    }
    span += (double)(last - first);
  }
  printf("%-58s %d waves/SIMD: %8.1f ticks per wave, %8.1f per compute unit\n", what, threads / 256, s / n, span / grid);
  CHECK(hipFree(d));
  return 0;
}

int main() {
  for (int threads : {256, 512}) {
    if (run<kExp>("64 v_exp_f32", threads)) return 1;
    if (run<kFma>("64 v_fma_f32", threads)) return 1;
    if (run<kNop>("64 s_nop 0", threads)) return 1;
    if (run<kMfma>("32 mfma", threads)) return 1;
    if (run<kMfmaExp>("32 x (mfma, exp)", threads)) return 1;
    if (run<kMfmaFmaExp>("32 x (mfma, fma, exp)", threads)) return 1;
    if (run<kMfma4>("32 x (mfma, 4 fma)", threads)) return 1;
    if (run<kMfma7>("32 x (mfma, 7 fma)", threads)) return 1;
    if (run<kMfma11>("32 x (mfma, 11 fma)", threads)) return 1;
    if (run<kTwoBlocks>("32 mfma, softmax of 32 scores, 8 K + 8 V fragments", threads)) return 1;
    if (run<kOneBlock>("32 mfma, softmax of 32 scores, 16 K + 16 V fragments", threads)) return 1;
    if (run<kKLinear>("64 ds_read_b128, linear addresses", threads)) return 1;
    if (run<kKPattern>("64 ds_read_b128, K fragment addresses", threads)) return 1;
    if (run<kVLinear>("128 ds_read_b64_tr_b16, linear addresses", threads)) return 1;
    if (run<kVPattern>("128 ds_read_b64_tr_b16, V fragment addresses", threads)) return 1;
    if (run<kVRotated>("128 ds_read_b64_tr_b16, V fragments, rotated-bits swizzle", threads)) return 1;
  }
  return 0;
}
