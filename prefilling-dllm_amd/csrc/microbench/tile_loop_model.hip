// Microbenchmark: a hand-written model of one iteration of the attention tile loop (gfx950, run on one MI355X).
//
// Two workgroups of four wavefronts per compute unit (64 KB of LDS each), as the default attention kernel runs.  One
// iteration is what a wavefront does for a 32 x 64 tile: 16 QK steps (wait, MFMA, two multiply-adds, two exponentials,
// a pack, a dot into the row sum, one 128-bit K read) and 16 PV steps (wait, MFMA, two transposing 64-bit V reads),
// the LDS addresses following the kernel's swizzle.  Features are switched on one at a time to see what each costs:
//   1 = barrier per tile, 2 = the 8 direct-to-LDS copies per wave and tile with a vmcnt(0) wait before the barrier,
//   4 = 32 more vector instructions (moves / address updates), 8 = 16 more scalar instructions,
//   16 = one v_max3 per PV step (row maximum of the next tile), 32 = the copies read the same 32 KB every time (L2 hits)
//       instead of streaming 32 KB per workgroup and tile from HBM.
// The model never waits for LDS data (every wait finds its counter satisfied), so it is a floor for the instruction
// mix, not a prediction.
//
// Build:  make -C prefilling-dllm_amd/csrc microbench      Run:  prefilling-dllm_amd/csrc/build/tile_loop_model
// Output: one line per case: shader clocks (s_memtime) per tile and wavefront -- with two wavefronts per SIMD that is
// the time of a pair of tiles on one SIMD -- and the span of the launch in us.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
#define CLOB "v100","v101","v102","v103","v104","v105","v106","v107","v108","v109","v110","v111","v112","v113","v114","v115", \
 "v116","v117","v118","v119","v120","v121","v122","v123","v124","v125","v126","v127","v128","v129","v130","v131", \
 "v132","v133","v134","v135","v136","v137","v138","v139","v140","v141","v142","v143","v144","v145","v146","v147", \
 "v148","v149","v150","v151","v152","v153","v154","v155","v156","v157","v158","v159","v160","v161","v162","v163", \
 "v164","v165","v166","v167","v168","v169","v170","v171","v172","v173","v174","v175","v176","v177","v178","v179", \
 "v60","v61","v62","v63","v64","v65","v66","v67","v68","v69","v70","v71","v72","v73","v74","v75","v76","v77","v78","v79","v80","v81","v82","v83","v84","v85","v86","v87","v88","v89","v90","v91"
// QK: one dependent chain of 8 per key block into v[164:179]; PV: four accumulators
#define MQ "v_mfma_f32_32x32x16_bf16 v[164:179], v[76:79], %1, v[164:179]\n"
#define MP(n) "v_mfma_f32_32x32x16_bf16 v[" #n "], v[80:83], %1, v[" #n "]\n"
#define STEPA(x, y) "s_waitcnt lgkmcnt(1)\n" MQ "v_fma_f32 v" #x ", v" #x ", %2, %2\n v_fma_f32 v" #y ", v" #y ", %2, %2\n v_exp_f32 v" #x ", v" #x "\n v_exp_f32 v" #y ", v" #y "\n v_cvt_pk_bf16_f32 v66, v" #x ", v" #y "\n v_dot2c_f32_bf16 v67, %2, v66\n ds_read_b128 v[76:79], %3\n"
#define STEPB(n, o) "s_waitcnt lgkmcnt(2)\n" MP(n) "ds_read_b64_tr_b16 v[80:81], %4 offset:" #o "\n ds_read_b64_tr_b16 v[82:83], %4 offset:" #o "+512\n"
#define STEPBM(n, o) "s_waitcnt lgkmcnt(2)\n" MP(n) "ds_read_b64_tr_b16 v[80:81], %4 offset:" #o "\n ds_read_b64_tr_b16 v[82:83], %4 offset:" #o "+512\n v_max3_f32 v68, v68, v60, v61\n"
#define A16 STEPA(60,61) STEPA(62,63) STEPA(64,65) STEPA(60,61) STEPA(62,63) STEPA(64,65) STEPA(60,61) STEPA(62,63) STEPA(64,65) STEPA(60,61) STEPA(62,63) STEPA(64,65) STEPA(60,61) STEPA(62,63) STEPA(64,65) STEPA(60,61)
#define B16 STEPB(100:115,0) STEPB(116:131,1024) STEPB(132:147,2048) STEPB(148:163,3072) STEPB(100:115,4096) STEPB(116:131,5120) STEPB(132:147,6144) STEPB(148:163,7168) STEPB(100:115,0) STEPB(116:131,1024) STEPB(132:147,2048) STEPB(148:163,3072) STEPB(100:115,4096) STEPB(116:131,5120) STEPB(132:147,6144) STEPB(148:163,7168)
#define B16M STEPBM(100:115,0) STEPBM(116:131,1024) STEPBM(132:147,2048) STEPBM(148:163,3072) STEPBM(100:115,4096) STEPBM(116:131,5120) STEPBM(132:147,6144) STEPBM(148:163,7168) STEPBM(100:115,0) STEPBM(116:131,1024) STEPBM(132:147,2048) STEPBM(148:163,3072) STEPBM(100:115,4096) STEPBM(116:131,5120) STEPBM(132:147,6144) STEPBM(148:163,7168)
#define V8 "v_mov_b32 v84, v85\n v_mov_b32 v85, v86\n v_mov_b32 v86, v87\n v_mov_b32 v87, v88\n v_add_u32 v88, v89, v90\n v_add_u32 v89, v90, v91\n v_add_u32 v90, v91, v84\n v_add_u32 v91, v84, v85\n"
#define S8 "s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n"

template <int FEAT>
__global__ __launch_bounds__(256, 2) void k(unsigned long long* out, const char* src, int iters, float seed) {
  __shared__ __attribute__((aligned(1024))) char lds[65536];
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + i); b[i] = (__bf16)(seed * 2 + i); }
  const float c = seed;
  const int lane = threadIdx.x & 63, l32 = lane & 31, hh = lane >> 5, wave = threadIdx.x >> 6;
  auto swz = [](int row) { const int r = row & 15; return ((r & 3) << 2) | (((r >> 2) & 1) << 1) | (r >> 3); };
  const unsigned lbase = (unsigned)(size_t)lds;
  const unsigned kfrag = lbase + l32 * 256 + (((2 * 3 + hh) ^ swz(l32)) << 4);
  const int i16 = lane & 15, g4 = l32 >> 4, keyrow = 4 * hh + (i16 >> 2), cg = 4 * 1 + 2 * g4 + ((i16 & 3) >> 1);
  const unsigned vfrag = lbase + 16384 + keyrow * 256 + ((cg ^ swz(keyrow)) << 4) + ((i16 & 1) << 3);
  if (seed == 12345.f) lds[threadIdx.x] = 1;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(src), 0, 0xffffffff, 0x00020000);
  // every workgroup streams its own 32 KB per tile (or, FEAT & 32, always the same 32 KB)
  unsigned goff = (FEAT & 32) ? 0u : (unsigned)blockIdx.x * (unsigned)iters * 32768u;
  goff += wave * 1024 + lane * 16;
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  const unsigned long long w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    const int buf = (it & 1) * 32768;
    if constexpr (FEAT & 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(lds + buf + wave * 1024 + i * 4096), 16,
                                                 goff + i * 4096, 0, 0, 0);
      if (!(FEAT & 32)) goff += 32768;
    }
    asm volatile(A16 : : "v"(a), "v"(b), "v"(c), "v"(kfrag), "v"(vfrag) : CLOB);
    if constexpr (FEAT & 4) asm volatile(V8 V8 V8 V8 : : : CLOB);
    if constexpr (FEAT & 8) asm volatile(S8 S8 : : : CLOB);
    if constexpr (FEAT & 16) asm volatile(B16M : : "v"(a), "v"(b), "v"(c), "v"(kfrag), "v"(vfrag) : CLOB);
    else asm volatile(B16 : : "v"(a), "v"(b), "v"(c), "v"(kfrag), "v"(vfrag) : CLOB);
    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
    if constexpr (FEAT & 2) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    if constexpr (FEAT & 1) __builtin_amdgcn_s_barrier();
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  const unsigned long long w1 = wall_clock64();
  if (lane == 0) {
    out[(blockIdx.x * 4 + wave) * 4 + 0] = t0; out[(blockIdx.x * 4 + wave) * 4 + 1] = t1;
    out[(blockIdx.x * 4 + wave) * 4 + 2] = w0; out[(blockIdx.x * 4 + wave) * 4 + 3] = w1;
  }
}

#define CHECK(x)                                                                                    \
  do {                                                                                              \
    const hipError_t e_ = (x);                                                                      \
    if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); exit(1); }      \
  } while (0)

template <int FEAT>
void run(const char* what, const char* src, int iters) {
  const int grid = 512;
  unsigned long long* d; CHECK(hipMalloc(&d, grid * 16 * 8));
  for (int rep = 0; rep < 3; ++rep) { hipLaunchKernelGGL(k<FEAT>, dim3(grid), dim3(256), 0, 0, d, src, iters, 1.0f); CHECK(hipDeviceSynchronize()); }
  std::vector<unsigned long long> h(grid * 16);
  CHECK(hipMemcpy(h.data(), d, grid * 16 * 8, hipMemcpyDeviceToHost));
  double clk = 0, first = 1e30, last = 0; int n = 0;
  for (int b = 0; b < grid; ++b) for (int w = 0; w < 4; ++w) {
    clk += (double)(h[(b * 4 + w) * 4 + 1] - h[(b * 4 + w) * 4 + 0]); ++n;
    first = std::min(first, (double)h[(b * 4 + w) * 4 + 2]); last = std::max(last, (double)h[(b * 4 + w) * 4 + 3]);
  }
  printf("%-70s %7.0f clk per tile and wave (2 waves/SIMD), launch span %.1f us = %.3f us per tile pair\n", what, clk / n / iters, (last - first) / 100.0, (last - first) / 100.0 / iters);
  CHECK(hipFree(d));
}

int main() {
  const int iters = 40;
  char* src;
  CHECK(hipMalloc(&src, (size_t)512 * iters * 32768 + 65536));
  CHECK(hipMemset(src, 0, (size_t)512 * iters * 32768 + 65536));
  run<0>("steps only", src, iters);
  run<16>("+ max3 in PV", src, iters);
  run<16 | 1>("+ max3 + barrier", src, iters);
  run<16 | 2>("+ max3 + copies (HBM stream)", src, iters);
  run<16 | 2 | 32>("+ max3 + copies (L2-resident source)", src, iters);
  run<16 | 1 | 2>("+ max3 + barrier + copies", src, iters);
  run<16 | 1 | 2 | 4>("+ max3 + barrier + copies + 32 VALU", src, iters);
  run<16 | 1 | 2 | 4 | 8>("+ max3 + barrier + copies + 32 VALU + 16 scalar", src, iters);
  run<16 | 4>("+ max3 + 32 VALU", src, iters);
  run<16 | 8>("+ max3 + 16 scalar", src, iters);
  return 0;
}
