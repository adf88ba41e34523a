// Instruction issue and MFMA rates of a gfx950 CU, measured with one or two waves per SIMD.
//
// The attention kernels in ../csrc interleave MFMAs with VALU, LDS and scalar instructions; how
// many of those fit beside an MFMA decides what a schedule can reach.  Every pattern below is a
// straight-line run of instructions (inline asm, .rept) executed 3000 times by every wave of a
// launch that puts exactly one work group on each of the 256 CUs (100 KiB of LDS per group); a
// group has 4 waves (one per SIMD) or 8 (two per SIMD).  Reported per "unit" of the pattern:
//   ticks per unit and wave   (s_memtime around the loop, averaged over the waves)
//   ns per unit and SIMD      (kernel duration by HIP events / units executed per SIMD)
//   ticks per ns              (the clock the counter ran at: it drops under heavy load)
// Build: hipcc --offload-arch=gfx950 -O2 -o bin/issue_rate issue_rate.hip   (setup.py build_microbench)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <vector>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f2v __attribute__((ext_vector_type(2)));

#define CHECK(x)                                                                          \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                      \
      return 1;                                                                           \
    }                                                                                     \
  } while (0)

#define REP(n, body) ".rept " #n "\n\t" body "\n\t.endr\n\t"
// four MFMAs on four accumulators in accumulation registers, two on two in vector registers
#define MF0 "v_mfma_f32_32x32x16_f16 %0, %[x], %[y], %0\n\t"
#define MF1 "v_mfma_f32_32x32x16_f16 %1, %[x], %[y], %1\n\t"
#define MF2 "v_mfma_f32_32x32x16_f16 %2, %[x], %[y], %2\n\t"
#define MF3 "v_mfma_f32_32x32x16_f16 %3, %[x], %[y], %3\n\t"
#define MV0 "v_mfma_f32_32x32x16_f16 %4, %[x], %[y], %4\n\t"
#define MV1 "v_mfma_f32_32x32x16_f16 %5, %[x], %[y], %5\n\t"
#define FMA2 "v_fma_f32 %6, %6, %6, %6\n\tv_fma_f32 %7, %7, %7, %7\n\t"
#define FMA4 FMA2 "v_fma_f32 %8, %8, %8, %8\n\tv_fma_f32 %9, %9, %9, %9\n\t"
#define EXP1 "v_exp_f32 %8, %8\n\t"
#define EXP2 "v_exp_f32 %6, %6\n\tv_exp_f32 %7, %7\n\t"
#define NOP2 "s_nop 0\n\ts_nop 0\n\t"
#define TR2 "ds_read_b64_tr_b16 %[d2], %[lds]\n\tds_read_b64_tr_b16 %[d2], %[lds] offset:1024\n\t"
#define B128 "ds_read_b128 %[d4], %[lds]\n\t"
#define EACH4(tail) MF0 tail MF1 tail MF2 tail MF3 tail

template <int P>
__device__ __forceinline__ void pattern(f16v& a0, f16v& a1, f16v& a2, f16v& a3, f16v& c0, f16v& c1, const h8& x, const h8& y,
                                        float& f0, float& f1, float& f2, float& f3, unsigned lds_addr) {
  f4v d4 = {};
  f2v d2 = {};
#define OPS                                                                                                        \
  : "+a"(a0), "+a"(a1), "+a"(a2), "+a"(a3), "+v"(c0), "+v"(c1), "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3),           \
    [d4] "+v"(d4), [d2] "+v"(d2)                                                                                   \
  : [x] "v"(x), [y] "v"(y), [lds] "v"(lds_addr)
  if constexpr (P == 0) asm volatile(REP(16, FMA4) OPS);
  if constexpr (P == 1) asm volatile(REP(64, "v_fma_f32 %6, %6, %6, %6") OPS);
  if constexpr (P == 2) asm volatile(REP(16, EXP2 EXP2) OPS);
  if constexpr (P == 3) asm volatile(REP(64, "s_nop 0") OPS);
  if constexpr (P == 4) asm volatile(REP(64, "s_mov_b32 s20, 0") OPS : "s20");
  if constexpr (P == 5) asm volatile(REP(32, B128) "s_waitcnt lgkmcnt(0)\n\t" OPS);
  if constexpr (P == 6) asm volatile(REP(4, MF0 MF1 MF2 MF3) OPS);
  if constexpr (P == 7) asm volatile(REP(8, MV0 MV1) OPS);
  if constexpr (P == 8) asm volatile(REP(4, EACH4(FMA4)) OPS);
  if constexpr (P == 9) asm volatile(REP(4, EACH4(FMA4 FMA2)) OPS);
  if constexpr (P == 10) asm volatile(REP(4, EACH4(FMA4 FMA4)) OPS);
  if constexpr (P == 11) asm volatile(REP(4, EACH4(FMA2 EXP2)) OPS);
  if constexpr (P == 12) asm volatile(REP(4, EACH4(FMA4 NOP2)) OPS);
  if constexpr (P == 13) asm volatile(REP(4, MF0 FMA4 TR2 MF1 FMA4 B128 "s_nop 0\n\t" MF2 FMA4 TR2 MF3 FMA4 B128 "s_nop 0\n\t")
                                      "s_waitcnt lgkmcnt(0)\n\t" OPS);
#undef OPS
}

template <int P>
__global__ void __launch_bounds__(512) bench(long* out, int iters) {
  __shared__ char lds[100 * 1024];  // one work group per CU
  f16v a0 = {}, a1 = {}, a2 = {}, a3 = {}, c0 = {}, c1 = {};
  h8 x, y;
  for (int e = 0; e < 8; ++e) {
    x[e] = (_Float16)0.001f;
    y[e] = (_Float16)0.002f;
  }
  float f0 = 0.1f, f1 = 0.2f, f2 = 0.3f, f3 = 0.4f;
  const unsigned lds_addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds + (threadIdx.x & 63) * 16;
  pattern<P>(a0, a1, a2, a3, c0, c1, x, y, f0, f1, f2, f3, lds_addr);  // warm the instruction cache
  __syncthreads();
  const long t0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) pattern<P>(a0, a1, a2, a3, c0, c1, x, y, f0, f1, f2, f3, lds_addr);
  const long t1 = __builtin_readcyclecounter();
  const float sink = f0 + f1 + f2 + f3 + a0[0] + a1[0] + a2[0] + a3[0] + c0[0] + c1[0];
  if (sink == 12345.f) out[1 << 20] = 1;  // keeps the results alive; never true
  if ((threadIdx.x & 63) == 0) out[blockIdx.x * 8 + (threadIdx.x >> 6)] = t1 - t0;
}

template <int P>
int run(const char* name, int units, long* d_out) {
  const int iters = 3000, groups = 256;
  for (int threads : {256, 512}) {
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    bench<P><<<groups, threads>>>(d_out, iters);
    CHECK(hipEventRecord(e0));
    bench<P><<<groups, threads>>>(d_out, iters);
    CHECK(hipEventRecord(e1));
    CHECK(hipDeviceSynchronize());
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    std::vector<long> h(groups * 8);
    CHECK(hipMemcpy(h.data(), d_out, h.size() * sizeof(long), hipMemcpyDeviceToHost));
    double sum = 0;
    const int waves = threads / 64;
    for (int b = 0; b < groups; ++b)
      for (int w = 0; w < waves; ++w) sum += h[b * 8 + w];
    const double ticks = sum / (groups * waves) / iters;
    printf("%-40s waves/SIMD %d: %7.2f ticks per unit and wave | %6.2f ns per unit and SIMD | %.2f ticks/ns\n", name,
           threads / 256, ticks / units, ms * 1e6 / iters / units / (threads / 256), ticks * iters / (ms * 1e6));
    fflush(stdout);
  }
  return 0;
}

int main() {
  long* d_out;
  CHECK(hipMalloc(&d_out, ((1 << 20) + 1) * sizeof(long)));
  int rc = 0;
  rc |= run<0>("v_fma_f32, independent", 64, d_out);
  rc |= run<1>("v_fma_f32, dependent chain", 64, d_out);
  rc |= run<2>("v_exp_f32", 64, d_out);
  rc |= run<3>("s_nop 0", 64, d_out);
  rc |= run<4>("s_mov_b32", 64, d_out);
  rc |= run<5>("ds_read_b128 (1 KiB per wave)", 32, d_out);
  rc |= run<6>("mfma 32x32x16 f16, acc in AGPRs", 16, d_out);
  rc |= run<7>("mfma 32x32x16 f16, acc in VGPRs", 16, d_out);
  rc |= run<8>("mfma + 4 v_fma", 16, d_out);
  rc |= run<9>("mfma + 6 v_fma", 16, d_out);
  rc |= run<10>("mfma + 8 v_fma", 16, d_out);
  rc |= run<11>("mfma + 2 v_fma + 2 v_exp", 16, d_out);
  rc |= run<12>("mfma + 4 v_fma + 2 s_nop", 16, d_out);
  rc |= run<13>("mfma + 4 v_fma + 1 KiB of LDS reads", 16, d_out);
  CHECK(hipFree(d_out));
  return rc;
}
