// Throughput of fire-and-forget fp32 atomic adds (global_atomic_add_f32) laid out the way a fused
// backward pass would add per-tile partial sums of dQ: 64 (batch, head) slices x 16 work groups; per
// iteration each of a group's 8 waves adds a 32 x 32 piece of a 64-row x 128-feature fp32 tile to
// dq[slice][rows][features], two 128-byte row segments per instruction.  Slices are assigned so that
// one slice is only touched from one XCD (work groups go round-robin over the 8 XCDs).  The same
// addresses are then written with plain stores for comparison.  64 iterations are 2.15 GB of fp32
// payload, what the dQ partial sums of B2 H32 N4096 D128 causal with 128-key blocks come to.
// Build: hipcc --offload-arch=gfx950 -O2 -munsafe-fp-atomics -o bin/atomic_add atomic_add.hip
#include <hip/hip_runtime.h>
#include <stdio.h>

#define CHECK(x)                                                                          \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                      \
      return 1;                                                                           \
    }                                                                                     \
  } while (0)

constexpr int kSlices = 64, kRows = 4096, kFeatures = 128, kGroups = 1024;

template <bool ATOMIC>
__global__ void __launch_bounds__(512) add_tiles(float* dq, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i = lane & 31, hh = lane >> 5;
  const int b = blockIdx.x;
  const int slice = (b & 7) + 8 * ((b >> 3) & 7);  // < kSlices; b & 7 is the XCD
  const int first_tile = (b >> 6) * 4;             // the 16 groups of a slice start at different tiles
  const int qb = wave >> 2, db = wave & 3;
  float* base = dq + (long)slice * kRows * kFeatures;
  for (int it = 0; it < iters; ++it) {
    const int tile = (first_tile + it) % (kRows / 64);
    float* p = base + (long)(tile * 64 + qb * 32) * kFeatures + db * 32 + i;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 8 * (r >> 2) + 4 * hh + (r & 3);  // MFMA 32x32 accumulator layout: < 32
      if (ATOMIC) __builtin_amdgcn_global_atomic_fadd_f32((__attribute__((address_space(1))) float*)(p + row * kFeatures), 1.0f);
      else p[row * kFeatures] = 1.0f;
    }
  }
}

int main() {
  float* dq;
  const size_t bytes = (size_t)kSlices * kRows * kFeatures * sizeof(float);
  CHECK(hipMalloc(&dq, bytes));
  CHECK(hipMemset(dq, 0, bytes));
  for (int atomic = 1; atomic >= 0; --atomic)
    for (int iters : {64, 256}) {
      hipEvent_t e0, e1;
      CHECK(hipEventCreate(&e0));
      CHECK(hipEventCreate(&e1));
      auto launch = [&]() {
        if (atomic) add_tiles<true><<<kGroups, 512>>>(dq, iters);
        else add_tiles<false><<<kGroups, 512>>>(dq, iters);
      };
      launch();
      CHECK(hipEventRecord(e0));
      launch();
      CHECK(hipEventRecord(e1));
      CHECK(hipDeviceSynchronize());
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      const double payload = (double)kGroups * iters * 64 * kFeatures * sizeof(float);
      printf("%-12s %3d iterations: %7.3f ms for %.2f GB of fp32 payload = %.2f TB/s\n", atomic ? "atomic add" : "plain store", iters,
             ms, payload / 1e9, payload / ms / 1e9);
    }
  CHECK(hipFree(dq));
  return 0;
}
