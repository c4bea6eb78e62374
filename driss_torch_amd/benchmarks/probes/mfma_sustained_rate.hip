// What the scaled MFMA sustains on a whole MI355X with nothing else going on: one wave per SIMD
// streams independent v_mfma_scale_f32_* instructions out of registers (no LDS, no memory) for
// about a millisecond per launch, launches back to back until the clocks have settled.  Operands
// are constant or pseudo-random bytes; with NOPER > 1 consecutive MFMAs see different registers.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 driss_torch_amd/benchmarks/probes/mfma_sustained_rate.hip -o mfma_sustained_rate
//   ./mfma_sustained_rate
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ uint32_t hash32(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// SHAPE 0: 16x16x128 e4m3, 1: 32x32x64 e4m3, 2: 16x16x128 e2m1 (twice the MFMAs per iteration)
template <int SHAPE, bool RANDOM, int NOPER>
__global__ __launch_bounds__(256) void stream(float* out, int iters) {
  v8i a[NOPER], b[NOPER];
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  for (int n = 0; n < NOPER; ++n)
    for (int i = 0; i < 8; ++i) {
      const uint32_t ra = RANDOM ? hash32(t * 64 + n * 16 + i) : 0x38383838u;
      const uint32_t rb = RANDOM ? hash32(t * 64 + n * 16 + 8 + i) : 0x3c3c3c3cu;
      a[n][i] = (int)(ra & 0xBFBFBFBFu);  // top exponent bit cleared: every e4m3 byte finite and moderate
      b[n][i] = (int)(rb & 0xBFBFBFBFu);
    }
  v4f acc4[16];
  v16f acc16[8];
  for (int i = 0; i < 16; ++i) acc4[i] = v4f{0, 0, 0, 0};
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 16; ++j) acc16[i][j] = 0;
  for (int it = 0; it < iters; ++it) {
    if constexpr (SHAPE == 0) {
#pragma unroll
      for (int m = 0; m < 16; ++m)
        acc4[m] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[m % NOPER], b[(m / 4) % NOPER], acc4[m], 0, 0, 0, 127, 0, 127);
    } else if constexpr (SHAPE == 1) {
#pragma unroll
      for (int m = 0; m < 8; ++m)
        acc16[m] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[m % NOPER], b[(m / 4) % NOPER], acc16[m], 0, 0, 0, 127, 0, 127);
    } else {
#pragma unroll
      for (int m = 0; m < 32; ++m)
        acc4[m % 16] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[m % NOPER], b[(m / 4) % NOPER], acc4[m % 16], 4, 4, 0, 127, 0, 127);
    }
  }
  float s = 0;
  for (int i = 0; i < 16; ++i) s += acc4[i][0] + acc4[i][3];
  for (int i = 0; i < 8; ++i) s += acc16[i][0] + acc16[i][15];
  if (s == 12345.f) out[t] = s;  // keeps the accumulators alive
}

template <int SHAPE, bool RANDOM, int NOPER>
void run(float* out, int cus) {
  const int iters = 4000;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) exit(1);
  for (int i = 0; i < 60; ++i) stream<SHAPE, RANDOM, NOPER><<<cus, 256>>>(out, iters);
  (void)hipEventRecord(e0);
  const int n = 40;
  for (int i = 0; i < n; ++i) stream<SHAPE, RANDOM, NOPER><<<cus, 256>>>(out, iters);
  (void)hipEventRecord(e1);
  if (hipDeviceSynchronize() != hipSuccess) { printf("launch failed\n"); exit(1); }
  float ms = 0;
  (void)hipEventElapsedTime(&ms, e0, e1);
  const double flops = (double)cus * 4 * iters * (SHAPE == 2 ? 32 : 16) * (16.0 * 16 * 128 * 2) * n;
  printf("%-16s %-8s operands, %d register set(s): %5.2f PFLOP/s\n",
         SHAPE == 2 ? "16x16x128 e2m1" : SHAPE == 1 ? "32x32x64 e4m3" : "16x16x128 e4m3", RANDOM ? "random" : "constant", NOPER,
         flops / (ms * 1e-3) / 1e15);
  fflush(stdout);
}

int main() {
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess || cus <= 0) return 1;
  float* out = nullptr;
  if (hipMalloc(&out, (size_t)cus * 256 * sizeof(float)) != hipSuccess) return 1;
  run<0, false, 1>(out, cus); run<1, false, 1>(out, cus); run<2, false, 1>(out, cus);
  run<0, true, 1>(out, cus);  run<1, true, 1>(out, cus);  run<2, true, 1>(out, cus);
  run<0, true, 4>(out, cus);  run<1, true, 4>(out, cus);  run<2, true, 4>(out, cus);
  (void)hipFree(out);
  return 0;
}
