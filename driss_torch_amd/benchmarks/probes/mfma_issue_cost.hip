// What an LDS read or an LDS-DMA load costs a wave that is streaming scaled MFMAs.  One workgroup
// per CU (forced by its LDS allocation), 4 or 8 waves; every wave issues independent MFMAs with,
// pinned after each of the first NLDS (NDMA) of them, one ds_read_b128 (one global_load_lds_dwordx4
// from a buffer that stays in L2).  Reported: cycles per iteration seen by wave 0 and wall time per
// iteration; the difference to the row without extra instructions, divided by their number, is the
// cost of one.  With 8 waves (two per SIMD) the other wave's MFMAs fill those gaps.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 driss_torch_amd/benchmarks/probes/mfma_issue_cost.hip -o mfma_issue_cost
//   ./mfma_issue_cost
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint8_t* lptr_t;

constexpr int kLdsBytes = 144 * 1024;  // more than half of the CU's LDS: one workgroup per CU

// FP4 false: 16 e4m3 MFMAs (32 cycles each) per iteration; true: 32 e2m1 MFMAs (16 cycles each)
template <bool FP4, int NDMA, int NLDS>
__global__ __launch_bounds__(512) void k(const uint8_t* src, uint64_t* out, int iters) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  v8i a, b;
  for (int i = 0; i < 8; ++i) { a[i] = 0x38383838 + lane * (i + 1); b[i] = 0x3c3c3c3c ^ (lane << i); }
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds + wave * 16384;
  const uint32_t lane_off = lane * 16;
  v4f acc[16];
  for (int i = 0; i < 16; ++i) acc[i] = v4f{0, 0, 0, 0};
  v4i sink = {0, 0, 0, 0};
  __syncthreads();
  const uint64_t t0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) {
    const uint8_t* base = src + ((it & 7) * 8 + wave) * 16384;
    constexpr int NM = FP4 ? 32 : 16;
    v4i r[NLDS > 0 ? NLDS : 1];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      if constexpr (FP4) acc[m % 16] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[m % 16], 4, 4, 0, 127, 0, 127);
      else acc[m] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[m], 0, 0, 0, 127, 0, 127);
      __builtin_amdgcn_sched_barrier(0);
      if (m < NDMA)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_base + m * 1024), "v"(lane_off + m * 1024), "s"(base)
                     : "memory");
      if (m < NLDS) r[m] = *reinterpret_cast<const v4i*>(lds + wave * 16384 + m * 1024 + lane * 16);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");  // the previous iteration's loads
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < NLDS; ++n) sink ^= r[n];
    __builtin_amdgcn_sched_barrier(0);
  }
  const uint64_t t1 = __builtin_readcyclecounter();
  float s = 0;
  for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][3];
  if (threadIdx.x == 0) out[blockIdx.x] = t1 - t0;
  if (s == 12345.f || sink[0] == 0x7fffffff) out[blockIdx.x] = 0;
}

template <bool FP4, int NDMA, int NLDS>
void run(const uint8_t* src, uint64_t* out, int cus, int threads) {
  const int iters = 2000;
  auto kern = k<FP4, NDMA, NLDS>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess) exit(1);
  kern<<<cus, threads, kLdsBytes>>>(src, out, iters);
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) exit(1);
  (void)hipEventRecord(e0);
  kern<<<cus, threads, kLdsBytes>>>(src, out, iters);
  (void)hipEventRecord(e1);
  if (hipDeviceSynchronize() != hipSuccess) { printf("launch failed\n"); exit(1); }
  float ms = 0;
  (void)hipEventElapsedTime(&ms, e0, e1);
  uint64_t h = 0;
  if (hipMemcpy(&h, out, sizeof h, hipMemcpyDeviceToHost) != hipSuccess) exit(1);
  printf("%s  waves %d  lds-dma/iter %2d  lds reads/iter %2d: %8.1f cycles/iter (wave 0)  %7.1f ns/iter\n", FP4 ? "32 e2m1 MFMAs" : "16 e4m3 MFMAs",
         threads / 64, NDMA, NLDS, (double)h / iters, ms * 1e6 / iters);
  fflush(stdout);
}

int main() {
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess || cus <= 0) return 1;
  uint8_t* src = nullptr;
  uint64_t* out = nullptr;
  if (hipMalloc(&src, 1 << 20) != hipSuccess || hipMalloc(&out, 8 * (size_t)cus) != hipSuccess) return 1;
  if (hipMemset(src, 0x38, 1 << 20) != hipSuccess) return 1;
  for (int threads : {256, 512}) {
    run<false, 0, 0>(src, out, cus, threads);
    run<false, 8, 0>(src, out, cus, threads);
    run<false, 0, 8>(src, out, cus, threads);
    run<false, 0, 16>(src, out, cus, threads);
    run<false, 8, 8>(src, out, cus, threads);
    run<true, 0, 0>(src, out, cus, threads);
    run<true, 8, 0>(src, out, cus, threads);
    run<true, 16, 0>(src, out, cus, threads);
    run<true, 0, 16>(src, out, cus, threads);
    run<true, 0, 32>(src, out, cus, threads);
  }
  (void)hipFree(src);
  (void)hipFree(out);
  return 0;
}
