// What HBM gives on one MI355X for the access shapes the cast kernels use, measured with kernels
// that do nothing else: 128 MiB buffers, rotated over six of them so that nothing is served by the
// 256 MiB memory-side cache, 30 launches between one pair of events.
//
//   read        grid-strided 16-byte streaming loads, DEPTH of them in flight per lane, one or more
//               workgroups of 4 waves per CU
//   write       grid-strided 16-byte streaming stores
//   read+write  2 bytes read per byte written (a bf16 -> fp8 cast) and 1:1
//   tile read   128 rows x 512 bytes per workgroup (the transposing MX casts), tiles ordered along
//               the rows of the matrix or down its columns
//   tile write  the same tiles written in pieces of 128 or 256 bytes, streaming or plain stores
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 driss_torch_amd/benchmarks/probes/hbm_stream_rates.hip -o hbm_stream_rates
//   ./hbm_stream_rates
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int64_t kBytes = 128ll << 20;
constexpr uint32_t kRows = 8192, kPitch = 16384;  // the 128 MiB buffer as a matrix of 8192 rows of 16 KiB

template <int DEPTH>
__global__ __launch_bounds__(256) void read_kernel(const u32x4* in, int64_t nvec, uint32_t* out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  uint32_t acc = 0;
  for (; i + (DEPTH - 1) * stride < nvec; i += DEPTH * stride) {
    u32x4 w[DEPTH];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) w[u] = __builtin_nontemporal_load(in + i + u * stride);
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) acc ^= w[u].x ^ w[u].w;
  }
  if (acc == 0x12345678u) out[threadIdx.x] = acc;
}

__global__ __launch_bounds__(256) void write_kernel(u32x4* out, int64_t nvec, uint32_t seed) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  u32x4 v = {seed + threadIdx.x, seed * 3, seed ^ 0x55, seed + 7};
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) __builtin_nontemporal_store(v, out + i);
}

template <int RATIO>
__global__ __launch_bounds__(256) void copy_kernel(const u32x4* in, u32x4* out, int64_t nvec_out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec_out; i += stride) {
    u32x4 a = __builtin_nontemporal_load(in + i * RATIO);
    if (RATIO == 2) {
      const u32x4 b = __builtin_nontemporal_load(in + i * RATIO + 1);
      a.x ^= b.x; a.y ^= b.y; a.z ^= b.z; a.w ^= b.w;
    }
    __builtin_nontemporal_store(a, out + i);
  }
}

// one workgroup per tile of 128 rows x 512 bytes; a wave reads 32 rows, its lower half rows 0..15
__global__ __launch_bounds__(256) void tile_read_kernel(const uint8_t* x, int along_rows, uint32_t* out) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, h = lane >> 5, c = lane & 31;
  const uint32_t col_tiles = kPitch / 512, row_tiles = kRows / 128;
  uint32_t tr, tc;
  if (along_rows) { tr = blockIdx.x / col_tiles; tc = blockIdx.x % col_tiles; } else { tc = blockIdx.x / row_tiles; tr = blockIdx.x % row_tiles; }
  const uint8_t* p = x + (uint64_t)(tr * 128 + w * 32 + h * 16) * kPitch + tc * 512 + c * 16;
  u32x4 v[16];
  uint32_t acc = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = __builtin_nontemporal_load((const u32x4*)(p + (uint64_t)i * kPitch));
#pragma unroll
  for (int i = 0; i < 16; ++i) acc ^= v[i].x ^ v[i].y;
  if (acc == 0x12345678u) out[threadIdx.x] = acc;
}

// a 64 MiB matrix of 8192 rows of 8 KiB written in tiles of ROWS rows x PIECE bytes
template <int PIECE, int ROWS, bool STREAM>
__global__ __launch_bounds__(256) void tile_write_kernel(uint8_t* out, int along_rows) {
  constexpr uint32_t pitch = 8192;
  constexpr int kChunks = PIECE / 16, kRowsPerPass = 256 / kChunks;
  static_assert(kRowsPerPass >= 1 && ROWS % kRowsPerPass == 0, "piece size");
  const uint32_t col_tiles = pitch / PIECE, row_tiles = 8192 / ROWS;
  uint32_t tr, tc;
  if (along_rows) { tr = blockIdx.x / col_tiles; tc = blockIdx.x % col_tiles; } else { tc = blockIdx.x / row_tiles; tr = blockIdx.x % row_tiles; }
  const uint32_t r0 = threadIdx.x / kChunks, q = threadIdx.x % kChunks;
  const u32x4 v = {blockIdx.x, r0, q, 7u};
#pragma unroll 8
  for (uint32_t r = r0; r < ROWS; r += kRowsPerPass) {
    u32x4* p = reinterpret_cast<u32x4*>(out + (uint64_t)(tr * ROWS + r) * pitch + tc * PIECE + q * 16);
    if (STREAM) __builtin_nontemporal_store(v, p); else *p = v;
  }
}

int main() {
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess || cus <= 0) return 1;
  std::vector<uint8_t*> bufs(6);
  for (auto& b : bufs)
    if (hipMalloc(&b, kBytes) != hipSuccess || hipMemset(b, 1, kBytes) != hipSuccess) return 1;
  uint32_t* out = nullptr;
  if (hipMalloc(&out, 4096) != hipSuccess) return 1;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return 1;
  auto timeit = [&](const char* name, double megabytes, auto launch) {
    for (int i = 0; i < 5; ++i) launch(i);
    (void)hipEventRecord(e0);
    const int n = 30;
    for (int i = 0; i < n; ++i) launch(i);
    (void)hipEventRecord(e1);
    if (hipEventSynchronize(e1) != hipSuccess) { printf("launch failed\n"); exit(1); }
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    const double us = ms * 1e3 / n;
    printf("%-66s %6.1f us %6.0f GB/s\n", name, us, megabytes / us * 1e3);
    fflush(stdout);
  };
  const int64_t nvec = kBytes / 16;
  auto in = [&](int i) { return reinterpret_cast<const u32x4*>(bufs[i % 6]); };
  auto outv = [&](int i) { return reinterpret_cast<u32x4*>(bufs[(i + 3) % 6]); };
  timeit("read 128 MiB, 4 loads in flight, 1 workgroup per CU", 134.2, [&](int i) { read_kernel<4><<<cus, 256>>>(in(i), nvec, out); });
  timeit("read 128 MiB, 8 loads in flight, 1 workgroup per CU", 134.2, [&](int i) { read_kernel<8><<<cus, 256>>>(in(i), nvec, out); });
  timeit("read 128 MiB, 16 loads in flight, 1 workgroup per CU", 134.2, [&](int i) { read_kernel<16><<<cus, 256>>>(in(i), nvec, out); });
  timeit("read 128 MiB, 8 loads in flight, 4 workgroups per CU", 134.2, [&](int i) { read_kernel<8><<<cus * 4, 256>>>(in(i), nvec, out); });
  timeit("write 128 MiB, 1 workgroup per CU", 134.2, [&](int i) { write_kernel<<<cus, 256>>>(outv(i), nvec, i); });
  timeit("write 128 MiB, 4 workgroups per CU", 134.2, [&](int i) { write_kernel<<<cus * 4, 256>>>(outv(i), nvec, i); });
  timeit("read 128 MiB + write 64 MiB, 2 workgroups per CU", 201.3, [&](int i) { copy_kernel<2><<<cus * 2, 256>>>(in(i), outv(i), nvec / 2); });
  timeit("read 128 MiB + write 128 MiB, 2 workgroups per CU", 268.4, [&](int i) { copy_kernel<1><<<cus * 2, 256>>>(in(i), outv(i), nvec); });
  const int tiles = (kRows / 128) * (kPitch / 512);
  timeit("tile read 128 x 512 B, tiles along the rows", 134.2, [&](int i) { tile_read_kernel<<<tiles, 256>>>(bufs[i % 6], 1, out); });
  timeit("tile read 128 x 512 B, tiles down the columns", 134.2, [&](int i) { tile_read_kernel<<<tiles, 256>>>(bufs[i % 6], 0, out); });
  timeit("tile write 64 MiB, 256 rows x 128 B, along the rows, streaming", 67.1, [&](int i) { tile_write_kernel<128, 256, true><<<32 * 64, 256>>>(bufs[i % 6], 1); });
  timeit("tile write 64 MiB, 256 rows x 128 B, down the columns, streaming", 67.1, [&](int i) { tile_write_kernel<128, 256, true><<<32 * 64, 256>>>(bufs[i % 6], 0); });
  timeit("tile write 64 MiB, 256 rows x 128 B, down the columns, plain", 67.1, [&](int i) { tile_write_kernel<128, 256, false><<<32 * 64, 256>>>(bufs[i % 6], 0); });
  timeit("tile write 64 MiB, 128 rows x 256 B, along the rows, streaming", 67.1, [&](int i) { tile_write_kernel<256, 128, true><<<64 * 32, 256>>>(bufs[i % 6], 1); });
  timeit("tile write 64 MiB, 128 rows x 256 B, down the columns, streaming", 67.1, [&](int i) { tile_write_kernel<256, 128, true><<<64 * 32, 256>>>(bufs[i % 6], 0); });
  for (auto& b : bufs) (void)hipFree(b);
  (void)hipFree(out);
  return 0;
}
