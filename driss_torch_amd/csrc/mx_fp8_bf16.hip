// dt_mx_fp8_bf16: block-scaled e4m3 x e4m3 -> bf16 GEMM on the CDNA4 scaled MFMA (C ABI).
//
// D[M,N] = sum_k (A[m,k] 2^(sfa[m,k/32]-127)) (B[n,k] 2^(sfb[n,k/32]-127)); A is [M,K] and B is
// [N,K], both with K contiguous.  Operand layout of v_mfma_scale_f32_16x16x128_f8f6f4 (measured
// on gfx950): lane l = 16*g + i supplies, for row i, K = 16g..16g+15 in its first four VGPRs
// and K = 64+16g..64+16g+15 in the last four; the E8M0 byte lane l supplies scales K-block g
// (K = 32g..32g+31) of row i.  So a fragment is two 16-byte reads 64 bytes apart, and one MX
// block maps to one scale lane.
//
// A workgroup of 4 waves owns a BM x BN output tile and walks K in steps of 128.  The A and B
// panels of a step are staged through LDS (rows padded by 16 bytes so the 16-byte fragment
// reads of 8 consecutive rows fall in distinct banks); the next step's panels are fetched
// into registers while the current step is multiplied.  The MFMA is issued with B as the
// row operand, so a lane's four accumulators are four consecutive columns of one output
// row and leave as one 8-byte store.
#include "dt_device.hpp"
#include "dt_host.hpp"

namespace dt {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kBK = 128;            // K bytes per step = one 16x16x128 MFMA
constexpr int kLdsRow = kBK + 16;   // padded LDS row pitch in bytes

__device__ __forceinline__ uint32_t bf16_rne_bits(float f) {
  uint32_t u = as_u32(f);
  if (f != f) return (u >> 16) | 0x0040u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// byte offset inside a blocked scale buffer of the 4-byte group (row r, K-step ks)
__device__ __forceinline__ int64_t sf_group_offset(int r, int ks, int k_steps) {
  return ((int64_t)(r >> 7) * k_steps + ks) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4;
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(WAVES_M* WAVES_N* kWave) void mx_gemm_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const uint8_t* __restrict__ sfa,
    const uint8_t* __restrict__ sfb, int M, int N, int K, int64_t lda, int64_t ldb, uint16_t* __restrict__ out,
    int64_t ldo, int tiles_m, int tiles_n) {
  constexpr int kThreads = WAVES_M * WAVES_N * kWave;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
  constexpr int TM = WM / 16, TN = WN / 16;            // MFMA tiles per wave
  constexpr int kChunksA = BM * (kBK / 16) / kThreads; // 16-byte chunks per thread and step
  constexpr int kChunksB = BN * (kBK / 16) / kThreads;
  static_assert(kChunksA * kThreads == BM * 8 && kChunksB * kThreads == BN * 8, "tile/threads mismatch");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  uint8_t* ldsA = lds;
  uint8_t* ldsB = lds + BM * kLdsRow;

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous run of tile
  // ids so that neighbours in the tile grid share an L2, then walk tiles in column groups.
  int bid = blockIdx.x;
  const int nb = tiles_m * tiles_n;
  if (nb % 8 == 0) bid = (bid % 8) * (nb / 8) + bid / 8;
  constexpr int kGroup = 8;  // tile rows per group
  const int group_size = kGroup * tiles_n;
  const int g = bid / group_size, first_m = g * kGroup;
  const int gm = (tiles_m - first_m) < kGroup ? (tiles_m - first_m) : kGroup;
  const int tile_m = first_m + (bid % group_size) % gm;
  const int tile_n = (bid % group_size) / gm;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int k_steps = K / kBK;

  // ---- global -> register staging of one K-step (rows past the edge re-read the last row;
  // their products are never stored)
  u32x4 stA[kChunksA], stB[kChunksB];
  auto fetch = [&](int ks) {
#pragma unroll
    for (int i = 0; i < kChunksA; ++i) {
      const int q = tid + i * kThreads, r = q >> 3, c = q & 7;
      int gr = m0 + r;
      gr = gr < M ? gr : M - 1;
      stA[i] = *reinterpret_cast<const u32x4*>(A + (int64_t)gr * lda + (int64_t)ks * kBK + c * 16);
    }
#pragma unroll
    for (int i = 0; i < kChunksB; ++i) {
      const int q = tid + i * kThreads, r = q >> 3, c = q & 7;
      int gr = n0 + r;
      gr = gr < N ? gr : N - 1;
      stB[i] = *reinterpret_cast<const u32x4*>(B + (int64_t)gr * ldb + (int64_t)ks * kBK + c * 16);
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < kChunksA; ++i) {
      const int q = tid + i * kThreads, r = q >> 3, c = q & 7;
      *reinterpret_cast<u32x4*>(ldsA + r * kLdsRow + c * 16) = stA[i];
    }
#pragma unroll
    for (int i = 0; i < kChunksB; ++i) {
      const int q = tid + i * kThreads, r = q >> 3, c = q & 7;
      *reinterpret_cast<u32x4*>(ldsB + r * kLdsRow + c * 16) = stB[i];
    }
  };

  // ---- scales: one 4-byte group (4 K-blocks of this step) per row, read from the blocked
  // buffers; the lane's own K-block is lane/16, moved to byte 0 for op_sel 0.
  const int kq = lane >> 4, l16 = lane & 15;
  const int rows_a_pad = ((M + 127) / 128) * 128, rows_b_pad = ((N + 127) / 128) * 128;
  uint32_t scA[TM], scB[TN];
  auto fetch_scales = [&](int ks) {
#pragma unroll
    for (int t = 0; t < TM; ++t) {
      int r = m0 + wm * WM + t * 16 + l16;
      r = r < rows_a_pad ? r : rows_a_pad - 1;
      scA[t] = *reinterpret_cast<const uint32_t*>(sfa + sf_group_offset(r, ks, k_steps));
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      int r = n0 + wn * WN + t * 16 + l16;
      r = r < rows_b_pad ? r : rows_b_pad - 1;
      scB[t] = *reinterpret_cast<const uint32_t*>(sfb + sf_group_offset(r, ks, k_steps));
    }
  };

  v4f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  fetch(0);
  for (int ks = 0; ks < k_steps; ++ks) {
    stage();
    fetch_scales(ks);
    __syncthreads();
    if (ks + 1 < k_steps) fetch(ks + 1);

    v8i fa[TM], fb[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) {
      const uint8_t* p = ldsA + (wm * WM + t * 16 + l16) * kLdsRow + kq * 16;
      const u32x4 lo = *reinterpret_cast<const u32x4*>(p), hi = *reinterpret_cast<const u32x4*>(p + 64);
      fa[t] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      const uint8_t* p = ldsB + (wn * WN + t * 16 + l16) * kLdsRow + kq * 16;
      const u32x4 lo = *reinterpret_cast<const u32x4*>(p), hi = *reinterpret_cast<const u32x4*>(p + 64);
      fb[t] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int sa = (int)(scA[i] >> (8 * kq));
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int sb = (int)(scB[j] >> (8 * kq));
        // B fragment as the row operand: acc[i][j][v] = D[m = l16][n = 4*kq + v] of the tile
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i], acc[i][j], 0, 0, 0, sb, 0, sa);
      }
    }
    __syncthreads();
  }

  // ---- epilogue: fp32 -> bf16 (round to nearest even), 4 consecutive columns per lane
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * WM + i * 16 + l16;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * WN + j * 16 + kq * 4;
      if (n >= N) continue;  // N % 4 == 0 is checked on the host, so the 4 columns are all inside
      u32x2 w;
      w.x = bf16_rne_bits(acc[i][j].x) | (bf16_rne_bits(acc[i][j].y) << 16);
      w.y = bf16_rne_bits(acc[i][j].z) | (bf16_rne_bits(acc[i][j].w) << 16);
      *reinterpret_cast<u32x2*>(out + (int64_t)m * ldo + n) = w;
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch_gemm(const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N,
                int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo, hipStream_t stream) {
  const int tiles_m = (int)ceil_div(M, BM), tiles_n = (int)ceil_div(N, BN);
  const size_t lds_bytes = (size_t)(BM + BN) * kLdsRow;
  auto kernel = mx_gemm_kernel<BM, BN, WAVES_M, WAVES_N>;
  if (lds_bytes > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess)
      return DT_ERR_LAUNCH;
  }
  kernel<<<(unsigned)(tiles_m * tiles_n), WAVES_M * WAVES_N * kWave, lds_bytes, stream>>>(
      a, b, sfa, sfb, (int)M, (int)N, (int)K, lda, ldb, static_cast<uint16_t*>(out), ldo, tiles_m, tiles_n);
  return launch_status();
}

}  // namespace dt

extern "C" int dt_mx_fp8_bf16(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M,
                              int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo,
                              dt_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return DT_ERR_INVALID_SHAPE;
  if (M == 0 || N == 0) return DT_OK;
  if (K == 0 || K % dt::kBK != 0) return DT_ERR_INVALID_SHAPE;
  if (N % 4 != 0 || ldo % 4 != 0 || ldo < N || lda < K || ldb < K) return DT_ERR_INVALID_SHAPE;
  if (M > 0x7FFFFF00ll || N > 0x7FFFFF00ll || K > 0x7FFFFF00ll) return DT_ERR_INVALID_SHAPE;
  if (!a || !b || !sfa || !sfb || !out) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(a, 16) || !dt::aligned(b, 16) || lda % 16 != 0 || ldb % 16 != 0) return DT_ERR_MISALIGNED;
  if (!dt::aligned(out, 8) || !dt::aligned(sfa, 4) || !dt::aligned(sfb, 4)) return DT_ERR_MISALIGNED;
  const uint8_t* A = static_cast<const uint8_t*>(a);
  const uint8_t* B = static_cast<const uint8_t*>(b);
  hipStream_t s = dt::as_hip(stream);
  const int variant = dt::tuning("gemm.variant");
  const int64_t tiles256 = dt::ceil_div(M, 256) * dt::ceil_div(N, 256);
  const bool big = variant == 2 || (variant == 0 && tiles256 >= dt::device_facts().cu_count / 2);
  if (big) return dt::launch_gemm<256, 256, 2, 2>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s);
  return dt::launch_gemm<128, 128, 2, 2>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s);
}
