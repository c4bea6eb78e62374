// MXFP8 cast kernels: one E8M0 scale byte per 32 elements plus the fp8 payload.
//
//  mx_row_kernel   blocks along rows.  A 32-element block is spread over 4 lanes (16-bit
//                  input, 8 elements per 16-byte load) or 8 lanes (fp32 input); the block
//                  maximum is an integer max over DPP quad/row permutes -- no LDS.
//  mx_col_kernel   blocks down columns, payload in the input orientation.  A lane owns 8
//                  (fp32: 4) adjacent columns x 8 rows; the four waves of a workgroup cover
//                  a 32-row tile and merge their column maxima through LDS.
//  mx_col_t_kernel blocks down columns, payload transposed through LDS so that the stores
//                  are full 128-byte rows of the [cols, rows] output.
//  mx_dual_kernel  blocks along rows (payload as is) and down columns (payload transposed) from
//                  one read of the input.
//  mx_row_t_kernel blocks along rows, payload transposed through the same LDS tile.
//  mx_any_kernel   one thread per block, arbitrary strides: covers every (axis, transpose)
//                  pair and shapes the fast kernels do not take.
#pragma once

#include <type_traits>

#include "dt_device.hpp"
#include "dt_host.hpp"
#include "quant_kernels.hpp"

namespace dt {

// position of scale (r, c) of an [R, C] scale matrix in the 128x4 blocked layout
__host__ __device__ __forceinline__ int64_t blocked_offset(int64_t r, int64_t c, int64_t col_tiles /* ceil(C/4) */) {
  return ((r >> 7) * col_tiles + (c >> 2)) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + (c & 3);
}

template <int LAYOUT>
__device__ __forceinline__ int64_t scale_offset(int64_t r, int64_t c, int64_t C) {
  if constexpr (LAYOUT == DT_SCALE_BLOCKED)
    return blocked_offset(r, c, (C + 3) >> 2);
  else
    return r * C + c;
}

// Block magnitude (fp32 bit pattern of max|x|, NaN patterns sort highest) -> E8M0 byte and
// the fp32 multiplier 2^(127-byte) that scales the block into the fp8 range.
template <int OUT>
struct MxScale {
  uint32_t byte;  // 0..254, or 255 for a block that holds a NaN
  float mult;     // 2^(127-b): what the block is multiplied by
  float scale;    // 2^(b-127) as the scaled conversion instructions take it (they divide by it)
  bool nan;
};
template <int OUT>
__device__ __forceinline__ MxScale<OUT> mx_scale_from_absbits(uint32_t absbits) {
  if constexpr (OUT == DT_E2M1) {
    // MXFP4: shared exponent floor(log2(max)) - 2 (2 = exponent of e2m1's largest value, 6), taken
    // from the exponent field; an infinite maximum reads as field 255 (byte 253)
    const int be = (int)(absbits >> 23);
    const int b = be < 2 ? 0 : (be - 2 > 254 ? 254 : be - 2);
    MxScale<OUT> r;
    r.nan = absbits > 0x7F800000u;
    r.byte = r.nan ? 255u : (uint32_t)b;
    r.mult = as_f32((uint32_t)(254 - b) << 23);
    r.scale = as_f32((uint32_t)b << 23);
    return r;
  }
  constexpr int kTargetPow2 = OUT == DT_E5M2 ? 15 : 8;
  const int be = (int)(absbits >> 23);
  const int mant_nz = (absbits & 0x7FFFFFu) ? 1 : 0;
  int e = be - 127 + mant_nz;                       // ceil(log2) from the exponent field
  if (be == 0) e = absbits == 0 ? -128 : -126;      // zero / subnormal maxima
  int b = e - kTargetPow2 + 127;
  b = b < 0 ? 0 : (b > 254 ? 254 : b);
  MxScale<OUT> r;
  r.nan = absbits > 0x7F800000u;
  r.byte = r.nan ? 255u : (uint32_t)b;
  r.mult = as_f32((uint32_t)(254 - b) << 23);       // b <= 248 for any input, so never 2^-127
  r.scale = as_f32((uint32_t)b << 23);              // only the exponent field is read: 0 stands for 2^-127
  return r;
}

// saturating convert without the NaN patch (NaN blocks are overwritten wholesale)
template <int OUT>
__device__ __forceinline__ uint32_t pack4_finite(float p0, float p1, float p2, float p3) {
  uint32_t w = cvt_pk<OUT, false>(clamp_fp8<OUT>(p0), clamp_fp8<OUT>(p1), 0u);
  return cvt_pk<OUT, true>(clamp_fp8<OUT>(p2), clamp_fp8<OUT>(p3), w);
}

// low (half 0) or high (half 1) 16 bits of a and of b as one word {a.half, b.half}
__device__ __forceinline__ uint32_t gather_halves(int half, uint32_t a, uint32_t b) {
  return __builtin_amdgcn_perm(b, a, half ? 0x07060302u : 0x05040100u);
}
// Four adjacent elements with four different scales (blocks down the columns, payload in place).
// A conversion writes two bytes with one scale; the byte that belongs to the other scale is
// overwritten or dropped by the byte permute at the end.
template <int IN, int OUT>
__device__ __forceinline__ uint32_t cvt_scaled_4x16_each(uint32_t w0, uint32_t w1, const float* sc /* 4 scales */) {
  // byte 0 = w.lo / sc[0], byte 3 = w.hi / sc[1]
  const uint32_t u0 = cvt_scaled_pair16<IN, OUT, true>(cvt_scaled_pair16<IN, OUT, false>(w0, w0, sc[0]), w0, sc[1]);
  const uint32_t u1 = cvt_scaled_pair16<IN, OUT, true>(cvt_scaled_pair16<IN, OUT, false>(w1, w1, sc[2]), w1, sc[3]);
  return __builtin_amdgcn_perm(u1, u0, 0x07040300u);
}
template <int OUT>
__device__ __forceinline__ uint32_t cvt_scaled_4x32_each(uint32_t a, uint32_t b, uint32_t c, uint32_t d, const float* sc) {
  const uint32_t e = cvt_scaled_pair32<OUT, true>(cvt_scaled_pair32<OUT, false>(a, a, a, sc[0]), c, c, sc[2]);  // bytes 0, 2
  const uint32_t o = cvt_scaled_pair32<OUT, true>(cvt_scaled_pair32<OUT, false>(b, b, b, sc[1]), d, d, sc[3]);  // bytes 1, 3
  return __builtin_amdgcn_perm(o, e, 0x07020500u);
}

template <int IN>
__device__ __forceinline__ float load_elem(const void* x, int64_t i) {
  if constexpr (IN == DT_F32) return static_cast<const float*>(x)[i];
  else if constexpr (IN == DT_BF16) return as_f32((uint32_t)static_cast<const uint16_t*>(x)[i] << 16);
  else return (float)static_cast<const _Float16*>(x)[i];
}

// 8 consecutive 16-bit elements (one 16-byte vector) as floats
template <int IN>
__device__ __forceinline__ void unpack8(u32x4 w, float (&f)[8]) {
  if constexpr (IN == DT_BF16) {
    f[0] = bf16_lo(w.x); f[1] = bf16_hi(w.x); f[2] = bf16_lo(w.y); f[3] = bf16_hi(w.y);
    f[4] = bf16_lo(w.z); f[5] = bf16_hi(w.z); f[6] = bf16_lo(w.w); f[7] = bf16_hi(w.w);
  } else {
    f[0] = f16_lo(w.x); f[1] = f16_hi(w.x); f[2] = f16_lo(w.y); f[3] = f16_hi(w.y);
    f[4] = f16_lo(w.z); f[5] = f16_hi(w.z); f[6] = f16_lo(w.w); f[7] = f16_hi(w.w);
  }
}

// fp32 bit pattern of the largest magnitude in one 16-byte vector
template <int IN>
__device__ __forceinline__ uint32_t vec_absmax_bits(u32x4 w) {
  if constexpr (IN == DT_F32) {
    return umax(umax(absbits_f32(w.x), absbits_f32(w.y)), umax(absbits_f32(w.z), absbits_f32(w.w)));
  } else if constexpr (IN == DT_BF16) {
    uint32_t p = pk_absmax16(pk_absmax16(pk_absmax16(pk_absmax16(0u, w.x), w.y), w.z), w.w);
    return umax(p & 0xFFFFu, p >> 16) << 16;
  } else {
    float f[8];
    unpack8<IN>(w, f);
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) m = umax(m, absbits_f32(as_u32(f[i])));
    return m;
  }
}

// Streaming loads of x through vector types that claim no more than the element's alignment.  The
// instruction is the same global_load_dwordx4 / dwordx2 ... nt as for an aligned type, and the device
// serves it at any address (an access that straddles a line costs the second line), so every kernel
// below takes an x that is only aligned to its element, e.g. a view that starts one element into its
// buffer (8192 x 8192 bf16 one element off: within a few percent of the aligned case).
typedef u32x2 u32x2_elem2 __attribute__((aligned(2)));
template <int IN>
__device__ __forceinline__ u32x4 ld_x16(const void* p) {
  typedef typename std::conditional<IN == DT_F32, u32x4_elem4, u32x4_elem2>::type vec_t;
  return __builtin_nontemporal_load(static_cast<const vec_t*>(p));
}
__device__ __forceinline__ u32x2 ld_x8_16bit(const void* p) {
  return __builtin_nontemporal_load(static_cast<const u32x2_elem2*>(p));
}

// ------------------------------------------------------------------ blocks along rows
// The matrix is a flat run of 32-element blocks.  One wave pass ("super-chunk") covers 64
// blocks as LPB chunks of 64 vectors; lane l ends up holding the scale byte of chunk
// l % LPB, block l / LPB, so the 64 scale bytes leave in a single store instruction.
//
// BAND4 (blocked scale layout, rows % 128 == 0, cols % 512 == 0): a pass covers 4 rows x 512
// elements instead -- rows q, q+32, q+64, q+96 of a 128-row band, one chunk (fp32: two) per
// row -- because those are the scales that sit next to each other in the blocked layout: the 64
// bytes of a pass then fall into 4 runs of 16 bytes instead of 16 runs of 4, which costs a
// quarter of the memory transactions (36.8 -> 33 us at 8192 x 8192 bf16).
template <int IN, int OUT, int LAYOUT, bool BAND4 = false>
__global__ __launch_bounds__(kBlock) void mx_row_kernel(const void* __restrict__ x, uint32_t nblocks,
                                                        uint32_t kblocks, uint8_t* __restrict__ data,
                                                        uint8_t* __restrict__ scale) {
  static_assert(!BAND4 || LAYOUT == DT_SCALE_BLOCKED, "the 4-row pass exists for the blocked layout");
  constexpr int kV = InTraits<IN>::kVec;      // elements per vector
  constexpr int LPB = 32 / kV;                // lanes per block: 4 or 8
  constexpr int BPC = kWave / LPB;            // blocks per chunk: 16 or 8
  const int lane = threadIdx.x % kWave;
  const uint32_t nvec = nblocks * LPB;
  const u32x4* v = static_cast<const u32x4*>(x);
  const uint32_t nsuper = (nblocks + 63u) / 64u;
  const uint32_t wave_id = (blockIdx.x * kBlock + threadIdx.x) / kWave;
  const uint32_t nwaves = gridDim.x * (kBlock / kWave);
  saturate_fp8_conversions();

  const uint32_t segs = kblocks / 16u;                 // BAND4: 512-element segments per row
  const uint32_t row_vecs = kblocks * (uint32_t)LPB;   // vectors per row
  for (uint32_t sc = wave_id; sc < nsuper; sc += nwaves) {
    // vector index of chunk c of this pass
    uint32_t band_row = 0, seg = 0;
    if constexpr (BAND4) {
      const uint32_t band = sc / (32u * segs), rem = sc - band * 32u * segs, q = rem / segs;
      seg = rem - q * segs;
      band_row = band * 128u + q;
    }
    auto vec_index = [&](int c) -> uint32_t {
      if constexpr (BAND4) return (band_row + 32u * (c & 3)) * row_vecs + seg * (16u * LPB) + (uint32_t)(c >> 2) * kWave + lane;
      else return sc * 64u * LPB + c * kWave + lane;
    };
    u32x4 w[LPB];
#pragma unroll
    for (int c = 0; c < LPB; ++c) {
      const uint32_t vi = vec_index(c);
      w[c] = vi < nvec ? ld_x16<IN>(v + vi) : u32x4{0u, 0u, 0u, 0u};
    }
    uint32_t mybyte = 0;
#pragma unroll
    for (int c = 0; c < LPB; ++c) {
      const uint32_t vi = vec_index(c);
      uint32_t m = quad_umax(vec_absmax_bits<IN>(w[c]));
      if constexpr (LPB == 8) m = umax(m, dpp<kDppRowHalfMirror>(m));
      const MxScale<OUT> s = mx_scale_from_absbits<OUT>(m);
      if ((lane % LPB) == c) mybyte = s.byte;
      if (vi < nvec) {
        if constexpr (OUT == DT_E2M1) {
          // two elements per byte: a vector leaves as 4 bytes (16-bit inputs) or 2 (fp32); a block
          // with a NaN gets 0x7 in every nibble under its NaN scale
          if constexpr (IN == DT_F32) {
            const uint32_t r = cvt_fp4_4x32(w[c], s.scale);
            reinterpret_cast<uint16_t*>(data)[vi] = (uint16_t)(s.nan ? 0x7777u : r);
          } else {
            const uint32_t r = cvt_fp4_8x16<IN>(w[c], s.scale);
            st_words(reinterpret_cast<uint32_t*>(data) + vi, s.nan ? 0x77777777u : r);
          }
        } else if constexpr (IN == DT_F32) {
          const uint32_t r = cvt_scaled_4x32<OUT>(w[c].x, w[c].y, w[c].z, w[c].w, s.scale);
          st_words(reinterpret_cast<uint32_t*>(data) + vi, s.nan ? 0x7F7F7F7Fu : r);
        } else {
          u32x2 r;
          r.x = cvt_scaled_4x16<IN, OUT>(w[c].x, w[c].y, s.scale);
          r.y = cvt_scaled_4x16<IN, OUT>(w[c].z, w[c].w, s.scale);
          if (s.nan) r = u32x2{0x7F7F7F7Fu, 0x7F7F7F7Fu};
          st_stream(reinterpret_cast<u32x2*>(data) + vi, r);
        }
      }
    }
    if constexpr (BAND4) {
      const uint32_t c = lane % LPB, b = lane / LPB;   // mybyte: chunk c, block b of that chunk
      scale[blocked_offset(band_row + 32u * (c & 3), seg * 16u + (c >> 2) * BPC + b, kblocks >> 2)] = (uint8_t)mybyte;
      continue;
    }
    const uint32_t g = sc * 64u + (lane % LPB) * BPC + lane / LPB;  // block index of mybyte
    if (g < nblocks) {
      if constexpr (LAYOUT == DT_SCALE_BLOCKED) {
        const uint32_t r = g / kblocks, c = g - r * kblocks;
        scale[blocked_offset(r, c, (kblocks + 3) >> 2)] = (uint8_t)mybyte;
      } else {
        scale[g] = (uint8_t)mybyte;
      }
    }
  }
}

// --------------------------------------------------------------- blocks down columns
// In-place payload [rows, cols], scales [rows/32, cols].  A workgroup works on tiles of 32 rows x
// 64*kV columns; wave w takes rows 8w..8w+7 of the tile, a lane kV adjacent columns x 8 rows
// (eight 16-byte loads).  Every load instruction of a wave then reads one contiguous run of a
// single row and a wave touches 8 rows, not 32: a read-only probe of this access pattern runs
// at 5.9 TB/s against 5.0-5.4 TB/s for a wave that walks down 32 rows.  The four partial
// column maxima meet in LDS (16 bytes per lane: packed 16-bit magnitudes, or four fp32
// magnitudes), every wave derives the same scales and converts its own rows.  Tiles walk along
// the columns first, so a band of 32 rows is one contiguous stretch of memory on the input and
// on the output side.  The grid is persistent and the loads of a workgroup's next tile are
// issued before the current tile is converted, so that reads, conversion and writes of
// different tiles overlap.
template <int IN, int OUT>
__global__ __launch_bounds__(kBlock) void mx_col_kernel(const void* __restrict__ x, uint32_t rows, uint32_t cols,
                                                        uint8_t* __restrict__ data, uint8_t* __restrict__ scale,
                                                        uint32_t ntiles) {
  constexpr int kV = InTraits<IN>::kVec;   // columns per lane
  constexpr int kW = kV / 4;               // fp8 words per lane and row: 2 or 1
  constexpr int kB = InTraits<IN>::kBytes;
  __shared__ u32x4 part[2][kBlock / kWave][kWave];
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const uint32_t col_tiles = (cols + kWave * kV - 1) / (kWave * kV);
  const uint64_t pitch = (uint64_t)cols * kB;

  // cols % kV == 0, so a lane is either fully inside or outside; rows % 32 == 0
  auto load_tile = [&](u32x4 (&v)[8], uint32_t t) {
    const uint32_t tr = t / col_tiles, tc = t - tr * col_tiles;
    const uint32_t col0 = tc * (kWave * kV) + lane * kV;
    if (col0 < cols) {
      const uint8_t* p = static_cast<const uint8_t*>(x) + (uint64_t)(tr * 32u + w * 8u) * pitch + (uint64_t)col0 * kB;
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = ld_x16<IN>(p + i * pitch);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto process = [&](const u32x4 (&v)[8], uint32_t t, int buf) {
    const uint32_t tr = t / col_tiles, tc = t - tr * col_tiles;
    const uint32_t col0 = tc * (kWave * kV) + lane * kV;
    // this wave's column maxima over its 8 rows
    u32x4 pm = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (IN == DT_F32) {
        pm.x = umax(pm.x, absbits_f32(v[i].x)); pm.y = umax(pm.y, absbits_f32(v[i].y));
        pm.z = umax(pm.z, absbits_f32(v[i].z)); pm.w = umax(pm.w, absbits_f32(v[i].w));
      } else {
        pm.x = pk_absmax16(pm.x, v[i].x); pm.y = pk_absmax16(pm.y, v[i].y);
        pm.z = pk_absmax16(pm.z, v[i].z); pm.w = pk_absmax16(pm.w, v[i].w);
      }
    }
    part[buf][w][lane] = pm;
    __syncthreads();
#pragma unroll
    for (int o = 1; o < kBlock / kWave; ++o) {
      const u32x4 q = part[buf][(w + o) % (kBlock / kWave)][lane];
      if constexpr (IN == DT_F32) {
        pm.x = umax(pm.x, q.x); pm.y = umax(pm.y, q.y); pm.z = umax(pm.z, q.z); pm.w = umax(pm.w, q.w);
      } else {
        pm.x = pk_absmax16(pm.x, q.x); pm.y = pk_absmax16(pm.y, q.y);
        pm.z = pk_absmax16(pm.z, q.z); pm.w = pk_absmax16(pm.w, q.w);
      }
    }
    uint32_t cm[kV];  // fp32 magnitude bits of the column maxima
    if constexpr (IN == DT_F32) {
      cm[0] = pm.x; cm[1] = pm.y; cm[2] = pm.z; cm[3] = pm.w;
    } else if constexpr (IN == DT_BF16) {
      cm[0] = pm.x << 16; cm[1] = pm.x & 0xFFFF0000u; cm[2] = pm.y << 16; cm[3] = pm.y & 0xFFFF0000u;
      cm[4] = pm.z << 16; cm[5] = pm.z & 0xFFFF0000u; cm[6] = pm.w << 16; cm[7] = pm.w & 0xFFFF0000u;
    } else {  // the largest f16 magnitude pattern is the largest magnitude; widen it exactly
      cm[0] = as_u32(f16_lo(pm.x)); cm[1] = as_u32(f16_hi(pm.x)); cm[2] = as_u32(f16_lo(pm.y)); cm[3] = as_u32(f16_hi(pm.y));
      cm[4] = as_u32(f16_lo(pm.z)); cm[5] = as_u32(f16_hi(pm.z)); cm[6] = as_u32(f16_lo(pm.w)); cm[7] = as_u32(f16_hi(pm.w));
    }
    float scl[kV];
    uint32_t nanmask[kW] = {};
    uint32_t bytes[kW] = {};  // the kV scale bytes packed in column order
#pragma unroll
    for (int c = 0; c < kV; ++c) {
      const MxScale<OUT> sc = mx_scale_from_absbits<OUT>(cm[c]);
      scl[c] = sc.scale;
      bytes[c / 4] |= sc.byte << (8 * (c % 4));
      nanmask[c / 4] |= sc.nan ? (0xFFu << (8 * (c % 4))) : 0u;
    }
    if (col0 < cols) {
      uint8_t* drow = data + (uint64_t)(tr * 32u + w * 8u) * cols + col0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        uint32_t r[kW];
        if constexpr (IN == DT_F32) {
          r[0] = cvt_scaled_4x32_each<OUT>(v[i].x, v[i].y, v[i].z, v[i].w, scl);
        } else {
          r[0] = cvt_scaled_4x16_each<IN, OUT>(v[i].x, v[i].y, scl);
          r[1] = cvt_scaled_4x16_each<IN, OUT>(v[i].z, v[i].w, scl + 4);
        }
#pragma unroll
        for (int q = 0; q < kW; ++q) r[q] = (r[q] & ~nanmask[q]) | (0x7F7F7F7Fu & nanmask[q]);
        if constexpr (kW == 2) st_stream(reinterpret_cast<u32x2*>(drow + (uint64_t)i * cols), u32x2{r[0], r[1]});
        else st_words(reinterpret_cast<uint32_t*>(drow + (uint64_t)i * cols), r[0]);
      }
      if (w == 0) {  // scales [rows/32, cols]: kV adjacent bytes
        uint8_t* srow = scale + (uint64_t)tr * cols + col0;
        if constexpr (kW == 2) *reinterpret_cast<u32x2*>(srow) = u32x2{bytes[0], bytes[1]};
        else *reinterpret_cast<uint32_t*>(srow) = bytes[0];
      }
    }
  };

  // part[] alternates between iterations, so one barrier per tile is enough: a wave can be at
  // most one barrier ahead of the slowest reader of the buffer it will write two tiles on
  saturate_fp8_conversions();
  const uint32_t stride = gridDim.x;
  uint32_t t = blockIdx.x;  // < ntiles
  u32x4 va[8], vb[8];
  load_tile(va, t);
  for (;;) {
    uint32_t tn = t + stride;
    if (tn < ntiles) load_tile(vb, tn);
    process(va, t, 0);
    if (tn >= ntiles) break;
    t = tn;
    tn = t + stride;
    if (tn < ntiles) load_tile(va, tn);
    process(vb, t, 1);
    if (tn >= ntiles) break;
    t = tn;
  }
}

// ------------------------------------------- blocks down columns, transposed payload
// A workgroup owns 128 rows x 256 columns.  Wave w takes the 32-row tile w: a lane holds 4
// adjacent columns x 32 rows in registers (8- or 16-byte loads), so the block maximum is again
// lane-local, and converts column by column (4 consecutive rows per packed word).  The fp8
// bytes go to LDS as [column][128 rows] and leave as full 128-byte rows of the [cols, rows]
// output; the 4 scale bytes of a column (one per wave) leave as one word.
// With the e2m1 output code two rows of x share an output byte: a column's 128 rows are 64 bytes.
constexpr int kColTRows = 128, kColTCols = 256, kColTPitch = 144;  // LDS row pitch: 128 + 16 pad
template <int IN, int OUT, int LAYOUT>
__global__ __launch_bounds__(kBlock) void mx_col_t_kernel(const void* __restrict__ x, uint32_t rows, uint32_t cols,
                                                          uint8_t* __restrict__ data, uint8_t* __restrict__ scale) {
  constexpr int kB = InTraits<IN>::kBytes;
  __shared__ __attribute__((aligned(16))) uint8_t tile[kColTCols * kColTPitch];
  __shared__ __attribute__((aligned(16))) uint32_t stile[kColTCols];  // 4 scale bytes per column
  const int tid = threadIdx.x, lane = tid % kWave, w = tid / kWave;
  // Tiles are numbered down the rows first, so that neighbours write adjacent 128-byte output
  // segments and adjacent words of the same scale line.  Workgroup b runs on XCD b % 8 and
  // each XCD has its own L2: runs of 8 consecutive tiles are given to one XCD (workgroups
  // b, b+8, ... which start together), so that its L2 can merge their partial lines.
  const uint32_t row_tiles128 = (rows + kColTRows - 1) / kColTRows;
  uint32_t t = blockIdx.x;
  if (t < (gridDim.x & ~63u)) {
    const uint32_t xcd = t & 7u, slot = t >> 3;
    t = (slot & ~7u) * 8u + xcd * 8u + (slot & 7u);
  }
  const uint32_t tc = t / row_tiles128, tr = t - tc * row_tiles128;
  const uint32_t row0 = tr * kColTRows + w * 32, col0 = tc * kColTCols + lane * 4;
  const bool active = row0 < rows && col0 < cols;  // rows % 32 == 0 and cols % 4 == 0

  saturate_fp8_conversions();
  uint32_t sbyte[4] = {0, 0, 0, 0};
  if (active) {
    // 32 rows x 4 columns kept packed as loaded: fp32 -> one 16-byte load per row, 16-bit -> one
    // 8-byte load; elements are unpacked where they are used
    typedef typename std::conditional<IN == DT_F32, u32x4, u32x2>::type row_t;
    row_t wv[32];
    uint32_t cm[4] = {0, 0, 0, 0};
    const uint8_t* p = static_cast<const uint8_t*>(x) + ((uint64_t)row0 * cols + col0) * kB;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      if constexpr (IN == DT_F32) wv[i] = ld_x16<IN>(p + (uint64_t)i * cols * kB);
      else wv[i] = ld_x8_16bit(p + (uint64_t)i * cols * kB);
    }
    // the word that holds column c of row i (fp32: the element itself; 16-bit: it and its neighbour)
    auto word = [&](int i, int c) -> uint32_t {
      if constexpr (IN == DT_F32) return c == 0 ? wv[i].x : c == 1 ? wv[i].y : c == 2 ? wv[i].z : wv[i].w;
      else return c < 2 ? wv[i].x : wv[i].y;
    };
    auto elem = [&](int i, int c) -> float {  // (only for the column maxima of f16 / fp32 inputs)
      if constexpr (IN == DT_F32) return as_f32(word(i, c));
      else if constexpr (IN == DT_BF16) return (c & 1) ? bf16_hi(word(i, c)) : bf16_lo(word(i, c));
      else return (c & 1) ? f16_hi(word(i, c)) : f16_lo(word(i, c));
    };
    if constexpr (IN == DT_BF16) {
      uint32_t p0 = 0, p1 = 0;
#pragma unroll
      for (int i = 0; i < 32; ++i) { p0 = pk_absmax16(p0, wv[i].x); p1 = pk_absmax16(p1, wv[i].y); }
      cm[0] = p0 << 16; cm[1] = p0 & 0xFFFF0000u; cm[2] = p1 << 16; cm[3] = p1 & 0xFFFF0000u;
    } else {
#pragma unroll
      for (int i = 0; i < 32; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) cm[c] = umax(cm[c], absbits_f32(as_u32(elem(i, c))));
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const MxScale<OUT> s = mx_scale_from_absbits<OUT>(cm[c]);
      sbyte[c] = s.byte;
      if constexpr (OUT == DT_E2M1) {
        uint32_t r4[4];  // 8 consecutive rows per word: byte j = rows 8q+2j (low nibble), 8q+2j+1
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint32_t r = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int i = 8 * q + 2 * j;
            if constexpr (IN == DT_F32) {
              r = cvt_fp4_pair32(r, word(i, c), word(i + 1, c), s.scale, j);
            } else {
              r = cvt_fp4_pair16<IN>(r, gather_halves(c & 1, word(i, c), word(i + 1, c)), s.scale, j);
            }
          }
          r4[q] = s.nan ? 0x77777777u : r;
        }
        *reinterpret_cast<u32x4*>(tile + (lane * 4 + c) * kColTPitch + w * 16) = u32x4{r4[0], r4[1], r4[2], r4[3]};
        continue;
      }
      uint32_t r[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        if constexpr (IN == DT_F32)
          r[q] = cvt_scaled_4x32<OUT>(word(4 * q, c), word(4 * q + 1, c), word(4 * q + 2, c), word(4 * q + 3, c), s.scale);
        else
          r[q] = cvt_scaled_4x16<IN, OUT>(gather_halves(c & 1, word(4 * q, c), word(4 * q + 1, c)),
                                          gather_halves(c & 1, word(4 * q + 2, c), word(4 * q + 3, c)), s.scale);
        if (s.nan) r[q] = 0x7F7F7F7Fu;
      }
      u32x4* t = reinterpret_cast<u32x4*>(tile + (lane * 4 + c) * kColTPitch + w * 32);
      t[0] = u32x4{r[0], r[1], r[2], r[3]};
      t[1] = u32x4{r[4], r[5], r[6], r[7]};
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) reinterpret_cast<uint8_t*>(stile)[(lane * 4 + c) * 4 + w] = (uint8_t)sbyte[c];
  __syncthreads();

  // 256 output rows (columns of x) x 8 chunks of 16 bytes; 8 consecutive lanes write one row
  const uint32_t trow0 = tr * kColTRows, tcol0 = tc * kColTCols;
  if constexpr (OUT == DT_E2M1) {  // 4 chunks of 16 bytes (32 rows of x each) per output row
#pragma unroll
    for (int i = 0; i < kColTCols * 4 / kBlock; ++i) {
      const int id = tid + i * kBlock, r = id >> 2, q = id & 3;
      if (tcol0 + r < cols && trow0 + q * 32 < rows) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(tile + r * kColTPitch + q * 16);
        st_stream(reinterpret_cast<u32x4*>(data + (uint64_t)(tcol0 + r) * (rows / 2) + trow0 / 2 + q * 16), v);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < kColTCols * 8 / kBlock; ++i) {
      const int id = tid + i * kBlock, r = id >> 3, q = id & 7;
      if (tcol0 + r < cols && trow0 + q * 16 < rows) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(tile + r * kColTPitch + q * 16);
        st_stream(reinterpret_cast<u32x4*>(data + (uint64_t)(tcol0 + r) * rows + trow0 + q * 16), v);
      }
    }
  }
  // scales [cols, rows/32]: 4 bytes per column of this tile
  const uint32_t RB = rows / 32, rb0 = tr * 4;
  if (tcol0 + tid < cols) {
    const uint32_t sw = stile[tid];
    const uint32_t c = tcol0 + tid;
    if (LAYOUT == DT_SCALE_BLOCKED || (RB % 4 == 0)) {
      // rb0 % 4 == 0: the four bytes are adjacent and word aligned in both layouts (bytes of
      // row tiles past the end are zero, which is what the padding must hold)
      *reinterpret_cast<uint32_t*>(scale + scale_offset<LAYOUT>(c, rb0, RB)) = sw;
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (rb0 + k < RB) scale[scale_offset<LAYOUT>(c, rb0 + k, RB)] = (uint8_t)(sw >> (8 * k));
    }
  }
}

// -------------------------------- both blockings from one read of the input ("dual")
// Row-wise cast in the input orientation plus the column-wise cast with a transposed payload:
// the two operands a training step needs of one tensor (x for the forward product, x^T for the
// weight gradient), from a single pass over x.  A workgroup owns 128 rows x 32*kV columns.  Wave
// w takes rows 32w..32w+31: its lower 32 lanes hold rows 0..15 of those, the upper 32 lanes rows
// 16..31, each lane kV adjacent columns (sixteen 16-byte loads; one load instruction of a wave
// reads two contiguous row segments).  The row-block maximum is a max over the 4 (fp32: 8)
// neighbouring lanes, the column-block maximum a lane-local max over 16 rows merged with the
// other half of the wave.  Row payload and nothing else goes straight to memory; the column
// payload is transposed through LDS as in mx_col_t_kernel, and both sets of scale bytes are
// staged in LDS so that they leave as whole words.
//
// LDS tile: [column][128 rows] with a pitch of 144 bytes; the 16-byte chunk index is XORed
// with bits 4..6 of the column so that the 16 lanes of one write phase (columns kV apart) fall
// on 16 different bank groups.
constexpr int kDualRows = 128, kDualPitch = 144;
// (e2m1 output: a column's 128 rows are 64 bytes; pitch 80, the chunk index XORed with bits 4..5 of the column)
constexpr int kDualPitch4 = 80;

__device__ __forceinline__ uint32_t other_half_max_u32(uint32_t v) {
  const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);  // [0]: lower half's value, [1]: upper half's
  return umax(r[0], r[1]);
}
__device__ __forceinline__ uint32_t other_half_max_pk16(uint32_t v) {  // v: two 16-bit magnitudes
  const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return pk_absmax16(r[0], r[1]);
}

// WITH_ROWS = false leaves out the row-wise half (data_r / scale_r unused): the transposed column
// cast on its own.  cols then only has to be a multiple of a lane's kV columns.
// PIPE: a grid smaller than the tile count; a workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...
// and has the loads of its next tile in flight while it converts and stores the one in hand.
template <int IN, int OUT, int LAYOUT, bool WITH_ROWS = true, bool PIPE = false>
__global__ __launch_bounds__(kBlock) void mx_dual_kernel(const void* __restrict__ x, uint32_t rows, uint32_t cols,
                                                         uint8_t* __restrict__ data_r, uint8_t* __restrict__ scale_r,
                                                         uint8_t* __restrict__ data_c, uint8_t* __restrict__ scale_c, int cols_first) {
  constexpr int kV = InTraits<IN>::kVec;     // columns per lane: 8 or 4
  constexpr int kB = InTraits<IN>::kBytes;
  constexpr int kTileCols = 32 * kV;         // 256 or 128
  constexpr int kRowBlocks = kTileCols / 32; // row-direction blocks per tile row: 8 or 4
  constexpr int LPB = 32 / kV;               // lanes per row-direction block: 4 or 8
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileCols * kDualPitch];
  __shared__ __attribute__((aligned(16))) uint32_t ctile[kTileCols];            // [column] -> 4 bytes, one per wave
  __shared__ __attribute__((aligned(16))) uint8_t rtile[kRowBlocks * kDualRows];  // [block][row]
  const int tid = threadIdx.x, lane = tid % kWave, w = tid / kWave, h = lane >> 5, c8 = lane & 31;

  // Tile order.  Along the columns first keeps neighbouring workgroups on the same rows of the
  // input and of the row-wise payload; down the rows first (in runs of 8 tiles per XCD, as in
  // mx_col_t_kernel) keeps them on the same rows of the transposed payload.  Measured, the first
  // is faster unless the matrix is much wider than tall (16384 x 4096 bf16: 50 vs 57 us; 4096 x
  // 16384: 53 vs 52 us; without the row-wise half the second wins from square on), so the host
  // picks by shape (cols_first: 1 = the first, 0 = the second, 2 = the banded order below, which is
  // 1-2 % ahead of the first where the row count is a multiple of 8 tiles: 8192 x 8192 bf16 46.8
  // against 47.2-47.8 us, fp32 67.1 against 67.7 us).
  const uint32_t row_tiles = (rows + kDualRows - 1) / kDualRows;
  const uint32_t col_tiles = (cols + kTileCols - 1) / kTileCols;
  const uint32_t ntiles = row_tiles * col_tiles;
  const uint32_t lrow0 = w * 32 + h * 16;                      // first of this lane's 16 rows inside the tile
  auto locate = [&](uint32_t t, uint32_t& tr, uint32_t& tc) {
    if (cols_first == 1) {
      tr = t / col_tiles;
      tc = t - tr * col_tiles;
    } else if (cols_first == 2 && row_tiles % 8 == 0) {
      // bands of 8 row tiles: inside a band 8 tiles down the rows, then on to the next column tile, so that
      // the workgroups in flight cover whole rows of x and still write 8 adjacent pieces of an output row
      if (t < (ntiles & ~63u)) {
        const uint32_t xcd = t & 7u, slot = t >> 3;
        t = (slot & ~7u) * 8u + xcd * 8u + (slot & 7u);
      }
      const uint32_t band = t / (8u * col_tiles), rem = t - band * 8u * col_tiles;
      tc = rem >> 3;
      tr = band * 8u + (rem & 7u);
    } else {
      if (t < (ntiles & ~63u)) {
        const uint32_t xcd = t & 7u, slot = t >> 3;
        t = (slot & ~7u) * 8u + xcd * 8u + (slot & 7u);
      }
      tc = t / row_tiles;
      tr = t - tc * row_tiles;
    }
  };
  auto load_tile = [&](uint32_t t, u32x4 (&dst)[16]) {
    uint32_t ltr, ltc;
    locate(t, ltr, ltc);
    const uint32_t lr0 = ltr * kDualRows + lrow0, lc0 = ltc * kTileCols + c8 * kV;
    if (t < ntiles && lr0 < rows && lc0 < cols) {
      const uint8_t* p = static_cast<const uint8_t*>(x) + ((uint64_t)lr0 * cols + lc0) * kB;
#pragma unroll
      for (int i = 0; i < 16; ++i) dst[i] = ld_x16<IN>(p + (uint64_t)i * cols * kB);
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) dst[i] = u32x4{0u, 0u, 0u, 0u};
    }
  };

  saturate_fp8_conversions();
  u32x4 v[16], vn[PIPE ? 16 : 1];
  if constexpr (PIPE) load_tile(blockIdx.x, vn);
  for (uint32_t tix = blockIdx.x; tix < ntiles; tix += gridDim.x) {  // tix: number of the tile in hand
  uint32_t tr, tc;
  locate(tix, tr, tc);
  const uint32_t row0 = tr * kDualRows + lrow0, col0 = tc * kTileCols + c8 * kV;
  const bool active = row0 < rows && col0 < cols;              // rows % 32 == 0 and cols % 32 == 0
  if constexpr (PIPE) {
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = vn[i];
    load_tile(tix + gridDim.x, vn);  // in flight under everything below
  } else {
    load_tile(tix, v);
  }

  // ---- blocks down the columns: maxima over this lane's 16 rows, then over both halves
  u32x4 pm = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if constexpr (IN == DT_F32) {
      pm.x = umax(pm.x, absbits_f32(v[i].x)); pm.y = umax(pm.y, absbits_f32(v[i].y));
      pm.z = umax(pm.z, absbits_f32(v[i].z)); pm.w = umax(pm.w, absbits_f32(v[i].w));
    } else {
      pm.x = pk_absmax16(pm.x, v[i].x); pm.y = pk_absmax16(pm.y, v[i].y);
      pm.z = pk_absmax16(pm.z, v[i].z); pm.w = pk_absmax16(pm.w, v[i].w);
    }
  }
  uint32_t cm[kV];
  if constexpr (IN == DT_F32) {
    cm[0] = other_half_max_u32(pm.x); cm[1] = other_half_max_u32(pm.y);
    cm[2] = other_half_max_u32(pm.z); cm[3] = other_half_max_u32(pm.w);
  } else {
    pm.x = other_half_max_pk16(pm.x); pm.y = other_half_max_pk16(pm.y);
    pm.z = other_half_max_pk16(pm.z); pm.w = other_half_max_pk16(pm.w);
    if constexpr (IN == DT_BF16) {
      cm[0] = pm.x << 16; cm[1] = pm.x & 0xFFFF0000u; cm[2] = pm.y << 16; cm[3] = pm.y & 0xFFFF0000u;
      cm[4] = pm.z << 16; cm[5] = pm.z & 0xFFFF0000u; cm[6] = pm.w << 16; cm[7] = pm.w & 0xFFFF0000u;
    } else {
      cm[0] = as_u32(f16_lo(pm.x)); cm[1] = as_u32(f16_hi(pm.x)); cm[2] = as_u32(f16_lo(pm.y)); cm[3] = as_u32(f16_hi(pm.y));
      cm[4] = as_u32(f16_lo(pm.z)); cm[5] = as_u32(f16_hi(pm.z)); cm[6] = as_u32(f16_lo(pm.w)); cm[7] = as_u32(f16_hi(pm.w));
    }
  }
  // the word that holds column c of row i (fp32: the element itself; 16-bit: it and its neighbour)
  auto word = [&](int i, int c) -> uint32_t {
    const int k = IN == DT_F32 ? c : c / 2;
    return k == 0 ? v[i].x : k == 1 ? v[i].y : k == 2 ? v[i].z : v[i].w;
  };
  const uint32_t chunk = (uint32_t)(w * 2 + h);
#pragma unroll
  for (int c = 0; c < kV; ++c) {
    const MxScale<OUT> s = mx_scale_from_absbits<OUT>(cm[c]);
    if constexpr (OUT == DT_E2M1) {
      // two rows of x per byte: the lane's 16 rows of a column are 8 bytes, the half h of the wave's
      // 16-byte chunk w of that column's 64 (byte j of a word = rows 8 q + 2 j in the low nibble, + 1 in the high)
      uint32_t r2[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        uint32_t r = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = 8 * q + 2 * j;
          if constexpr (IN == DT_F32) r = cvt_fp4_pair32(r, word(i, c), word(i + 1, c), s.scale, j);
          else r = cvt_fp4_pair16<IN>(r, gather_halves(c & 1, word(i, c), word(i + 1, c)), s.scale, j);
        }
        r2[q] = s.nan ? 0x77777777u : r;
      }
      const uint32_t col = (uint32_t)(c8 * kV + c);
      *reinterpret_cast<u32x2*>(tile + col * kDualPitch4 + ((((uint32_t)w) ^ ((col >> 4) & 3u)) << 4) + h * 8) = u32x2{r2[0], r2[1]};
      if (h == 0) reinterpret_cast<uint8_t*>(ctile)[col * 4 + w] = (uint8_t)(active ? s.byte : 0u);
      continue;
    }
    uint32_t r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if constexpr (IN == DT_F32)
        r[q] = cvt_scaled_4x32<OUT>(word(4 * q, c), word(4 * q + 1, c), word(4 * q + 2, c), word(4 * q + 3, c), s.scale);
      else
        r[q] = cvt_scaled_4x16<IN, OUT>(gather_halves(c & 1, word(4 * q, c), word(4 * q + 1, c)),
                                        gather_halves(c & 1, word(4 * q + 2, c), word(4 * q + 3, c)), s.scale);
      if (s.nan) r[q] = 0x7F7F7F7Fu;
    }
    const uint32_t col = (uint32_t)(c8 * kV + c);
    *reinterpret_cast<u32x4*>(tile + col * kDualPitch + ((chunk ^ ((col >> 4) & 7u)) << 4)) = u32x4{r[0], r[1], r[2], r[3]};
    if (h == 0) reinterpret_cast<uint8_t*>(ctile)[col * 4 + w] = (uint8_t)(active ? s.byte : 0u);
  }

  // ---- blocks along the rows: straight to memory
  uint32_t rb[4] = {0u, 0u, 0u, 0u};  // this lane's 16 row-scale bytes, rows in byte order
  uint8_t* drow = data_r + (uint64_t)row0 * cols + col0;
#pragma unroll
  for (int i = 0; i < (WITH_ROWS ? 16 : 0); ++i) {
    uint32_t m = quad_umax(vec_absmax_bits<IN>(v[i]));
    if constexpr (LPB == 8) m = umax(m, dpp<kDppRowHalfMirror>(m));
    const MxScale<OUT> s = mx_scale_from_absbits<OUT>(m);
    rb[i / 4] |= s.byte << (8 * (i % 4));
    if (active) {
      if constexpr (OUT == DT_E2M1) {
        // two columns per byte: a lane's kV columns leave as kV / 2 bytes of the row's cols / 2
        uint8_t* const d4 = data_r + (uint64_t)(row0 + i) * (cols / 2) + col0 / 2;
        if constexpr (IN == DT_F32) {
          const uint32_t r = cvt_fp4_4x32(v[i], s.scale);
          *reinterpret_cast<uint16_t*>(d4) = (uint16_t)(s.nan ? 0x7777u : r);
        } else {
          const uint32_t r = cvt_fp4_8x16<IN>(v[i], s.scale);
          st_stream(reinterpret_cast<uint32_t*>(d4), s.nan ? 0x77777777u : r);
        }
      } else if constexpr (IN == DT_F32) {
        const uint32_t r = cvt_scaled_4x32<OUT>(v[i].x, v[i].y, v[i].z, v[i].w, s.scale);
        st_stream(reinterpret_cast<uint32_t*>(drow + (uint64_t)i * cols), s.nan ? 0x7F7F7F7Fu : r);
      } else {
        u32x2 r;
        r.x = cvt_scaled_4x16<IN, OUT>(v[i].x, v[i].y, s.scale);
        r.y = cvt_scaled_4x16<IN, OUT>(v[i].z, v[i].w, s.scale);
        if (s.nan) r = u32x2{0x7F7F7F7Fu, 0x7F7F7F7Fu};
        st_stream(reinterpret_cast<u32x2*>(drow + (uint64_t)i * cols), r);
      }
    }
  }
  if (WITH_ROWS && (c8 % LPB) == 0)  // inactive lanes hold zero bytes: what the padding of the blocked layout must be
    *reinterpret_cast<u32x4*>(rtile + (c8 / LPB) * kDualRows + lrow0) = u32x4{rb[0], rb[1], rb[2], rb[3]};
  __syncthreads();

  // ---- transposed payload: kTileCols output rows (columns of x) x 8 chunks of 16 bytes
  const uint32_t trow0 = tr * kDualRows, tcol0 = tc * kTileCols;
  if constexpr (OUT == DT_E2M1) {  // 4 chunks of 16 bytes (32 rows of x each) per output row of rows / 2 bytes
#pragma unroll
    for (int i = 0; i < kTileCols * 4 / kBlock; ++i) {
      const uint32_t id = tid + i * kBlock, r = id >> 2, q = id & 3;
      if (tcol0 + r < cols && trow0 + q * 32 < rows) {
        const u32x4 o = *reinterpret_cast<const u32x4*>(tile + r * kDualPitch4 + ((q ^ ((r >> 4) & 3u)) << 4));
        *reinterpret_cast<u32x4*>(data_c + (uint64_t)(tcol0 + r) * (rows / 2) + trow0 / 2 + q * 16) = o;
      }
    }
  } else {
#pragma unroll
  for (int i = 0; i < kTileCols * 8 / kBlock; ++i) {
    const uint32_t id = tid + i * kBlock, r = id >> 3, q = id & 7;
    if (tcol0 + r < cols && trow0 + q * 16 < rows) {
      const u32x4 o = *reinterpret_cast<const u32x4*>(tile + r * kDualPitch + ((q ^ ((r >> 4) & 7u)) << 4));
      // a plain store: these 128-byte pieces arrive in the order that walks down the output's rows, where
      // write-back from L2 beats streaming stores (8192 x 8192 bf16: 47.4 vs 54.1 us for the kernel)
      *reinterpret_cast<u32x4*>(data_c + (uint64_t)(tcol0 + r) * rows + trow0 + q * 16) = o;
    }
  }
  }
  // ---- column-block scales [cols, rows/32]: 4 bytes per column of this tile
  const uint32_t RB = rows / 32, rb0 = tr * 4;
  if (tid < kTileCols && tcol0 + tid < cols) {
    const uint32_t sw = ctile[tid];
    const uint32_t c = tcol0 + tid;
    if (LAYOUT == DT_SCALE_BLOCKED || (RB % 4 == 0)) {
      *reinterpret_cast<uint32_t*>(scale_c + scale_offset<LAYOUT>(c, rb0, RB)) = sw;
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (rb0 + k < RB) scale_c[scale_offset<LAYOUT>(c, rb0 + k, RB)] = (uint8_t)(sw >> (8 * k));
    }
  }
  // ---- row-block scales [rows, cols/32]: kRowBlocks bytes per row of this tile
  const uint32_t KB = cols / 32, kb0 = tc * kRowBlocks;
  if (WITH_ROWS && tid < kDualRows && trow0 + tid < rows) {
    const uint32_t r = trow0 + tid;
#pragma unroll
    for (int g = 0; g < kRowBlocks / 4; ++g) {
      uint32_t sw = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) sw |= (uint32_t)rtile[(4 * g + k) * kDualRows + tid] << (8 * k);
      const uint32_t c = kb0 + 4 * g;
      if (c >= KB) continue;
      if (LAYOUT == DT_SCALE_BLOCKED || (KB % 4 == 0)) {
        *reinterpret_cast<uint32_t*>(scale_r + scale_offset<LAYOUT>(r, c, KB)) = sw;
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (c + k < KB) scale_r[scale_offset<LAYOUT>(r, c + k, KB)] = (uint8_t)(sw >> (8 * k));
      }
    }
  }
  if (tix + gridDim.x < ntiles) __syncthreads();  // the LDS tiles are written again
  }  // tile loop
}

// ----------------------------------------- blocks along rows, transposed payload
// (axis 1, transpose): the row-wise cast written as [cols, rows], scales [cols/32, rows].  The
// geometry of mx_dual_kernel: a workgroup owns 128 rows x 32*kV columns, a lane 16 rows x kV adjacent
// columns, which lie in one row-direction block.  Row-block maxima over the neighbouring lanes; the
// payload is converted four rows of one column at a time (four different scales per word) into the
// same swizzled LDS tile [column][128 rows] and leaves as 128-byte rows; the scale bytes leave as
// kRowBlocks runs of 128 bytes.  Tiles are numbered down the rows first, so that neighbouring
// workgroups write adjacent pieces of the same output rows.  rows % 16 == 0.
template <int IN, int OUT>
__global__ __launch_bounds__(kBlock) void mx_row_t_kernel(const void* __restrict__ x, uint32_t rows, uint32_t cols,
                                                          uint8_t* __restrict__ data, uint8_t* __restrict__ scale) {
  constexpr int kV = InTraits<IN>::kVec;
  constexpr int kB = InTraits<IN>::kBytes;
  constexpr int kTileCols = 32 * kV;
  constexpr int kRowBlocks = kTileCols / 32;
  constexpr int LPB = 32 / kV;
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileCols * kDualPitch];
  __shared__ __attribute__((aligned(16))) uint8_t rtile[kRowBlocks * kDualRows];  // [block][row]
  const int tid = threadIdx.x, lane = tid % kWave, w = tid / kWave, h = lane >> 5, c8 = lane & 31;
  const uint32_t row_tiles = (rows + kDualRows - 1) / kDualRows;
  const uint32_t tc = blockIdx.x / row_tiles, tr = blockIdx.x - tc * row_tiles;
  const uint32_t lrow0 = w * 32 + h * 16;
  const uint32_t row0 = tr * kDualRows + lrow0, col0 = tc * kTileCols + c8 * kV;
  const bool active = row0 < rows && col0 < cols;  // rows % 16 == 0 and cols % 32 == 0: all of a lane or none

  saturate_fp8_conversions();
  u32x4 v[16];
  if (active) {
    const uint8_t* p = static_cast<const uint8_t*>(x) + ((uint64_t)row0 * cols + col0) * kB;
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = ld_x16<IN>(p + (uint64_t)i * cols * kB);
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = u32x4{0u, 0u, 0u, 0u};
  }
  float sc[16];
  uint32_t rb[4] = {0u, 0u, 0u, 0u}, nanmask[4] = {0u, 0u, 0u, 0u};  // per row: scale byte, 0xFF where the block holds a NaN
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    uint32_t m = quad_umax(vec_absmax_bits<IN>(v[i]));
    if constexpr (LPB == 8) m = umax(m, dpp<kDppRowHalfMirror>(m));
    const MxScale<OUT> s = mx_scale_from_absbits<OUT>(m);
    sc[i] = s.scale;
    rb[i / 4] |= s.byte << (8 * (i % 4));
    nanmask[i / 4] |= s.nan ? (0xFFu << (8 * (i % 4))) : 0u;
  }
  auto word = [&](int i, int c) -> uint32_t {
    const int k = IN == DT_F32 ? c : c / 2;
    return k == 0 ? v[i].x : k == 1 ? v[i].y : k == 2 ? v[i].z : v[i].w;
  };
  const uint32_t chunk = (uint32_t)(w * 2 + h);
#pragma unroll
  for (int c = 0; c < kV; ++c) {
    uint32_t r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if constexpr (IN == DT_F32)
        r[q] = cvt_scaled_4x32_each<OUT>(word(4 * q, c), word(4 * q + 1, c), word(4 * q + 2, c), word(4 * q + 3, c), sc + 4 * q);
      else
        r[q] = cvt_scaled_4x16_each<IN, OUT>(gather_halves(c & 1, word(4 * q, c), word(4 * q + 1, c)),
                                             gather_halves(c & 1, word(4 * q + 2, c), word(4 * q + 3, c)), sc + 4 * q);
      r[q] = (r[q] & ~nanmask[q]) | (0x7F7F7F7Fu & nanmask[q]);
    }
    const uint32_t col = (uint32_t)(c8 * kV + c);
    *reinterpret_cast<u32x4*>(tile + col * kDualPitch + ((chunk ^ ((col >> 4) & 7u)) << 4)) = u32x4{r[0], r[1], r[2], r[3]};
  }
  if ((c8 % LPB) == 0) *reinterpret_cast<u32x4*>(rtile + (c8 / LPB) * kDualRows + lrow0) = u32x4{rb[0], rb[1], rb[2], rb[3]};
  __syncthreads();

  const uint32_t trow0 = tr * kDualRows, tcol0 = tc * kTileCols;
#pragma unroll
  for (int i = 0; i < kTileCols * 8 / kBlock; ++i) {
    const uint32_t id = tid + i * kBlock, r = id >> 3, q = id & 7;
    if (tcol0 + r < cols && trow0 + q * 16 < rows) {
      const u32x4 o = *reinterpret_cast<const u32x4*>(tile + r * kDualPitch + ((q ^ ((r >> 4) & 7u)) << 4));
      st_stream(reinterpret_cast<u32x4*>(data + (uint64_t)(tcol0 + r) * rows + trow0 + q * 16), o);
    }
  }
  // scales [cols/32, rows]: for each of the tile's row-direction blocks the bytes of its 128 rows
  if (tid < kRowBlocks * 32) {
    const uint32_t g = tid >> 5, r4 = (tid & 31) * 4, kb = tc * kRowBlocks + g;
    if (kb < cols / 32 && trow0 + r4 < rows)
      *reinterpret_cast<uint32_t*>(scale + (uint64_t)kb * rows + trow0 + r4) = *reinterpret_cast<const uint32_t*>(rtile + g * kDualRows + r4);
  }
}

// ----------------------------------------------------------------- any orientation ---
// One thread per 32-element block with explicit strides (in elements / bytes).
template <int IN, int OUT, int LAYOUT>
__global__ __launch_bounds__(kBlock) void mx_any_kernel(const void* __restrict__ x, int64_t outer, int64_t inner_blocks,
                                                        int64_t x_outer_stride, int64_t x_elem_stride,
                                                        int64_t d_outer_stride, int64_t d_elem_stride,
                                                        int64_t s_rows, int64_t s_cols, int s_transposed,
                                                        uint8_t* __restrict__ data, uint8_t* __restrict__ scale) {
  const int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (g >= outer * inner_blocks) return;
  const int64_t o = g / inner_blocks, b = g - o * inner_blocks;
  const int64_t xfirst = o * x_outer_stride + b * 32 * x_elem_stride;
  uint32_t m = 0;
  for (int i = 0; i < 32; ++i) m = umax(m, absbits_f32(as_u32(load_elem<IN>(x, xfirst + i * x_elem_stride))));
  const MxScale<OUT> s = mx_scale_from_absbits<OUT>(m);
  const int64_t dfirst = o * d_outer_stride + b * 32 * d_elem_stride;
  for (int i = 0; i < 32; ++i) {
    const float p = load_elem<IN>(x, xfirst + i * x_elem_stride) * s.mult;
    const uint32_t code = pack4_finite<OUT>(p, 0.f, 0.f, 0.f) & 0xFFu;
    data[dfirst + i * d_elem_stride] = s.nan ? (uint8_t)0x7F : (uint8_t)code;
  }
  // the scale matrix is [outer, inner_blocks], stored transposed when s_transposed
  const int64_t sr = s_transposed ? b : o, scol = s_transposed ? o : b;
  scale[scale_offset<LAYOUT>(sr, scol, s_cols)] = (uint8_t)s.byte;
  (void)s_rows;
}

__global__ void fill_bytes_kernel(uint8_t* p, int64_t n, uint8_t value) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = value;
}

// plain [R, C] scale matrix -> blocked layout (padding already zeroed by the caller)
__global__ void to_blocked_kernel(const uint8_t* __restrict__ in, int64_t R, int64_t C, uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= R * C) return;
  const int64_t r = i / C, c = i - r * C;
  out[blocked_offset(r, c, (C + 3) >> 2)] = in[i];
}

}  // namespace dt
