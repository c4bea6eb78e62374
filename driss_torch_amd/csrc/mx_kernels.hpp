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
  float mult;
  bool nan;
};
template <int OUT>
__device__ __forceinline__ MxScale<OUT> mx_scale_from_absbits(uint32_t absbits) {
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
  return r;
}

// saturating convert without the NaN patch (NaN blocks are overwritten wholesale)
template <int OUT>
__device__ __forceinline__ uint32_t pack4_finite(float p0, float p1, float p2, float p3) {
  uint32_t w = cvt_pk<OUT, false>(clamp_fp8<OUT>(p0), clamp_fp8<OUT>(p1), 0u);
  return cvt_pk<OUT, true>(clamp_fp8<OUT>(p2), clamp_fp8<OUT>(p3), w);
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

// ------------------------------------------------------------------ blocks along rows
// The matrix is a flat run of 32-element blocks.  One wave pass ("super-chunk") covers 64
// blocks as LPB chunks of 64 vectors; lane l ends up holding the scale byte of chunk
// l % LPB, block l / LPB, so the 64 scale bytes leave in a single store instruction.
template <int IN, int OUT, int LAYOUT>
__global__ __launch_bounds__(kBlock) void mx_row_kernel(const void* __restrict__ x, uint32_t nblocks,
                                                        uint32_t kblocks, uint8_t* __restrict__ data,
                                                        uint8_t* __restrict__ scale) {
  constexpr int kV = InTraits<IN>::kVec;      // elements per vector
  constexpr int LPB = 32 / kV;                // lanes per block: 4 or 8
  constexpr int BPC = kWave / LPB;            // blocks per chunk: 16 or 8
  const int lane = threadIdx.x % kWave;
  const uint32_t nvec = nblocks * LPB;
  const u32x4* v = static_cast<const u32x4*>(x);
  const uint32_t nsuper = (nblocks + 63u) / 64u;
  const uint32_t wave_id = (blockIdx.x * kBlock + threadIdx.x) / kWave;
  const uint32_t nwaves = gridDim.x * (kBlock / kWave);

  for (uint32_t sc = wave_id; sc < nsuper; sc += nwaves) {
    const uint32_t vbase = sc * 64u * LPB + lane;
    u32x4 w[LPB];
#pragma unroll
    for (int c = 0; c < LPB; ++c) {
      const uint32_t vi = vbase + c * kWave;
      w[c] = vi < nvec ? ld_stream(v + vi) : u32x4{0u, 0u, 0u, 0u};
    }
    uint32_t mybyte = 0;
#pragma unroll
    for (int c = 0; c < LPB; ++c) {
      const uint32_t vi = vbase + c * kWave;
      uint32_t m = quad_umax(vec_absmax_bits<IN>(w[c]));
      if constexpr (LPB == 8) m = umax(m, dpp<kDppRowHalfMirror>(m));
      const MxScale<OUT> s = mx_scale_from_absbits<OUT>(m);
      if ((lane % LPB) == c) mybyte = s.byte;
      if (vi < nvec) {
        if constexpr (IN == DT_F32) {
          uint32_t r = pack4_finite<OUT>(as_f32(w[c].x) * s.mult, as_f32(w[c].y) * s.mult, as_f32(w[c].z) * s.mult,
                                         as_f32(w[c].w) * s.mult);
          st_stream(reinterpret_cast<uint32_t*>(data) + vi, s.nan ? 0x7F7F7F7Fu : r);
        } else {
          float f[8];
          unpack8<IN>(w[c], f);
          u32x2 r;
          r.x = pack4_finite<OUT>(f[0] * s.mult, f[1] * s.mult, f[2] * s.mult, f[3] * s.mult);
          r.y = pack4_finite<OUT>(f[4] * s.mult, f[5] * s.mult, f[6] * s.mult, f[7] * s.mult);
          if (s.nan) r = u32x2{0x7F7F7F7Fu, 0x7F7F7F7Fu};
          st_stream(reinterpret_cast<u32x2*>(data) + vi, r);
        }
      }
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
      for (int i = 0; i < 8; ++i) v[i] = ld_stream(reinterpret_cast<const u32x4*>(p + i * pitch));
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
    float mult[kV];
    uint32_t nanmask[kW] = {};
    uint32_t bytes[kW] = {};  // the kV scale bytes packed in column order
#pragma unroll
    for (int c = 0; c < kV; ++c) {
      const MxScale<OUT> sc = mx_scale_from_absbits<OUT>(cm[c]);
      mult[c] = sc.mult;
      bytes[c / 4] |= sc.byte << (8 * (c % 4));
      nanmask[c / 4] |= sc.nan ? (0xFFu << (8 * (c % 4))) : 0u;
    }
    if (col0 < cols) {
      uint8_t* drow = data + (uint64_t)(tr * 32u + w * 8u) * cols + col0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float f[8];
        if constexpr (IN == DT_F32) {
          f[0] = as_f32(v[i].x); f[1] = as_f32(v[i].y); f[2] = as_f32(v[i].z); f[3] = as_f32(v[i].w);
        } else {
          unpack8<IN>(v[i], f);
        }
        uint32_t r[kW];
#pragma unroll
        for (int q = 0; q < kW; ++q) {
          r[q] = pack4_finite<OUT>(f[4 * q] * mult[4 * q], f[4 * q + 1] * mult[4 * q + 1], f[4 * q + 2] * mult[4 * q + 2],
                                   f[4 * q + 3] * mult[4 * q + 3]);
          r[q] = (r[q] & ~nanmask[q]) | (0x7F7F7F7Fu & nanmask[q]);
        }
        if constexpr (kW == 2) st_stream(reinterpret_cast<u32x2*>(drow + (uint64_t)i * cols), u32x2{r[0], r[1]});
        else st_stream(reinterpret_cast<uint32_t*>(drow + (uint64_t)i * cols), r[0]);
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

  uint32_t sbyte[4] = {0, 0, 0, 0};
  if (active) {
    // 32 rows x 4 columns kept packed as loaded: fp32 -> one 16-byte load per row, 16-bit -> one
    // 8-byte load; elements are unpacked where they are used
    typedef typename std::conditional<IN == DT_F32, u32x4, u32x2>::type row_t;
    row_t wv[32];
    uint32_t cm[4] = {0, 0, 0, 0};
    const uint8_t* p = static_cast<const uint8_t*>(x) + ((uint64_t)row0 * cols + col0) * kB;
#pragma unroll
    for (int i = 0; i < 32; ++i) wv[i] = ld_stream(reinterpret_cast<const row_t*>(p + (uint64_t)i * cols * kB));
    auto elem = [&](int i, int c) -> float {
      if constexpr (IN == DT_F32) {
        return as_f32(c == 0 ? wv[i].x : c == 1 ? wv[i].y : c == 2 ? wv[i].z : wv[i].w);
      } else {
        const uint32_t d = c < 2 ? wv[i].x : wv[i].y;
        if constexpr (IN == DT_BF16) return (c & 1) ? bf16_hi(d) : bf16_lo(d);
        else return (c & 1) ? f16_hi(d) : f16_lo(d);
      }
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
      uint32_t r[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        r[q] = pack4_finite<OUT>(elem(4 * q, c) * s.mult, elem(4 * q + 1, c) * s.mult, elem(4 * q + 2, c) * s.mult,
                                 elem(4 * q + 3, c) * s.mult);
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
#pragma unroll
  for (int i = 0; i < kColTCols * 8 / kBlock; ++i) {
    const int id = tid + i * kBlock, r = id >> 3, q = id & 7;
    if (tcol0 + r < cols && trow0 + q * 16 < rows) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(tile + r * kColTPitch + q * 16);
      st_stream(reinterpret_cast<u32x4*>(data + (uint64_t)(tcol0 + r) * rows + trow0 + q * 16), v);
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
