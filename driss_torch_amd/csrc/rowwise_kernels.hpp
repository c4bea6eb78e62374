// Row-wise dynamic quantization: per-row amax -> scale -> saturating fp8 cast.
//
// Fast path: one wavefront owns one row and keeps it in registers between the reduction
// and the cast, so the row is read from memory once; no LDS and no barrier is involved.
// Rows too long for that use one workgroup per row and read the row twice (the second
// read hits cache); rows that are not 16-byte aligned use the scalar kernel.
#pragma once

#include "quant_kernels.hpp"

namespace dt {

constexpr int kRowsPerBlock = kBlock / kWave;  // one wave per row

template <int IN, int OUT, int NV>
__global__ __launch_bounds__(kBlock) void rowwise_wave_kernel(const void* __restrict__ x, int64_t rows,
                                                              int row_vecs, uint8_t* __restrict__ out,
                                                              float* __restrict__ amax_out,
                                                              float* __restrict__ scale_out) {
  constexpr int kV = InTraits<IN>::kVec;
  saturate_fp8_conversions();
  const int lane = threadIdx.x % kWave;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row >= rows) return;  // whole wave leaves together; the kernel has no barrier
  const u32x4* v = static_cast<const u32x4*>(x) + row * row_vecs;
  u32x4 w[NV];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int j = lane + u * kWave;
    w[u] = j < row_vecs ? ld_stream(v + j) : u32x4{0u, 0u, 0u, 0u};
  }
  uint32_t m = 0;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    if constexpr (IN == DT_F32) {
      m = umax(m, umax(umax(absbits_f32(w[u].x), absbits_f32(w[u].y)), umax(absbits_f32(w[u].z), absbits_f32(w[u].w))));
    } else {
      m = pk_absmax16(pk_absmax16(m, w[u].x), w[u].y);
      m = pk_absmax16(pk_absmax16(m, w[u].z), w[u].w);
    }
  }
  if constexpr (IN != DT_F32) m = umax(m & 0xFFFFu, m >> 16) << 16;
  m = wave_umax(m);
  const float amax = as_f32(m);
  const float s = amax_to_scale(amax, fp8_max<OUT>());
  uint8_t* orow = out + row * (int64_t)row_vecs * kV;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int j = lane + u * kWave;
    if (j < row_vecs) cast_vec<IN, OUT, false>(w[u], s, orow, j);
  }
  if (lane == 0) {
    if (amax_out) amax_out[row] = amax;
    if (scale_out) scale_out[row] = s;
  }
}

// Longer rows: one workgroup per row, NV vectors per lane kept in registers between the reduction
// (one LDS exchange between the four waves) and the cast: still a single read of the row.
// ANY: rows that are not 16-byte aligned or not a whole number of vectors (cols % kV = tail elements,
// done by the first lanes): the same loads and stores through vector types that claim only element /
// byte alignment, as in cast_kernel_unaligned.
template <int IN, int OUT, int NV, bool ANY = false>
__global__ __launch_bounds__(kBlock) void rowwise_block_resident_kernel(const void* __restrict__ x, int row_vecs,
                                                                        uint8_t* __restrict__ out,
                                                                        float* __restrict__ amax_out,
                                                                        float* __restrict__ scale_out, int tail = 0) {
  constexpr int kV = InTraits<IN>::kVec, kB = InTraits<IN>::kBytes;
  saturate_fp8_conversions();
  __shared__ uint32_t lds[kBlock / kWave];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int64_t cols = (int64_t)row_vecs * kV + tail;
  const uint8_t* xrow = static_cast<const uint8_t*>(x) + row * cols * kB;
  u32x4 w[NV];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int j = tid + u * kBlock;
    if constexpr (ANY) {
      typedef typename std::conditional<IN == DT_F32, u32x4_elem4, u32x4_elem2>::type vec_t;
      w[u] = j < row_vecs ? reinterpret_cast<const vec_t*>(xrow)[j] : u32x4{0u, 0u, 0u, 0u};
    } else {
      w[u] = j < row_vecs ? ld_stream(reinterpret_cast<const u32x4*>(xrow) + j) : u32x4{0u, 0u, 0u, 0u};
    }
  }
  uint32_t m = 0;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    if constexpr (IN == DT_F32) {
      m = umax(m, umax(umax(absbits_f32(w[u].x), absbits_f32(w[u].y)), umax(absbits_f32(w[u].z), absbits_f32(w[u].w))));
    } else {
      m = pk_absmax16(pk_absmax16(m, w[u].x), w[u].y);
      m = pk_absmax16(pk_absmax16(m, w[u].z), w[u].w);
    }
  }
  if constexpr (IN != DT_F32) m = umax(m & 0xFFFFu, m >> 16) << 16;
  if constexpr (ANY) {
    if (tid < tail) m = umax(m, absbits_of<IN>(xrow, (int64_t)row_vecs * kV + tid));
  }
  m = block_umax<kBlock / kWave>(m, lds);
  const float amax = as_f32(m);
  const float s = amax_to_scale(amax, fp8_max<OUT>());
  uint8_t* orow = out + row * cols;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int j = tid + u * kBlock;
    if (j < row_vecs) {
      if constexpr (ANY) {
        uint32_t r[kV / 4];
        cast_vec_to_words<IN, OUT, false>(w[u], s, r);
        if constexpr (IN == DT_F32) *reinterpret_cast<u32_byte*>(orow + (int64_t)j * 4) = r[0];
        else *reinterpret_cast<u32x2_byte*>(orow + (int64_t)j * 8) = u32x2{r[0], r[1]};
      } else {
        cast_vec<IN, OUT, false>(w[u], s, orow, j);
      }
    }
  }
  if constexpr (ANY) {
    if (tid < tail) orow[(int64_t)row_vecs * kV + tid] = cast_one<IN, OUT, false>(xrow, (int64_t)row_vecs * kV + tid, s);
  }
  if (tid == 0) {
    if (amax_out) amax_out[row] = amax;
    if (scale_out) scale_out[row] = s;
  }
}

// One workgroup per row; VEC selects 16-byte access (aligned rows) or element access.
template <int IN, int OUT, bool VEC>
__global__ __launch_bounds__(kBlock) void rowwise_block_kernel(const void* __restrict__ x, int64_t cols,
                                                               uint8_t* __restrict__ out,
                                                               float* __restrict__ amax_out,
                                                               float* __restrict__ scale_out) {
  constexpr int kB = InTraits<IN>::kBytes, kV = InTraits<IN>::kVec;
  saturate_fp8_conversions();
  __shared__ uint32_t lds[kBlock / kWave];
  const int64_t row = blockIdx.x;
  const uint8_t* xrow = static_cast<const uint8_t*>(x) + row * cols * kB;
  uint8_t* orow = out + row * cols;
  const int tid = threadIdx.x;
  uint32_t m = 0;
  if constexpr (VEC) {
    const u32x4* v = reinterpret_cast<const u32x4*>(xrow);
    for (int64_t j = tid; j < cols / kV; j += kBlock) {
      u32x4 w = v[j];
      if constexpr (IN == DT_F32) {
        m = umax(m, umax(umax(absbits_f32(w.x), absbits_f32(w.y)), umax(absbits_f32(w.z), absbits_f32(w.w))));
      } else {
        uint32_t p = pk_absmax16(pk_absmax16(pk_absmax16(pk_absmax16(0u, w.x), w.y), w.z), w.w);
        m = umax(m, umax(p & 0xFFFFu, p >> 16) << 16);
      }
    }
  } else {
    for (int64_t j = tid; j < cols; j += kBlock) m = umax(m, absbits_of<IN>(xrow, j));
  }
  m = block_umax<kBlock / kWave>(m, lds);
  const float amax = as_f32(m);
  const float s = amax_to_scale(amax, fp8_max<OUT>());
  if constexpr (VEC) {
    const u32x4* v = reinterpret_cast<const u32x4*>(xrow);
    for (int64_t j = tid; j < cols / kV; j += kBlock) cast_vec<IN, OUT, false>(v[j], s, orow, j);
  } else {
    for (int64_t j = tid; j < cols; j += kBlock) orow[j] = cast_one<IN, OUT, false>(xrow, j, s);
  }
  if (tid == 0) {
    if (amax_out) amax_out[row] = amax;
    if (scale_out) scale_out[row] = s;
  }
}

template <int IN, int OUT>
inline int launch_rowwise_impl(const void* x, int64_t rows, int64_t cols, void* out, float* amax_out,
                               float* scale_out, hipStream_t stream) {
  constexpr int kV = InTraits<IN>::kVec;
  constexpr size_t kStoreAlign = IN == DT_F32 ? 4 : 8;
  uint8_t* o = static_cast<uint8_t*>(out);
  const bool vec_ok = aligned(x, 16) && aligned(out, kStoreAlign) && cols % kV == 0;
  const int64_t row_vecs = cols / kV;
  const int64_t block_from = tuning("rowwise.block_from_vecs");  // rows at least this long take a workgroup each
  if (vec_ok && row_vecs >= block_from && row_vecs <= 64 * kBlock && rows <= 0x7FFFFFFFll) {
    const int rv = (int)row_vecs;
#define DT_ROWB(NV) \
  rowwise_block_resident_kernel<IN, OUT, NV><<<(unsigned)rows, kBlock, 0, stream>>>(x, rv, o, amax_out, scale_out)
    if (row_vecs <= 1 * kBlock) DT_ROWB(1);
    else if (row_vecs <= 2 * kBlock) DT_ROWB(2);
    else if (row_vecs <= 4 * kBlock) DT_ROWB(4);
    else if (row_vecs <= 8 * kBlock) DT_ROWB(8);
    else if (row_vecs <= 16 * kBlock) DT_ROWB(16);
    else if (row_vecs <= 32 * kBlock) DT_ROWB(32);
    else DT_ROWB(64);
#undef DT_ROWB
  } else if (!vec_ok && row_vecs >= 1 && row_vecs <= 64 * kBlock && rows <= 0x7FFFFFFFll) {
    // rows that are not aligned or not whole vectors: a workgroup per row with element-aligned vector accesses
    const int rv = (int)row_vecs, tail = (int)(cols % kV);
#define DT_ROWA(NV) \
  rowwise_block_resident_kernel<IN, OUT, NV, true><<<(unsigned)rows, kBlock, 0, stream>>>(x, rv, o, amax_out, scale_out, tail)
    if (row_vecs <= 1 * kBlock) DT_ROWA(1);
    else if (row_vecs <= 2 * kBlock) DT_ROWA(2);
    else if (row_vecs <= 4 * kBlock) DT_ROWA(4);
    else if (row_vecs <= 8 * kBlock) DT_ROWA(8);
    else if (row_vecs <= 16 * kBlock) DT_ROWA(16);
    else if (row_vecs <= 32 * kBlock) DT_ROWA(32);
    else DT_ROWA(64);
#undef DT_ROWA
  } else if (vec_ok && row_vecs <= 16 * kWave) {
    const unsigned grid = (unsigned)ceil_div(rows, kRowsPerBlock);
    const int rv = (int)row_vecs;
#define DT_ROW(NV) rowwise_wave_kernel<IN, OUT, NV><<<grid, kBlock, 0, stream>>>(x, rows, rv, o, amax_out, scale_out)
    if (row_vecs <= 1 * kWave) DT_ROW(1);
    else if (row_vecs <= 2 * kWave) DT_ROW(2);
    else if (row_vecs <= 4 * kWave) DT_ROW(4);
    else if (row_vecs <= 8 * kWave) DT_ROW(8);
    else DT_ROW(16);
#undef DT_ROW
  } else if (vec_ok) {
    rowwise_block_kernel<IN, OUT, true><<<(unsigned)rows, kBlock, 0, stream>>>(x, cols, o, amax_out, scale_out);
  } else {
    rowwise_block_kernel<IN, OUT, false><<<(unsigned)rows, kBlock, 0, stream>>>(x, cols, o, amax_out, scale_out);
  }
  return launch_status();
}

inline int launch_rowwise(const void* x, int in_dtype, int64_t rows, int64_t cols, int out_dtype, void* out,
                          float* amax_out, float* scale_out, hipStream_t stream) {
  if (rows > 0x7FFFFFFFll) return DT_ERR_INVALID_SHAPE;
  if (in_dtype == DT_F32) {
    if (out_dtype == DT_E4M3FN) return launch_rowwise_impl<DT_F32, DT_E4M3FN>(x, rows, cols, out, amax_out, scale_out, stream);
    return launch_rowwise_impl<DT_F32, DT_E5M2>(x, rows, cols, out, amax_out, scale_out, stream);
  }
  if (out_dtype == DT_E4M3FN) return launch_rowwise_impl<DT_BF16, DT_E4M3FN>(x, rows, cols, out, amax_out, scale_out, stream);
  return launch_rowwise_impl<DT_BF16, DT_E5M2>(x, rows, cols, out, amax_out, scale_out, stream);
}

}  // namespace dt
