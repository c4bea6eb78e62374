// dt_mx_fp8_quantize / dt_to_blocked: MXFP8 cast with E8M0 block-32 scales (C ABI).
#include "mx_kernels.hpp"

namespace {
using namespace dt;

struct MxArgs {
  const void* x;
  int64_t rows, cols;
  int axis, transpose;
  uint8_t* data;
  uint8_t* scale;
  hipStream_t stream;
};

template <int IN, int OUT, int LAYOUT>
int launch_mx(const MxArgs& a) {
  constexpr int kV = InTraits<IN>::kVec;
  const int64_t numel = a.rows * a.cols, nblocks = numel / 32;
  const int cus = device_facts().cu_count;
  // x only has to be aligned to its element: the kernels load it through element-aligned vector types
  if (a.axis == 1 && !a.transpose && aligned(a.data, 8) && nblocks < (1ll << 28)) {
    const int64_t nsuper = ceil_div(nblocks, 64);
    int64_t waves = (int64_t)cus * tuning("mx.blocks_per_cu") * (kBlock / kWave);
    if (waves > nsuper) waves = nsuper;
    const unsigned grid = (unsigned)ceil_div(waves, kBlock / kWave);
    if constexpr (LAYOUT == DT_SCALE_BLOCKED) {
      if (a.rows % 128 == 0 && a.cols % 512 == 0 && tuning("mx.row_band4")) {
        mx_row_kernel<IN, OUT, LAYOUT, true><<<grid, kBlock, 0, a.stream>>>(a.x, (uint32_t)nblocks, (uint32_t)(a.cols / 32),
                                                                           a.data, a.scale);
        return launch_status();
      }
    }
    mx_row_kernel<IN, OUT, LAYOUT><<<grid, kBlock, 0, a.stream>>>(a.x, (uint32_t)nblocks, (uint32_t)(a.cols / 32),
                                                                 a.data, a.scale);
    return launch_status();
  }
  // Transposed column cast: the one-read kernel without its row-wise half (16-byte loads, half-wave
  // row split) wherever a lane's kV columns are whole; 8192 x 8192 bf16 38.3 vs 40.2 us for
  // mx_col_t_kernel, 16384 x 4096 36.3 vs 41.0 us.  Tile order: bands of 8 row tiles where the row count
  // allows (8192 x 8192 bf16: 36.6-37.1 us against 38.0-38.6 down the rows first), else by shape.
  if (a.axis == 0 && a.transpose && a.cols % kV == 0 && aligned(a.data, 16) && aligned(a.scale, 4) &&
      a.rows < (1ll << 31) && a.cols < (1ll << 31) && tuning("mx.colt_via_dual")) {
    constexpr int kTileCols = 32 * kV;
    const int64_t tiles = ceil_div(a.rows, (int64_t)kDualRows) * ceil_div(a.cols, (int64_t)kTileCols);
    if (tiles <= 0x7FFFFFFFll) {
      const int order = tuning("mx.dual_order") >= 0 ? tuning("mx.dual_order") : (a.rows % (8 * kDualRows) == 0 ? 2 : (a.cols < a.rows ? 1 : 0));
      // A grid of mx.colt_pipe workgroups per CU that walk the tiles with the next tile's loads in flight:
      // 8192 x 8192 bf16 36.4 against 37.5 us, 4096 x 16384 37.1 against 39.2 us, fp32 and 16384 x 4096 the same
      // (with the row-wise half as well it is slower: 48.3 against 47.8 us)
      const int64_t pipe_grid = (int64_t)tuning("mx.colt_pipe") * device_facts().cu_count;
      if (pipe_grid > 0 && tiles > pipe_grid)
        mx_dual_kernel<IN, OUT, LAYOUT, false, true><<<(unsigned)pipe_grid, kBlock, 0, a.stream>>>(
            a.x, (uint32_t)a.rows, (uint32_t)a.cols, nullptr, nullptr, a.data, a.scale, order);
      else
        mx_dual_kernel<IN, OUT, LAYOUT, false><<<(unsigned)tiles, kBlock, 0, a.stream>>>(
            a.x, (uint32_t)a.rows, (uint32_t)a.cols, nullptr, nullptr, a.data, a.scale, order);
      return launch_status();
    }
  }
  if (a.axis == 0 && a.transpose && a.cols % 4 == 0 && aligned(a.data, 16) && aligned(a.scale, 4) &&
      a.rows < (1ll << 31) && a.cols < (1ll << 31)) {
    const int64_t tiles = ceil_div(a.rows, (int64_t)kColTRows) * ceil_div(a.cols, (int64_t)kColTCols);
    if (tiles <= 0x7FFFFFFFll) {
      mx_col_t_kernel<IN, OUT, LAYOUT><<<(unsigned)tiles, kBlock, 0, a.stream>>>(a.x, (uint32_t)a.rows, (uint32_t)a.cols,
                                                                              a.data, a.scale);
      return launch_status();
    }
  }
  if (a.axis == 0 && !a.transpose && a.cols % kV == 0 && aligned(a.data, 16) && aligned(a.scale, 8) &&
      a.rows < (1ll << 31) && a.cols < (1ll << 31) && LAYOUT == DT_SCALE_PLAIN) {
    const int64_t tiles = (a.rows / 32) * ceil_div(a.cols, (int64_t)kWave * kV);
    if (tiles <= 0x7FFFFFFFll) {
      int64_t grid = (int64_t)cus * tuning("mx.col_blocks_per_cu");
      if (grid > tiles) grid = tiles;
      mx_col_kernel<IN, OUT><<<(unsigned)grid, kBlock, 0, a.stream>>>(a.x, (uint32_t)a.rows, (uint32_t)a.cols, a.data,
                                                                     a.scale, (uint32_t)tiles);
      return launch_status();
    }
  }
  // blocks along the rows with a transposed payload: through the LDS transpose tile
  if constexpr (LAYOUT == DT_SCALE_PLAIN) {
    if (a.axis == 1 && a.transpose && a.rows % 16 == 0 && aligned(a.data, 16) && aligned(a.scale, 4) &&
        a.rows < (1ll << 31) && a.cols < (1ll << 31)) {
      const int64_t tiles = ceil_div(a.rows, (int64_t)kDualRows) * ceil_div(a.cols, (int64_t)(32 * kV));
      if (tiles <= 0x7FFFFFFFll) {
        mx_row_t_kernel<IN, OUT><<<(unsigned)tiles, kBlock, 0, a.stream>>>(a.x, (uint32_t)a.rows, (uint32_t)a.cols, a.data,
                                                                          a.scale);
        return launch_status();
      }
    }
  }
  // general orientation / alignment
  int64_t outer, inner_blocks, xos, xes, dos, des, s_rows, s_cols;
  int s_t;
  if (a.axis == 1) {
    outer = a.rows; inner_blocks = a.cols / 32; xos = a.cols; xes = 1;
    if (!a.transpose) { dos = a.cols; des = 1; s_rows = a.rows; s_cols = inner_blocks; s_t = 0; }
    else { dos = 1; des = a.rows; s_rows = inner_blocks; s_cols = a.rows; s_t = 1; }
  } else {
    outer = a.cols; inner_blocks = a.rows / 32; xos = 1; xes = a.cols;
    if (!a.transpose) { dos = 1; des = a.cols; s_rows = inner_blocks; s_cols = a.cols; s_t = 1; }
    else { dos = a.rows; des = 1; s_rows = a.cols; s_cols = inner_blocks; s_t = 0; }
  }
  const int64_t total = outer * inner_blocks;
  if (ceil_div(total, kBlock) > 0x7FFFFFFFll) return DT_ERR_INVALID_SHAPE;
  mx_any_kernel<IN, OUT, LAYOUT><<<(unsigned)ceil_div(total, kBlock), kBlock, 0, a.stream>>>(
      a.x, outer, inner_blocks, xos, xes, dos, des, s_rows, s_cols, s_t, a.data, a.scale);
  return launch_status();
}

template <int IN>
int launch_mx_in(const MxArgs& a, int out_dtype, int layout) {
  if (out_dtype == DT_E4M3FN)
    return layout == DT_SCALE_BLOCKED ? launch_mx<IN, DT_E4M3FN, DT_SCALE_BLOCKED>(a) : launch_mx<IN, DT_E4M3FN, DT_SCALE_PLAIN>(a);
  return layout == DT_SCALE_BLOCKED ? launch_mx<IN, DT_E5M2, DT_SCALE_BLOCKED>(a) : launch_mx<IN, DT_E5M2, DT_SCALE_PLAIN>(a);
}

struct DualArgs {
  const void* x;
  int64_t rows, cols;
  uint8_t *data_r, *scale_r, *data_c, *scale_c;
  hipStream_t stream;
};

// DT_OK when the one-read kernel was launched, kNotTaken when the shape or an alignment rules it out
constexpr int kNotTaken = -1;
template <int IN, int OUT, int LAYOUT>
int launch_dual(const DualArgs& a) {
  constexpr int kTileCols = 32 * InTraits<IN>::kVec;
  if (!aligned(a.data_r, 8) || !aligned(a.data_c, 16) || !aligned(a.scale_r, 4) ||
      !aligned(a.scale_c, 4) || a.rows >= (1ll << 31) || a.cols >= (1ll << 31))
    return kNotTaken;
  const int64_t tiles = ceil_div(a.rows, (int64_t)kDualRows) * ceil_div(a.cols, (int64_t)kTileCols);
  if (tiles > 0x7FFFFFFFll) return kNotTaken;
  const int order = tuning("mx.dual_order") >= 0 ? tuning("mx.dual_order")
                    : a.cols > 2 * a.rows                ? 0
                    : a.rows % (8 * kDualRows) == 0      ? 2
                                                         : 1;
  mx_dual_kernel<IN, OUT, LAYOUT><<<(unsigned)tiles, kBlock, 0, a.stream>>>(a.x, (uint32_t)a.rows, (uint32_t)a.cols, a.data_r,
                                                                           a.scale_r, a.data_c, a.scale_c, order);
  return launch_status();
}
template <int IN>
int launch_dual_in(const DualArgs& a, int out_dtype, int layout) {
  if (out_dtype == DT_E4M3FN)
    return layout == DT_SCALE_BLOCKED ? launch_dual<IN, DT_E4M3FN, DT_SCALE_BLOCKED>(a) : launch_dual<IN, DT_E4M3FN, DT_SCALE_PLAIN>(a);
  return layout == DT_SCALE_BLOCKED ? launch_dual<IN, DT_E5M2, DT_SCALE_BLOCKED>(a) : launch_dual<IN, DT_E5M2, DT_SCALE_PLAIN>(a);
}

int zero_blocked_padding(uint8_t* scale, int64_t SR, int64_t SC, hipStream_t s) {
  if (SR % 128 == 0 && SC % 4 == 0) return DT_OK;  // the cast writes every byte
  const int64_t n = dt_blocked_scale_bytes(SR, SC);
  dt::fill_bytes_kernel<<<(unsigned)std::min<int64_t>(dt::ceil_div(n, 256), 4096), 256, 0, s>>>(scale, n, 0);
  return dt::launch_status();
}
}  // namespace

extern "C" int64_t dt_blocked_scale_bytes(int64_t R, int64_t C) {
  if (R < 0 || C < 0) return 0;
  return 128 * dt::ceil_div(R, 128) * 4 * dt::ceil_div(C, 4);
}

extern "C" int dt_mx_fp8_quantize(const void* x, int in_dtype, int64_t rows, int64_t cols, int axis, int transpose,
                                  int out_dtype, int scale_layout, void* data, uint8_t* scale, dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16 && in_dtype != DT_F16) return DT_ERR_INVALID_DTYPE;
  if (out_dtype != DT_E4M3FN && out_dtype != DT_E5M2) return DT_ERR_INVALID_DTYPE;
  if ((axis != 0 && axis != 1) || (transpose != 0 && transpose != 1)) return DT_ERR_INVALID_MODE;
  if (scale_layout != DT_SCALE_PLAIN && scale_layout != DT_SCALE_BLOCKED) return DT_ERR_INVALID_MODE;
  if (rows < 0 || cols < 0) return DT_ERR_INVALID_SHAPE;
  if ((axis == 1 ? cols : rows) % 32 != 0) return DT_ERR_INVALID_SHAPE;
  // the blocked layout is defined for a scale matrix [outer, inner/32]
  if (scale_layout == DT_SCALE_BLOCKED && !((axis == 1 && !transpose) || (axis == 0 && transpose))) return DT_ERR_INVALID_MODE;
  if (rows == 0 || cols == 0) return DT_OK;
  if (!x || !data || !scale) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(x, in_dtype == DT_F32 ? 4 : 2)) return DT_ERR_MISALIGNED;
  hipStream_t s = dt::as_hip(stream);
  if (scale_layout == DT_SCALE_BLOCKED) {  // zero the padding the cast itself never writes
    if (int st = zero_blocked_padding(scale, axis == 1 ? rows : cols, (axis == 1 ? cols : rows) / 32, s)) return st;
  }
  MxArgs a{x, rows, cols, axis, transpose, static_cast<uint8_t*>(data), scale, s};
  switch (in_dtype) {
    case DT_F32: return launch_mx_in<DT_F32>(a, out_dtype, scale_layout);
    case DT_BF16: return launch_mx_in<DT_BF16>(a, out_dtype, scale_layout);
    default: return launch_mx_in<DT_F16>(a, out_dtype, scale_layout);
  }
}

extern "C" int dt_mx_fp8_quantize_dual(const void* x, int in_dtype, int64_t rows, int64_t cols, int out_dtype, int scale_layout,
                                       void* data_rows, uint8_t* scale_rows, void* data_cols_t, uint8_t* scale_cols_t,
                                       dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16 && in_dtype != DT_F16) return DT_ERR_INVALID_DTYPE;
  if (out_dtype != DT_E4M3FN && out_dtype != DT_E5M2) return DT_ERR_INVALID_DTYPE;
  if (scale_layout != DT_SCALE_PLAIN && scale_layout != DT_SCALE_BLOCKED) return DT_ERR_INVALID_MODE;
  if (rows < 0 || cols < 0 || rows % 32 != 0 || cols % 32 != 0) return DT_ERR_INVALID_SHAPE;
  if (rows == 0 || cols == 0) return DT_OK;
  if (!x || !data_rows || !scale_rows || !data_cols_t || !scale_cols_t) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(x, in_dtype == DT_F32 ? 4 : 2)) return DT_ERR_MISALIGNED;
  hipStream_t s = dt::as_hip(stream);
  DualArgs a{x, rows, cols, static_cast<uint8_t*>(data_rows), scale_rows, static_cast<uint8_t*>(data_cols_t), scale_cols_t, s};
  const bool fast_ok = dt::tuning("mx.dual") != 0;
  if (fast_ok) {
    if (scale_layout == DT_SCALE_BLOCKED) {
      if (int st = zero_blocked_padding(scale_rows, rows, cols / 32, s)) return st;
      if (int st = zero_blocked_padding(scale_cols_t, cols, rows / 32, s)) return st;
    }
    int st;
    switch (in_dtype) {
      case DT_F32: st = launch_dual_in<DT_F32>(a, out_dtype, scale_layout); break;
      case DT_BF16: st = launch_dual_in<DT_BF16>(a, out_dtype, scale_layout); break;
      default: st = launch_dual_in<DT_F16>(a, out_dtype, scale_layout); break;
    }
    if (st != kNotTaken) return st;
  }
  // two passes over x
  if (int st = dt_mx_fp8_quantize(x, in_dtype, rows, cols, 1, 0, out_dtype, scale_layout, data_rows, scale_rows, stream)) return st;
  return dt_mx_fp8_quantize(x, in_dtype, rows, cols, 0, 1, out_dtype, scale_layout, data_cols_t, scale_cols_t, stream);
}

namespace {
// MXFP4: the row-wise kernel with the e2m1 output code (same walk over the blocks, same scale stores)
template <int IN, int LAYOUT>
int launch_mx_fp4(const MxArgs& a) {
  const int64_t nblocks = a.rows * a.cols / 32;
  const int64_t nsuper = ceil_div(nblocks, (int64_t)64);
  int64_t waves = (int64_t)device_facts().cu_count * tuning("mx.blocks_per_cu") * (kBlock / kWave);
  if (waves > nsuper) waves = nsuper;
  const unsigned grid = (unsigned)ceil_div(waves, (int64_t)(kBlock / kWave));
  if constexpr (LAYOUT == DT_SCALE_BLOCKED) {
    if (a.rows % 128 == 0 && a.cols % 512 == 0 && tuning("mx.row_band4")) {
      mx_row_kernel<IN, DT_E2M1, LAYOUT, true><<<grid, kBlock, 0, a.stream>>>(a.x, (uint32_t)nblocks, (uint32_t)(a.cols / 32),
                                                                             a.data, a.scale);
      return launch_status();
    }
  }
  mx_row_kernel<IN, DT_E2M1, LAYOUT><<<grid, kBlock, 0, a.stream>>>(a.x, (uint32_t)nblocks, (uint32_t)(a.cols / 32), a.data,
                                                                   a.scale);
  return launch_status();
}
// blocks down the columns, payload transposed: [cols, rows/2], scales [cols, rows/32]
template <int IN, int LAYOUT>
int launch_mx_fp4_cols(const MxArgs& a) {
  // As for MXFP8, the one-read kernel without its row-wise half, on its grid of walking workgroups, for
  // 16-bit inputs with more tiles than that grid (bf16, us, this / mx_col_t_kernel: 8192 x 8192 33.1 / 33.9,
  // 16384 x 4096 30.5 / 35.5, 4096 x 16384 31.5 / 31.7; it loses for fp32, 55.4 / 51.9, and for small
  // tensors, 2048 x 4096 6.6 / 5.9)
  constexpr int kV = InTraits<IN>::kVec;
  if constexpr (IN != DT_F32) {
    const int64_t pipe_grid = (int64_t)tuning("mx.colt_pipe") * device_facts().cu_count;
    const int64_t dual_tiles = ceil_div(a.rows, (int64_t)kDualRows) * ceil_div(a.cols, (int64_t)(32 * kV));
    if (a.cols % kV == 0 && tuning("mx.colt_via_dual") && pipe_grid > 0 && dual_tiles > pipe_grid && dual_tiles <= 0x7FFFFFFFll) {
      const int order = tuning("mx.dual_order") >= 0 ? tuning("mx.dual_order") : (a.rows % (8 * kDualRows) == 0 ? 2 : (a.cols < a.rows ? 1 : 0));
      mx_dual_kernel<IN, DT_E2M1, LAYOUT, false, true><<<(unsigned)pipe_grid, kBlock, 0, a.stream>>>(
          a.x, (uint32_t)a.rows, (uint32_t)a.cols, nullptr, nullptr, a.data, a.scale, order);
      return launch_status();
    }
  }
  const int64_t tiles = ceil_div(a.rows, (int64_t)kColTRows) * ceil_div(a.cols, (int64_t)kColTCols);
  if (tiles > 0x7FFFFFFFll) return DT_ERR_INVALID_SHAPE;
  mx_col_t_kernel<IN, DT_E2M1, LAYOUT><<<(unsigned)tiles, kBlock, 0, a.stream>>>(a.x, (uint32_t)a.rows, (uint32_t)a.cols, a.data,
                                                                                a.scale);
  return launch_status();
}
}  // namespace

extern "C" int dt_mx_fp4_quantize(const void* x, int in_dtype, int64_t rows, int64_t cols, int axis, int scale_layout,
                                  void* data, uint8_t* scale, dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16 && in_dtype != DT_F16) return DT_ERR_INVALID_DTYPE;
  if (axis != 0 && axis != 1) return DT_ERR_INVALID_MODE;
  if (scale_layout != DT_SCALE_PLAIN && scale_layout != DT_SCALE_BLOCKED) return DT_ERR_INVALID_MODE;
  if (rows < 0 || cols < 0 || (axis == 1 ? cols : rows) % 32 != 0) return DT_ERR_INVALID_SHAPE;
  if (rows == 0 || cols == 0) return DT_OK;
  if (!x || !data || !scale) return DT_ERR_NULL_POINTER;
  hipStream_t s = dt::as_hip(stream);
  const bool blocked = scale_layout == DT_SCALE_BLOCKED;
  if (axis == 0) {
    // a lane loads 4 adjacent columns of a row with one 8- or 16-byte load
    const int64_t kB = in_dtype == DT_F32 ? 4 : 2;
    if (cols % 4 != 0 || rows >= (1ll << 31) || cols >= (1ll << 31)) return DT_ERR_INVALID_SHAPE;
    if (!dt::aligned(x, 4 * kB) || (cols * kB) % (4 * kB) != 0 || !dt::aligned(data, 16) || !dt::aligned(scale, 4))
      return DT_ERR_MISALIGNED;
    if (blocked) {
      if (int st = zero_blocked_padding(scale, cols, rows / 32, s)) return st;
    }
    MxArgs a{x, rows, cols, 0, 1, static_cast<uint8_t*>(data), scale, s};
    switch (in_dtype) {
      case DT_F32: return blocked ? launch_mx_fp4_cols<DT_F32, DT_SCALE_BLOCKED>(a) : launch_mx_fp4_cols<DT_F32, DT_SCALE_PLAIN>(a);
      case DT_BF16: return blocked ? launch_mx_fp4_cols<DT_BF16, DT_SCALE_BLOCKED>(a) : launch_mx_fp4_cols<DT_BF16, DT_SCALE_PLAIN>(a);
      default: return blocked ? launch_mx_fp4_cols<DT_F16, DT_SCALE_BLOCKED>(a) : launch_mx_fp4_cols<DT_F16, DT_SCALE_PLAIN>(a);
    }
  }
  if (rows * cols / 32 >= (1ll << 28)) return DT_ERR_INVALID_SHAPE;  // block indices are 32 bits wide in the kernel
  if (!dt::aligned(x, 16) || !dt::aligned(data, 4)) return DT_ERR_MISALIGNED;
  if (blocked) {
    if (int st = zero_blocked_padding(scale, rows, cols / 32, s)) return st;
  }
  MxArgs a{x, rows, cols, 1, 0, static_cast<uint8_t*>(data), scale, s};
  switch (in_dtype) {
    case DT_F32: return blocked ? launch_mx_fp4<DT_F32, DT_SCALE_BLOCKED>(a) : launch_mx_fp4<DT_F32, DT_SCALE_PLAIN>(a);
    case DT_BF16: return blocked ? launch_mx_fp4<DT_BF16, DT_SCALE_BLOCKED>(a) : launch_mx_fp4<DT_BF16, DT_SCALE_PLAIN>(a);
    default: return blocked ? launch_mx_fp4<DT_F16, DT_SCALE_BLOCKED>(a) : launch_mx_fp4<DT_F16, DT_SCALE_PLAIN>(a);
  }
}

namespace {
// both MXFP4 operands of one tensor from a single read: mx_dual_kernel with the e2m1 output code
template <int IN, int LAYOUT>
int launch_dual_fp4(const DualArgs& a) {
  constexpr int kTileCols = 32 * InTraits<IN>::kVec;
  if (!aligned(a.data_r, 4) || !aligned(a.data_c, 16) || !aligned(a.scale_r, 4) || !aligned(a.scale_c, 4) ||
      a.rows >= (1ll << 31) || a.cols >= (1ll << 31))
    return kNotTaken;
  const int64_t tiles = ceil_div(a.rows, (int64_t)kDualRows) * ceil_div(a.cols, (int64_t)kTileCols);
  if (tiles > 0x7FFFFFFFll) return kNotTaken;
  const int order = tuning("mx.dual_order") >= 0 ? tuning("mx.dual_order")
                    : a.cols > 2 * a.rows                ? 0
                    : a.rows % (8 * kDualRows) == 0      ? 2
                                                         : 1;
  mx_dual_kernel<IN, DT_E2M1, LAYOUT><<<(unsigned)tiles, kBlock, 0, a.stream>>>(a.x, (uint32_t)a.rows, (uint32_t)a.cols, a.data_r,
                                                                               a.scale_r, a.data_c, a.scale_c, order);
  return launch_status();
}
template <int IN>
int launch_dual_fp4_in(const DualArgs& a, int layout) {
  return layout == DT_SCALE_BLOCKED ? launch_dual_fp4<IN, DT_SCALE_BLOCKED>(a) : launch_dual_fp4<IN, DT_SCALE_PLAIN>(a);
}
}  // namespace

extern "C" int dt_mx_fp4_quantize_dual(const void* x, int in_dtype, int64_t rows, int64_t cols, int scale_layout, void* data_rows,
                                       uint8_t* scale_rows, void* data_cols_t, uint8_t* scale_cols_t, dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16 && in_dtype != DT_F16) return DT_ERR_INVALID_DTYPE;
  if (scale_layout != DT_SCALE_PLAIN && scale_layout != DT_SCALE_BLOCKED) return DT_ERR_INVALID_MODE;
  if (rows < 0 || cols < 0 || rows % 32 != 0 || cols % 32 != 0) return DT_ERR_INVALID_SHAPE;
  if (rows == 0 || cols == 0) return DT_OK;
  if (!x || !data_rows || !scale_rows || !data_cols_t || !scale_cols_t) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(x, in_dtype == DT_F32 ? 4 : 2)) return DT_ERR_MISALIGNED;
  hipStream_t s = dt::as_hip(stream);
  DualArgs a{x, rows, cols, static_cast<uint8_t*>(data_rows), scale_rows, static_cast<uint8_t*>(data_cols_t), scale_cols_t, s};
  if (dt::tuning("mx.dual") != 0) {
    if (scale_layout == DT_SCALE_BLOCKED) {
      if (int st = zero_blocked_padding(scale_rows, rows, cols / 32, s)) return st;
      if (int st = zero_blocked_padding(scale_cols_t, cols, rows / 32, s)) return st;
    }
    int st;
    switch (in_dtype) {
      case DT_F32: st = launch_dual_fp4_in<DT_F32>(a, scale_layout); break;
      case DT_BF16: st = launch_dual_fp4_in<DT_BF16>(a, scale_layout); break;
      default: st = launch_dual_fp4_in<DT_F16>(a, scale_layout); break;
    }
    if (st != kNotTaken) return st;
  }
  // two passes over x
  if (int st = dt_mx_fp4_quantize(x, in_dtype, rows, cols, 1, scale_layout, data_rows, scale_rows, stream)) return st;
  return dt_mx_fp4_quantize(x, in_dtype, rows, cols, 0, scale_layout, data_cols_t, scale_cols_t, stream);
}

extern "C" int dt_to_blocked(const uint8_t* scale, int64_t R, int64_t C, uint8_t* out, dt_stream_t stream) {
  if (R < 0 || C < 0) return DT_ERR_INVALID_SHAPE;
  if (R == 0 || C == 0) return DT_OK;
  if (!scale || !out) return DT_ERR_NULL_POINTER;
  hipStream_t s = dt::as_hip(stream);
  if (R % 128 != 0 || C % 4 != 0) {
    const int64_t n = dt_blocked_scale_bytes(R, C);
    dt::fill_bytes_kernel<<<(unsigned)std::min<int64_t>(dt::ceil_div(n, 256), 4096), 256, 0, s>>>(out, n, 0);
    if (int st = dt::launch_status()) return st;
  }
  if (dt::ceil_div(R * C, 256) > 0x7FFFFFFFll) return DT_ERR_INVALID_SHAPE;
  dt::to_blocked_kernel<<<(unsigned)dt::ceil_div(R * C, 256), 256, 0, s>>>(scale, R, C, out);
  return dt::launch_status();
}
