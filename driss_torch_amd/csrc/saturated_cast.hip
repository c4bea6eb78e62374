// dt_saturated_cast: fp8(clamp(x * scale)) with a per-tensor device scale (C ABI).
#include "quant_kernels.hpp"

extern "C" int dt_saturated_cast(const void* x, int in_dtype, int64_t numel, const float* scale, int out_dtype,
                                 int round_mode, void* out, dt_stream_t stream) {
  if (int st = dt::check_cast_args(x, in_dtype, numel, out_dtype, round_mode, out)) return st;
  if (!scale) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(scale, 4)) return DT_ERR_MISALIGNED;
  if (numel == 0) return DT_OK;
  return dt::launch_cast<false>(x, in_dtype, numel, scale, out_dtype, round_mode, out, nullptr, dt::as_hip(stream));
}
