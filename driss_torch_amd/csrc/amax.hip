// dt_amax: global max |x| of a flat tensor (C ABI).
#include "quant_kernels.hpp"

extern "C" int dt_amax(const void* x, int in_dtype, int64_t numel, float* out, void* workspace,
                       size_t workspace_bytes, dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16) return DT_ERR_INVALID_DTYPE;
  if (numel < 0) return DT_ERR_INVALID_SHAPE;
  if (numel == 0) return DT_ERR_EMPTY;
  if (!x || !out) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(x, in_dtype == DT_F32 ? 4 : 2) || !dt::aligned(out, 4)) return DT_ERR_MISALIGNED;
  if (int st = dt::check_workspace(workspace, workspace_bytes)) return st;
  hipStream_t s = dt::as_hip(stream);
  if (in_dtype == DT_F32) return dt::launch_amax<DT_F32>(x, numel, workspace, out, nullptr, 0, 0.f, 0.f, s);
  return dt::launch_amax<DT_BF16>(x, numel, workspace, out, nullptr, 0, 0.f, 0.f, s);
}
