// dt_dynamic_scaled_quant*: amax -> scale -> saturating fp8 cast, per tensor and per row (C ABI).
//
// For a caller that has said that its process owns the GPU (dt_set_exclusive_gpu, DRISS_TORCH_RESIDENT=1),
// a tensor that fits the chip's registers and LDS (128 MiB on 256 CUs) goes through one kernel
// that holds it there between the reduction and the cast (resident_kernels.hpp).  Otherwise
// the work is two stream-ordered kernels: the amax reduction, whose last workgroup also derives
// the scale(s) into the workspace, and the streaming cast, which reads the scale from there;
// the second read of x is then served from the memory-side cache as far as it fits.
#include "quant_kernels.hpp"
#include "resident_kernels.hpp"
#include "rowwise_kernels.hpp"

#include <mutex>

namespace {
inline float fmax_of(int out_dtype) { return out_dtype == DT_E5M2 ? 57344.0f : 448.0f; }

// ---- the reduction workspace of dt_dynamic_scaled_quant_noalloc: device memory that belongs to the
// library's code object, so that the caller neither allocates nor passes one.  Each device the library
// runs on holds its own copy at its own address until the process ends; host code never uses the
// array's name as an address, only what hipGetSymbolAddress returned for the device at hand.
static __device__ __align__(256) uint8_t scratch[dt::kWsBytes];

constexpr int kScratchDevices = 16;
std::mutex g_scratch_mu;
uint8_t* g_scratch_ptr[kScratchDevices] = {};  // per device, looked up at the entry point's first call there

// nullptr with *status set when the lookup fails
uint8_t* scratch_of_current_device(int* status) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kScratchDevices) {
    (void)hipGetLastError();
    *status = DT_ERR_LAUNCH;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      *status = DT_ERR_LAUNCH;
      return nullptr;
    }
    g_scratch_ptr[dev] = static_cast<uint8_t*>(p);
  }
  return g_scratch_ptr[dev];
}

// the words a reduction expects to find zero (a fill kernel, not hipMemsetAsync: callers may capture)
__global__ void clear_scratch_kernel(uint32_t* p) { p[blockIdx.x * blockDim.x + threadIdx.x] = 0u; }
}  // namespace

extern "C" int dt_dynamic_scaled_quant(const void* x, int in_dtype, int64_t numel, int out_dtype, int round_mode,
                                       void* out, float* amax_out, float* scale_out, void* workspace,
                                       size_t workspace_bytes, dt_stream_t stream) {
  if (int st = dt::check_cast_args(x, in_dtype, numel, out_dtype, round_mode, out)) return st;
  if (numel == 0) return DT_ERR_EMPTY;
  if (int st = dt::check_workspace(workspace, workspace_bytes)) return st;
  hipStream_t s = dt::as_hip(stream);
  const float fm = fmax_of(out_dtype);
  const int res = dt::launch_resident<false>(x, in_dtype, numel, out_dtype, round_mode, workspace, out, nullptr, amax_out,
                                             scale_out, fm, 0.f, s);
  if (res == DT_OK || res == DT_ERR_RESIDENT_GAVE_UP) return res;
  int st = in_dtype == DT_F32 ? dt::launch_amax<DT_F32>(x, numel, workspace, amax_out, scale_out, 1, fm, 0.f, s)
                              : dt::launch_amax<DT_BF16>(x, numel, workspace, amax_out, scale_out, 1, fm, 0.f, s);
  if (st) return st;
  const float* scale = reinterpret_cast<const float*>(static_cast<const uint8_t*>(workspace) + dt::kWsScale);
  return dt::launch_cast<false>(x, in_dtype, numel, scale, out_dtype, round_mode, out, nullptr, s);
}

extern "C" int dt_dynamic_scaled_quant_noalloc(const void* x, int in_dtype, int64_t numel, int out_dtype, int round_mode,
                                               void* out, float* amax_out, float* scale_out, dt_stream_t stream) {
  if (int st = dt::check_cast_args(x, in_dtype, numel, out_dtype, round_mode, out)) return st;
  if (numel == 0) return DT_ERR_EMPTY;
  if (numel > DT_NOALLOC_MAX_NUMEL) return DT_ERR_TOO_LARGE;
  int st = DT_OK;
  uint8_t* const ws = scratch_of_current_device(&st);
  if (!ws) return st;
  hipStream_t s = dt::as_hip(stream);
  // The array keeps whatever the last call on this device left in it.  A completed call leaves its
  // counters at zero, but one that was cut short would not: start from zero every time.
  clear_scratch_kernel<<<dt::kWsBytes / 4 / 256, 256, 0, s>>>(reinterpret_cast<uint32_t*>(ws));
  if (int e = dt::launch_status()) return e;
  const float fm = fmax_of(out_dtype);
  st = in_dtype == DT_F32 ? dt::launch_amax<DT_F32>(x, numel, ws, amax_out, scale_out, 1, fm, 0.f, s)
                          : dt::launch_amax<DT_BF16>(x, numel, ws, amax_out, scale_out, 1, fm, 0.f, s);
  if (st) return st;
  return dt::launch_cast<false>(x, in_dtype, numel, reinterpret_cast<const float*>(ws + dt::kWsScale), out_dtype, round_mode,
                                out, nullptr, s);
}

extern "C" int dt_amax_scales(const void* x, int in_dtype, int64_t numel, float* amax_out, float* scale_out,
                              void* workspace, size_t workspace_bytes, dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16) return DT_ERR_INVALID_DTYPE;
  if (numel < 0) return DT_ERR_INVALID_SHAPE;
  if (numel == 0) return DT_ERR_EMPTY;
  if (!x) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(x, in_dtype == DT_F32 ? 4 : 2)) return DT_ERR_MISALIGNED;
  if (int st = dt::check_workspace(workspace, workspace_bytes)) return st;
  hipStream_t s = dt::as_hip(stream);
  return in_dtype == DT_F32 ? dt::launch_amax<DT_F32>(x, numel, workspace, amax_out, scale_out, 2, 448.0f, 57344.0f, s)
                            : dt::launch_amax<DT_BF16>(x, numel, workspace, amax_out, scale_out, 2, 448.0f, 57344.0f, s);
}

extern "C" int dt_saturated_cast_pair(const void* x, int in_dtype, int64_t numel, const float* scale, int round_mode,
                                      void* out_e4m3fn, void* out_e5m2, dt_stream_t stream) {
  if (int st = dt::check_cast_args(x, in_dtype, numel, DT_E4M3FN, round_mode, out_e4m3fn)) return st;
  if (numel > 0 && !out_e5m2) return DT_ERR_NULL_POINTER;
  if (!scale) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(scale, 4)) return DT_ERR_MISALIGNED;
  if (numel == 0) return DT_OK;
  return dt::launch_cast<true>(x, in_dtype, numel, scale, DT_E4M3FN, round_mode, out_e4m3fn, out_e5m2, dt::as_hip(stream));
}

extern "C" int dt_dynamic_scaled_quant_pair(const void* x, int in_dtype, int64_t numel, int round_mode,
                                            void* out_e4m3fn, void* out_e5m2, float* amax_out, float* scale_out,
                                            void* workspace, size_t workspace_bytes, dt_stream_t stream) {
  if (int st = dt::check_cast_args(x, in_dtype, numel, DT_E4M3FN, round_mode, out_e4m3fn)) return st;
  if (!out_e5m2) return DT_ERR_NULL_POINTER;
  if (numel > 0 && dt::check_workspace(workspace, workspace_bytes) == DT_OK && (in_dtype == DT_F32 || in_dtype == DT_BF16)) {
    const int res = dt::launch_resident<true>(x, in_dtype, numel, DT_E4M3FN, round_mode, workspace, out_e4m3fn, out_e5m2,
                                              amax_out, scale_out, 448.0f, 57344.0f, dt::as_hip(stream));
    if (res == DT_OK || res == DT_ERR_RESIDENT_GAVE_UP) return res;
  }
  if (int st = dt_amax_scales(x, in_dtype, numel, amax_out, scale_out, workspace, workspace_bytes, stream)) return st;
  const float* scale = reinterpret_cast<const float*>(static_cast<const uint8_t*>(workspace) + dt::kWsScale);
  return dt::launch_cast<true>(x, in_dtype, numel, scale, DT_E4M3FN, round_mode, out_e4m3fn, out_e5m2, dt::as_hip(stream));
}

extern "C" int dt_dynamic_scaled_quant_rowwise(const void* x, int in_dtype, int64_t rows, int64_t cols, int out_dtype,
                                               void* out, float* amax_out, float* scale_out, dt_stream_t stream) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16) return DT_ERR_INVALID_DTYPE;
  if (out_dtype != DT_E4M3FN && out_dtype != DT_E5M2) return DT_ERR_INVALID_DTYPE;
  if (rows < 0 || cols < 0) return DT_ERR_INVALID_SHAPE;
  if (rows == 0) return DT_OK;
  if (cols == 0) return DT_ERR_EMPTY;
  if (!x || !out) return DT_ERR_NULL_POINTER;
  if (!dt::aligned(x, in_dtype == DT_F32 ? 4 : 2)) return DT_ERR_MISALIGNED;
  return dt::launch_rowwise(x, in_dtype, rows, cols, out_dtype, out, amax_out, scale_out, dt::as_hip(stream));
}

extern "C" int dt_dynamic_quant_gave_up(void) { return dt::resident_take_gave_up() ? 1 : 0; }

extern "C" int dt_set_exclusive_gpu(int on) {
  if (on) {
    // the current device's word of pinned host memory now, so that no quantization call has to make it
    // (a process without a usable device may still set the flag: the first launch tries again)
    int dev = -1;
    if (hipGetDevice(&dev) == hipSuccess) {
      dt::ResidentGate& gate = dt::resident_gate();
      std::lock_guard<std::mutex> lock(gate.mu);
      (void)dt::resident_host_word_locked(gate, dev);
    } else {
      (void)hipGetLastError();
    }
  }
  return dt_set_tuning("dynamic.resident", on ? 1 : 0);
}

extern "C" int dt_get_exclusive_gpu(void) { return dt::tuning("dynamic.resident") ? 1 : 0; }

extern "C" uint64_t dt_dynamic_quant_resident_launches(void) {
  return dt::resident_gate().launches.load(std::memory_order_relaxed);
}
