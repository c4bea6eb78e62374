// Host-side helpers shared by the C-ABI entry points: argument checks, device facts,
// the workspace layout and the tuning table.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "driss_torch_hip.h"

namespace dt {

// ---- workspace layout (see dt_workspace_bytes in the public header) -----------------
constexpr int kMaxPartials = 8192;          // upper bound on the grid of a reduction kernel
constexpr size_t kWsTicket = 0;             // u32 arrival counter, zero between launches
constexpr size_t kWsRunning = 128;          // u32 running max of |x| bits, zero between launches
constexpr size_t kWsAmax = 64;              // f32 amax of the last reduction
constexpr size_t kWsScale = 68;             // f32 scale[2] derived from it
constexpr size_t kWsBytes = 4096;

struct DeviceFacts {
  int cu_count;
};
const DeviceFacts& device_facts();  // of the current device, cached per device

int tuning(const char* key);  // current value of a launch knob

// Per-workgroup clock readings for the benchmark's phase report exist only in a build with
// -DDT_PHASE_LOG (a second library made for that report); in the product build kPhaseLog is false, the
// kernels' stamps compile to nothing and the entry point that sets the buffer is not there.
#ifdef DT_PHASE_LOG
constexpr bool kPhaseLog = true;
// Device buffer for the readings (dt_set_phase_log), or null when none is set, it holds fewer than
// `need_bytes`, or it lives on another device than the current one.
uint64_t* phase_log(size_t need_bytes);
#else
constexpr bool kPhaseLog = false;
inline uint64_t* phase_log(size_t) { return nullptr; }
#endif

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return a / b + (a % b != 0); }  // src/include/utils.h:37-39

inline int launch_status() { return hipGetLastError() == hipSuccess ? DT_OK : DT_ERR_LAUNCH; }

inline hipStream_t as_hip(dt_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace dt
