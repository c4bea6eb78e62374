// Status strings, device facts, tuning knobs and the workspace entry points of the C ABI.
#include <stdlib.h>
#include <string.h>
#include <strings.h>

#include <atomic>
#include <mutex>

#include "dt_device.hpp"
#include "dt_host.hpp"

namespace dt {

namespace {
struct Knob {
  const char* key;
  std::atomic<int> value;  // set from any thread while launches on other threads read it
};
// Launch-shape knobs.  Workgroups per CU for the persistent grids, chosen on MI355X.
//   dynamic.resident: 1 = per-tensor dynamic quantization of a tensor that fits the chip runs as one
//                 kernel that keeps it in registers and LDS.  That kernel waits inside for all of its
//                 workgroups and so assumes that this process has the GPU to itself: 0 unless the caller
//                 opts in (dt_set_exclusive_gpu, or DRISS_TORCH_RESIDENT=1 in the environment when the
//                 library is loaded); dynamic.resident_min_kib = smallest such
//                 tensor; sizes in [resident_gap_lo_kib, resident_gap_hi_kib) take the two kernels
//                 dynamic.resident_overflow: 1 = tensors of up to 4 x the chip's capacity keep what fits
//                 and read only the rest twice
//   rowwise.block_from_vecs: rows of at least this many 16-byte vectors get a workgroup each (shorter
//                 ones a wave each)
//   mx.dual:      1 = dt_mx_fp8_quantize_dual reads x once (0: two single casts)
//   mx.colt_via_dual: 1 = the transposed column cast runs as the one-read kernel without its row half
//   mx.dual_order: tile order of the one-read kernel: -1 = chosen by shape, 0 = down the rows first, 1 = along
//                 the columns first, 2 = bands of 8 row tiles
//   mx.colt_pipe: the transposed column cast as a grid of this many workgroups per CU that walk the tiles
//                 with the next tile's loads in flight (0 = one workgroup per tile)
//   mx.row_band4: 1 = row-wise MX cast with blocked scales walks 4 rows x 512 elements per wave pass
//   gemm.variant: 0 = pick the tile by problem size, 1 = 128x128 tiles, 2 = 256x256 tiles,
//                 7 = 256x256 tiles without the L2 prefetch loads, 9 = the kernel for at most 64 rows
//                 whatever the other dimensions
//   gemm.few_rows_tiles: 16-column tiles per wave of that kernel: 0 = by the number of columns, 1, 2
//   gemm.tail_quads: 1 = tiles left over after whole rounds of 256x256 tiles run as 128x128 quadrants
//                 or 256x128 halves when those fit the chip at once, 0 = never, 2 = always as
//                 quadrants, 3 = always as halves
//   gemm.split_k: 0 = share K between workgroups when the 128x128 tiling leaves CUs idle (needs the
//                 workspace of the _ws entry points), 1 = never, n = n workgroups per tile
Knob g_knobs[] = {
    {"gemm.few_rows_tiles", 0},
    {"gemm.few_rows_stagger", 1},
    {"gemm.few_rows_steps", 0},
    {"gemm.few_rows_per_cu", 0},
    {"amax.blocks_per_cu", 1},
    {"amax.stream_before_cast", 0},
    {"cast.blocks_per_cu", 0},
    {"cast.unroll", 0},
    {"cast.pair_blocks_per_cu", 0},
    {"rowwise.block_from_vecs", 257},
    {"mx.blocks_per_cu", 32},
    {"mx.col_blocks_per_cu", 32},
    {"mx.dual", 1},
    {"mx.dual_order", -1},
    {"mx.colt_pipe", 2},
    {"mx.colt_via_dual", 1},
    {"mx.row_band4", 1},
    {"gemm.variant", 0},
    {"gemm.split_k", 0},
    {"gemm.tail_quads", 1},
    {"dynamic.resident", 0},
    {"dynamic.resident_min_kib", 32768},
    {"dynamic.resident_gap_lo_kib", 0},
    {"dynamic.resident_gap_hi_kib", 0},
    {"dynamic.resident_overflow", 1},
    {"dynamic.resident_spin_limit", 1 << 19},
};
constexpr int kNumKnobs = sizeof(g_knobs) / sizeof(g_knobs[0]);

// DRISS_TORCH_RESIDENT: "1", "on", "true", "yes" (any case) switch the one-kernel dynamic quantization on;
// anything else, or no variable, leaves it off.
bool resident_opt_in_from(const char* v) {
  if (!v) return false;
  for (const char* yes : {"1", "on", "true", "yes"})
    if (strcasecmp(v, yes) == 0) return true;
  return false;
}
struct KnobsFromEnvironment {
  KnobsFromEnvironment() {
    if (resident_opt_in_from(getenv("DRISS_TORCH_RESIDENT")))
      for (int i = 0; i < kNumKnobs; ++i)
        if (strcmp(g_knobs[i].key, "dynamic.resident") == 0) g_knobs[i].value.store(1, std::memory_order_relaxed);
  }
} g_knobs_from_environment;  // after g_knobs in this file: initialised after it, when the library is loaded

#ifdef DT_PHASE_LOG
std::atomic<uint64_t*> g_phase_log{nullptr};
std::atomic<size_t> g_phase_log_bytes{0};
std::atomic<int> g_phase_log_device{-1};
#endif

constexpr int kMaxDevices = 16;
DeviceFacts g_facts[kMaxDevices];
std::once_flag g_facts_once[kMaxDevices];
}  // namespace

int tuning(const char* key) {
  for (int i = 0; i < kNumKnobs; ++i)
    if (strcmp(g_knobs[i].key, key) == 0) return g_knobs[i].value.load(std::memory_order_relaxed);
  return 0;
}

#ifdef DT_PHASE_LOG
uint64_t* phase_log(size_t need_bytes) {
  uint64_t* p = g_phase_log.load(std::memory_order_relaxed);
  if (!p || g_phase_log_bytes.load(std::memory_order_relaxed) < need_bytes) return nullptr;
  int dev = -1;
  (void)hipGetDevice(&dev);
  return dev == g_phase_log_device.load(std::memory_order_relaxed) ? p : nullptr;  // the buffer's own device only
}
#endif

const DeviceFacts& device_facts() {
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev < 0 || dev >= kMaxDevices) dev = 0;
  std::call_once(g_facts_once[dev], [dev] {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    g_facts[dev].cu_count = cus;
  });
  return g_facts[dev];
}

__global__ void zero_words_kernel(uint32_t* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

}  // namespace dt

extern "C" {

const char* dt_status_string(int status) {
  switch (status) {
    case DT_OK: return "ok";
    case DT_ERR_INVALID_DTYPE: return "unsupported dtype";
    case DT_ERR_INVALID_SHAPE: return "invalid shape";
    case DT_ERR_NULL_POINTER: return "null pointer";
    case DT_ERR_MISALIGNED: return "misaligned pointer";
    case DT_ERR_WORKSPACE: return "workspace missing or too small";
    case DT_ERR_INVALID_MODE: return "invalid mode";
    case DT_ERR_LAUNCH: return "kernel launch failed";
    case DT_ERR_EMPTY: return "reduction over zero elements";
    case DT_ERR_RESIDENT_GAVE_UP:
      return "an earlier dynamic quantization on this device gave up waiting for the whole chip and wrote NaN "
             "(is another process using the GPU?); the one-kernel path is now off for this process";
    case DT_ERR_TOO_LARGE: return "more elements than the no-allocation entry point takes (DT_NOALLOC_MAX_NUMEL)";
    default: return "unknown status";
  }
}

int dt_abi_version(void) { return 1; }

size_t dt_workspace_bytes(void) { return dt::kWsBytes; }

int dt_workspace_init(void* workspace, size_t workspace_bytes, dt_stream_t stream) {
  if (!workspace) return DT_ERR_NULL_POINTER;
  if (workspace_bytes < dt::kWsBytes) return DT_ERR_WORKSPACE;
  if (!dt::aligned(workspace, 256)) return DT_ERR_MISALIGNED;
  // a fill kernel rather than hipMemsetAsync, so the call is safe under graph capture
  dt::zero_words_kernel<<<dt::kWsBytes / 4 / 256, 256, 0, dt::as_hip(stream)>>>(static_cast<uint32_t*>(workspace), dt::kWsBytes / 4);
  return dt::launch_status();
}

#ifdef DT_PHASE_LOG
int dt_set_phase_log(void* device_buffer, size_t bytes) {
  if (device_buffer && !dt::aligned(device_buffer, 8)) return DT_ERR_MISALIGNED;
  int dev = -1;
  (void)hipGetDevice(&dev);
  dt::g_phase_log.store(nullptr, std::memory_order_relaxed);
  dt::g_phase_log_bytes.store(device_buffer ? bytes : 0, std::memory_order_relaxed);
  dt::g_phase_log_device.store(device_buffer ? dev : -1, std::memory_order_relaxed);
  dt::g_phase_log.store(static_cast<uint64_t*>(device_buffer), std::memory_order_relaxed);
  return DT_OK;
}
#endif

int dt_set_tuning(const char* key, int value) {
  if (!key) return DT_ERR_NULL_POINTER;
  for (int i = 0; i < dt::kNumKnobs; ++i)
    if (strcmp(dt::g_knobs[i].key, key) == 0) {
      dt::g_knobs[i].value.store(value, std::memory_order_relaxed);
      return DT_OK;
    }
  return DT_ERR_INVALID_MODE;
}

int dt_get_tuning(const char* key, int* value) {
  if (!key || !value) return DT_ERR_NULL_POINTER;
  for (int i = 0; i < dt::kNumKnobs; ++i)
    if (strcmp(dt::g_knobs[i].key, key) == 0) {
      *value = dt::g_knobs[i].value.load(std::memory_order_relaxed);
      return DT_OK;
    }
  return DT_ERR_INVALID_MODE;
}

}  // extern "C"
