// Per-tensor dynamic quantization with the tensor held on the chip between its two passes.
//
// amax -> scale -> cast needs x twice, and the second pass cannot start before the first has
// finished everywhere.  An MI355X has 256 CUs x (512 KB of vector registers + 160 KB of LDS):
// a tensor of up to 128 MiB fits into the registers and the LDS of one workgroup per CU.  So one
// persistent workgroup per CU loads its share of x once (16-byte vectors, grid-strided: 96 per
// lane stay in registers, 36 more go to LDS), reduces |x| on the way, meets the other workgroups
// at a grid-wide barrier built on the reduction's own atomics, derives the scale(s) and converts
// straight out of registers and LDS.  HBM sees one read of x and the fp8 writes; the two-kernel
// path reads x from HBM and again from the memory-side cache.  Measured on 8192 x 8192 bf16 ->
// e4m3fn + e5m2: 65 us for the two kernels, see bench.py for this one.
//
// The barrier needs every workgroup of the grid to be resident at once.  The grid is at most one
// workgroup per CU and a workgroup owns a CU's whole register file, so the dispatcher spreads
// the grid one per CU; other kernels only delay that.  (hipLaunchCooperativeKernel would check
// it, but costs 18 us per launch here, more than the kernel saves.)  What must not happen is two
// such grids at once, so the host chains them.  The wait is bounded all the same: a workgroup
// that gives up sets a sticky flag in the workspace and writes NaN, and every wave reaches the
// end of the kernel whatever happens.
#pragma once

#include <stdlib.h>

#include <type_traits>

#include <atomic>
#include <mutex>

#include "quant_kernels.hpp"

namespace dt {

constexpr int kResRegVecs = 92;   // 16-byte vectors per lane kept in registers (368 VGPRs)
constexpr int kResLdsVecs = 36;   // ... and in LDS (144 KiB per workgroup)
constexpr int kResVecs = kResRegVecs + kResLdsVecs;
constexpr int kResPipe = 4;       // loads per batch of the pipelined load phase (4..8 in flight per lane)

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}
constexpr size_t kResLdsBytes = (size_t)kResLdsVecs * kBlock * 16;
constexpr size_t kWsDepart = 192;  // u32 departure counter of the grid barrier, zero between launches
// u64 release words of the grid barrier, zero between launches: kWsReleaseWords of them, kWsReleaseStep
// bytes apart.  A workgroup polls word (workgroup index % kWsReleaseWords).  One word polled by every
// workgroup is one memory location serving a few hundred requests per polling round, one after the other:
// the release then reaches the workgroups spread over 3 us (measured with the phase log).
constexpr size_t kWsRelease = 1024;
constexpr size_t kWsReleaseStep = 256;
constexpr uint32_t kWsReleaseWords = 8;
static_assert(kWsRelease + kWsReleaseWords * kWsReleaseStep <= kWsBytes, "release words fit the workspace");
constexpr size_t kWsTimeout = 196; // u32, set (and left set) if a barrier wait ever gave up

// One vector to e4m3fn and e5m2 at once, for products that cannot be NaN.  The two scales are
// fmax / amax with fmax = 448 and 57344 = 128 * 448, so scale_e5m2 == 128 * scale_e4m3 exactly
// (a power of two commutes with every rounding on the way, also with the bf16 roundings of
// modes 1 and 2): the e5m2 bytes come from the same products, converted with a scale of 2^-7.
template <int IN, bool ROUND_BF16>
__device__ __forceinline__ void cast_vec_pair_finite(u32x4 w, float s4, uint8_t* __restrict__ out4,
                                                     uint8_t* __restrict__ out5, uint32_t vec_index) {
  constexpr int kV = InTraits<IN>::kVec;
  float p[kV];
  products_of<IN>(w, s4, p);
  uint32_t r4[kV / 4], r5[kV / 4];
  products_to_fp8<IN, DT_E4M3FN, ROUND_BF16>(p, r4, 1.0f);
  products_to_fp8<IN, DT_E5M2, ROUND_BF16>(p, r5, 0x1p-7f);  // the convert divides by its scale: x 128
  if constexpr (IN == DT_F32) {
    st_stream(reinterpret_cast<uint32_t*>(out4) + vec_index, r4[0]);
    st_stream(reinterpret_cast<uint32_t*>(out5) + vec_index, r5[0]);
  } else {
    st_stream(reinterpret_cast<u32x2*>(out4) + vec_index, u32x2{r4[0], r4[1]});
    st_stream(reinterpret_cast<u32x2*>(out5) + vec_index, u32x2{r5[0], r5[1]});
  }
}

// OVERFLOW: the tensor is larger than the chip holds (up to kResMaxOver times).  A workgroup's
// share then has vector slots past the kResVecs it can keep: pass 1 streams those first (reduce
// only), pass 2 reads them again after the kept part has been converted.  Memory sees the kept
// part once and only the rest twice.
constexpr int kResMaxOver = 4;
template <int IN, int OUT, bool ROUND_BF16, bool ROUND_SCALE, bool PAIR, bool OVERFLOW = false>
__global__ __launch_bounds__(kBlock) void resident_quant_kernel(const void* __restrict__ x, int64_t nvec, int tail,
                                                               uint8_t* __restrict__ ws, uint8_t* __restrict__ out,
                                                               uint8_t* __restrict__ out2, float* __restrict__ amax_out,
                                                               float* __restrict__ scale_out, float fmax0, float fmax1,
                                                               uint32_t spin_limit, uint32_t* __restrict__ host_flag,
                                                               uint64_t* __restrict__ phase_log) {
  constexpr int kV = InTraits<IN>::kVec;
  constexpr int OUT2 = OUT == DT_E4M3FN ? DT_E5M2 : DT_E4M3FN;
  extern __shared__ __attribute__((aligned(16))) u32x4 keep[];  // [kResLdsVecs][kBlock]
  __shared__ uint32_t red[kBlock / kWave];
  saturate_fp8_conversions();
  __shared__ uint32_t bcast;
  const int tid = threadIdx.x;
  const u32x4* v = static_cast<const u32x4*>(x);
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int64_t first = (int64_t)blockIdx.x * kBlock + tid;
  // phase_log (only in a build with DT_PHASE_LOG, and normally null there): four readings of the constant-rate 100 MHz counter per workgroup --
  // start, share loaded and reduced, released from the grid barrier, done -- for the benchmark's
  // per-phase report.  The counter is common to all CUs, so readings of different workgroups compare.
  auto stamp = [&](int k) {
    if constexpr (kPhaseLog) {
      if (phase_log && tid == 0) phase_log[blockIdx.x * 4 + k] = wall_clock64();
    }
  };
  stamp(0);

  // ---- pass 1: load the share once, keep it, reduce |x|
  u32x4 r[kResRegVecs];
  uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
  // Loads are issued in batches of kResBatch before any of them is looked at (one wave per SIMD:
  // nothing else keeps the memory system busy while a wave waits).  No branch around a load
  // either: past the end the last vector is read again and replaced by zeros.
  auto fetch = [&](int k) -> u32x4 {
    const int64_t i = first + k * stride;
    return ld_stream(v + (i < nvec ? i : nvec - 1));
  };
  auto absorb = [&](int k, u32x4& w) {
    const bool inside = first + k * stride < nvec;
    w.x = inside ? w.x : 0u; w.y = inside ? w.y : 0u; w.z = inside ? w.z : 0u; w.w = inside ? w.w : 0u;
    if constexpr (IN == DT_F32) {
      a0 = umax(a0, absbits_f32(w.x)); a1 = umax(a1, absbits_f32(w.y));
      a2 = umax(a2, absbits_f32(w.z)); a3 = umax(a3, absbits_f32(w.w));
    } else {
      a0 = pk_absmax16(a0, w.x); a1 = pk_absmax16(a1, w.y);
      a2 = pk_absmax16(a2, w.z); a3 = pk_absmax16(a3, w.w);
    }
  };
  constexpr int kResBatch = 16;
  static_assert(kResRegVecs % 4 == 0 && kResLdsVecs % 4 == 0, "batches");
  static_assert(kResLdsVecs % kResPipe == 0, "a pipelined batch is LDS slots or register slots, not both");
  // Vector slots k >= nk lie past the end for every lane of this workgroup: a tensor smaller than
  // the chip's capacity skips whole batches (a branch the workgroup takes as one), in both passes.
  const uint32_t block_first = blockIdx.x * kBlock;
  const uint32_t nk = block_first < (uint32_t)nvec ? ((uint32_t)nvec - block_first + (uint32_t)stride - 1u) / (uint32_t)stride : 0u;
  if constexpr (OVERFLOW) {  // slots that cannot be kept: before anything is held in registers
    for (uint32_t k0 = kResVecs; k0 < nk; k0 += kResBatch) {
      u32x4 t[kResBatch];
#pragma unroll
      for (int j = 0; j < kResBatch; ++j) t[j] = fetch((int)k0 + j);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < kResBatch; ++j) absorb((int)k0 + j, t[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // The kept part: LDS slots first (through temporaries), then the register slots in place.
  if (nk > (uint32_t)(kResVecs - 2 * kResBatch)) {
    // A (nearly) full share: one unconditional stream of batches of kResPipe loads, the loads of batch
    // n + 1 issued before batch n is looked at, so that the memory system never runs dry between
    // batches (load phase of 8192 x 8192 bf16: 21.8 -> see bench).  No branch anywhere: a slot past the
    // end reads the last vector again and counts as zeros.
    constexpr int kSeq = kResVecs, kBatches = (kSeq + kResPipe - 1) / kResPipe;
    u32x4 t[2][kResPipe];  // temporaries of the LDS slots (position p < kResLdsVecs of the sequence)
    auto issue = [&](auto n_tag) {
      constexpr int n = decltype(n_tag)::value;
#pragma unroll
      for (int j = 0; j < kResPipe; ++j) {
        const int p = n * kResPipe + j;
        if (p >= kSeq) continue;
        if (p < kResLdsVecs) t[n & 1][j] = fetch(kResRegVecs + p);
        else r[p - kResLdsVecs] = fetch(p - kResLdsVecs);
      }
    };
    auto retire = [&](auto n_tag) {
      constexpr int n = decltype(n_tag)::value;
#pragma unroll
      for (int j = 0; j < kResPipe; ++j) {
        const int p = n * kResPipe + j;
        if (p >= kSeq) continue;
        if (p < kResLdsVecs) {
          absorb(kResRegVecs + p, t[n & 1][j]);
          keep[p * kBlock + tid] = t[n & 1][j];
        } else {
          absorb(p - kResLdsVecs, r[p - kResLdsVecs]);
        }
      }
    };
    issue(std::integral_constant<int, 0>{});
    static_for<kBatches>([&](auto n_tag) {
      constexpr int n = decltype(n_tag)::value;
      if constexpr (n + 1 < kBatches) issue(std::integral_constant<int, n + 1>{});
      __builtin_amdgcn_sched_barrier(0);
      retire(n_tag);
      __builtin_amdgcn_sched_barrier(0);
    });
  } else {
#pragma unroll
    for (int b = 0; b < kResLdsVecs; b += kResBatch) {
      if ((uint32_t)(kResRegVecs + b) >= nk) break;
      u32x4 t[kResBatch];
  #pragma unroll
      for (int j = 0; j < kResBatch; ++j)
        if (b + j < kResLdsVecs) t[j] = fetch(kResRegVecs + b + j);
      __builtin_amdgcn_sched_barrier(0);
  #pragma unroll
      for (int j = 0; j < kResBatch; ++j)
        if (b + j < kResLdsVecs) {
          absorb(kResRegVecs + b + j, t[j]);
          keep[(b + j) * kBlock + tid] = t[j];
        }
      __builtin_amdgcn_sched_barrier(0);
    }
  #pragma unroll
    for (int b = 0; b < kResRegVecs; b += kResBatch) {
      if ((uint32_t)b >= nk) break;
  #pragma unroll
      for (int j = 0; j < kResBatch; ++j)
        if (b + j < kResRegVecs) r[b + j] = fetch(b + j);
      __builtin_amdgcn_sched_barrier(0);
  #pragma unroll
      for (int j = 0; j < kResBatch; ++j)
        if (b + j < kResRegVecs) absorb(b + j, r[b + j]);
      __builtin_amdgcn_sched_barrier(0);
    }
}
  uint32_t m;
  if constexpr (IN == DT_F32) {
    m = umax(umax(a0, a1), umax(a2, a3));
  } else {
    uint32_t p = pk_absmax16(pk_absmax16(a0, a1), pk_absmax16(a2, a3));
    m = umax(p & 0xFFFFu, p >> 16) << 16;
  }
  if (blockIdx.x == 0 && tid < tail) m = umax(m, absbits_of<IN>(x, nvec * kV + tid));  // x is 16-byte aligned: no head
  m = block_umax<kBlock / kWave>(m, red);
  stamp(1);

  // ---- grid barrier on the reduction's atomics: fold the partial into the running maximum,
  // take a ticket, wait until every workgroup has taken one, read the maximum.
  // The waiting workgroups poll a word of its own (another cache line): polling the line the
  // arrivals update slows those atomics down for everybody (measured: 8 us -> see bench).
  uint32_t* running = reinterpret_cast<uint32_t*>(ws + kWsRunning);
  uint32_t* ticket = reinterpret_cast<uint32_t*>(ws + kWsTicket);
  uint32_t* depart = reinterpret_cast<uint32_t*>(ws + kWsDepart);
  // (1 << 32) | amax bits once everybody has arrived; this workgroup polls its own copy
  uint64_t* release = reinterpret_cast<uint64_t*>(ws + kWsRelease + (blockIdx.x % kWsReleaseWords) * kWsReleaseStep);
  bool gave_up_here = false;  // thread 0's: this workgroup stopped waiting
  if (tid == 0) {
    uint32_t before = __hip_atomic_fetch_max(running, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t one = 1u;  // the ticket depends on the returned value, so the two atomics stay ordered
    asm volatile("v_and_or_b32 %0, %1, 0, %0" : "+v"(one) : "v"(before));
    const uint32_t t = __hip_atomic_fetch_add(ticket, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t bits;
    if (t == gridDim.x - 1) {
      // last to arrive: every other workgroup's maximum was folded in before it took its ticket
      bits = __hip_atomic_load(running, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint64_t word = (1ull << 32) | bits;
#pragma unroll
      for (uint32_t j = 0; j < kWsReleaseWords; ++j)
        __hip_atomic_store(reinterpret_cast<uint64_t*>(ws + kWsRelease + j * kWsReleaseStep), word, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    } else {
      uint32_t spins = 0;
      uint64_t rel;
      while (((rel = __hip_atomic_load(release, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 32) == 0) {
        __builtin_amdgcn_s_sleep(2);
        if (++spins >= spin_limit) {  // cannot happen when the grid is resident; never hang the GPU
          __hip_atomic_store(reinterpret_cast<uint32_t*>(ws + kWsTimeout), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          // and tell the host (a word of pinned host memory): the library's next call on this device reports it
          if (host_flag) __hip_atomic_store(host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          rel = 0x7FC00000ull;  // the outputs of this workgroup become NaN: a loud failure
          gave_up_here = true;
          break;
        }
      }
      bits = (uint32_t)rel;
    }
    bcast = bits;
  }
  __syncthreads();
  stamp(2);
  const float amax = as_f32(bcast);
  float s = amax_to_scale(amax, fmax0), s2 = PAIR ? amax_to_scale(amax, fmax1) : 0.f;
  if constexpr (ROUND_SCALE) { s = round_to_bf16(s); s2 = round_to_bf16(s2); }

  // ---- pass 2: convert out of registers and LDS.  A product can only be a NaN if the tensor
  // holds a NaN or an infinity (inf * 0), which amax tells: then x is simply read again by the
  // streaming cast with its NaN handling (a rare path, and the only one with a function call,
  // which must not sit among 368 live registers).  Otherwise no test is needed at all.
  if (bcast >= 0x7F800000u) {
    for (int64_t i = first; i < nvec; i += stride) {
      const u32x4 w = ld_stream(v + i);
      cast_vec<IN, OUT, ROUND_BF16>(w, s, out, i);
      if constexpr (PAIR) cast_vec<IN, OUT2, ROUND_BF16>(w, s2, out2, i);
    }
  } else {
    // The vector indices are recomputed from an opaque copy of the first one: reusing pass 1's
    // 128 index pairs would keep them in registers across the barrier, next to the data.
    // (at most 2^31 vectors fit the chip, so 32-bit indices do)
    uint32_t first2 = (uint32_t)first;
    asm volatile("" : "+v"(first2));
    const uint32_t stride32 = (uint32_t)stride, nvec32 = (uint32_t)nvec;
    auto emit_at = [&](uint32_t i, u32x4 w) {
      if constexpr (PAIR) {
        static_assert(!PAIR || OUT == DT_E4M3FN, "the pair is e4m3fn + e5m2");
        cast_vec_pair_finite<IN, ROUND_BF16>(w, s, out, out2, i);
      } else {
        cast_vec<IN, OUT, ROUND_BF16, false>(w, s, out, i);
      }
    };
    auto emit = [&](int k, u32x4 w) {
      const uint32_t i = first2 + k * stride32;
      if (i < nvec32) emit_at(i, w);
    };
    // A batch whose every slot lies inside for every lane of the workgroup is converted without the
    // per-slot test: with a branch around each vector its 25-30 instructions run as one dependent chain
    // (one wave per SIMD: nothing else fills the gaps), without it the compiler interleaves the batch
    // (store phase of 8192 x 8192 bf16 -> one fp8 output: 13.9 us -> see bench).
    auto whole_batch = [&](int k_last) { return block_first + (uint32_t)(kBlock - 1) + (uint32_t)k_last * stride32 < nvec32; };
#pragma unroll
    for (int b = 0; b < kResRegVecs; b += kResBatch) {
      if ((uint32_t)b >= nk) break;
      constexpr int kRegLast = kResRegVecs - 1;
      if (whole_batch(b + kResBatch - 1 < kRegLast ? b + kResBatch - 1 : kRegLast)) {
#pragma unroll
        for (int j = 0; j < kResBatch; ++j)
          if (b + j < kResRegVecs) emit_at(first2 + (uint32_t)(b + j) * stride32, r[b + j]);
      } else {
#pragma unroll
        for (int j = 0; j < kResBatch; ++j)
          if (b + j < kResRegVecs) emit(b + j, r[b + j]);
      }
    }
#pragma unroll
    for (int b = 0; b < kResLdsVecs; b += kResBatch) {
      if ((uint32_t)(kResRegVecs + b) >= nk) break;
      constexpr int kLdsLast = kResLdsVecs - 1;
      if (whole_batch(kResRegVecs + (b + kResBatch - 1 < kLdsLast ? b + kResBatch - 1 : kLdsLast))) {
#pragma unroll
        for (int j = 0; j < kResBatch; ++j)
          if (b + j < kResLdsVecs) emit_at(first2 + (uint32_t)(kResRegVecs + b + j) * stride32, keep[(b + j) * kBlock + tid]);
      } else {
#pragma unroll
        for (int j = 0; j < kResBatch; ++j)
          if (b + j < kResLdsVecs) emit(kResRegVecs + b + j, keep[(b + j) * kBlock + tid]);
      }
    }
    if constexpr (OVERFLOW) {  // the slots that were not kept: read again, the registers are free now
      for (uint32_t k0 = kResVecs; k0 < nk; k0 += kResBatch) {
        u32x4 t[kResBatch];
#pragma unroll
        for (int j = 0; j < kResBatch; ++j) {
          const uint32_t i = first2 + (k0 + j) * stride32;
          t[j] = ld_stream(v + (i < nvec32 ? i : nvec32 - 1u));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kResBatch; ++j) emit((int)k0 + j, t[j]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (blockIdx.x == 0 && tid < tail) {
    const int64_t e = nvec * kV + tid;
    out[e] = cast_one<IN, OUT, ROUND_BF16>(x, e, s);
    if constexpr (PAIR) out2[e] = cast_one<IN, OUT2, ROUND_BF16>(x, e, s2);
  }
  if constexpr (kPhaseLog) {
    if (phase_log) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores of this wave have left
      __syncthreads();
      stamp(3);
    }
  }
  // ---- departure, at the very end: counted here and not at the barrier, where the atomic's round trip
  // (the 256 of them queue on one address) held every workgroup back by 1.5-3 us before its stores.  The
  // last workgroup to leave publishes amax and the scales and re-arms the workspace for the next launch.
  if (tid == 0) {
    // everything this wave has sent to memory has been performed, the release words of the last
    // arriver included: whoever finds itself last may put them back to zero
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the counter's low half counts departures, its high half those of workgroups that gave up: the last
    // one to leave then knows whether any part of the output is NaN without another round trip
    const uint32_t left_before = __hip_atomic_fetch_add(depart, gave_up_here ? 0x10001u : 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((left_before & 0xFFFFu) == gridDim.x - 1) {
      const bool any_gave_up = gave_up_here || (left_before >> 16) != 0;
      __hip_atomic_store(running, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(depart, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (uint32_t j = 0; j < kWsReleaseWords; ++j)
        __hip_atomic_store(reinterpret_cast<uint64_t*>(ws + kWsRelease + j * kWsReleaseStep), 0ull, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      // after a give-up anywhere amax and the scales are NaN like the outputs of the workgroups that gave up
      const float amax_final = any_gave_up ? as_f32(0x7FC00000u) : as_f32(bcast);
      float* wscale = reinterpret_cast<float*>(ws + kWsScale);
      *reinterpret_cast<float*>(ws + kWsAmax) = amax_final;
      if (amax_out) *amax_out = amax_final;
      const float s0 = amax_to_scale(amax_final, fmax0);
      wscale[0] = s0;
      if (scale_out) scale_out[0] = s0;
      if constexpr (PAIR) {
        const float s1 = amax_to_scale(amax_final, fmax1);
        wscale[1] = s1;
        if (scale_out) scale_out[1] = s1;
      }
    }
  }
}

// Host-side chaining of resident launches (see launch_resident_impl).
struct ResidentGate {
  static constexpr int kMaxDevices = 16;
  std::mutex mu;
  bool used[kMaxDevices] = {};
  hipStream_t last_stream[kMaxDevices] = {};  // stream of the device's latest resident launch
  hipEvent_t event[kMaxDevices] = {};         // recorded there when a launch arrives on another stream
  // One word of pinned host memory per device, made at the device's first resident launch and kept for
  // the life of the process: a workgroup that gives up waiting sets it, the host reads it before the
  // next per-tensor dynamic quantization on that device.
  volatile uint32_t* gave_up_host[kMaxDevices] = {};
  uint32_t* gave_up_dev[kMaxDevices] = {};
  std::atomic<uint64_t> launches{0};  // one-kernel launches of this process (dt_dynamic_quant_resident_launches)
};
inline ResidentGate& resident_gate() {
  static ResidentGate* g = new ResidentGate();  // leaked on purpose: no HIP calls at process exit
  return *g;
}

// The device's word of pinned host memory, made if it is not there yet (gate.mu held).  False when it
// cannot be made.  dt_set_exclusive_gpu(1) calls this up front so that no quantization call allocates.
inline bool resident_host_word_locked(ResidentGate& gate, int dev) {
  if (dev < 0 || dev >= ResidentGate::kMaxDevices) return false;
  if (gate.gave_up_host[dev]) return true;
  void* host = nullptr;
  void* devp = nullptr;
  if (hipHostMalloc(&host, 64, hipHostMallocMapped) != hipSuccess || hipHostGetDevicePointer(&devp, host, 0) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  *static_cast<volatile uint32_t*>(host) = 0u;
  gate.gave_up_host[dev] = static_cast<volatile uint32_t*>(host);
  gate.gave_up_dev[dev] = static_cast<uint32_t*>(devp);
  return true;
}

// True when the process runs under a CU mask given through the environment, which
// hipExtStreamGetCUMask does not report: the grid might then never be resident as a whole.
inline bool cu_mask_in_environment() {
  static const bool masked = [] {
    for (const char* name : {"HSA_CU_MASK", "ROC_GLOBAL_CU_MASK", "HSA_CU_MASK_SKIP_INIT"}) {
      const char* v = getenv(name);
      if (v && *v) return true;
    }
    return false;
  }();
  return masked;
}

// Has a resident launch on the current device given up since the last time this was asked?  Reads and
// clears the host word; meaningful once the launch in question has completed.
inline bool resident_take_gave_up() {
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev < 0 || dev >= ResidentGate::kMaxDevices) return false;
  ResidentGate& gate = resident_gate();
  std::lock_guard<std::mutex> lock(gate.mu);
  volatile uint32_t* w = gate.gave_up_host[dev];
  if (!w || *w == 0u) return false;
  *w = 0u;
  return true;
}

// CUs a stream may use: all of them, unless it was created with a CU mask
// (hipExtStreamCreateWithCUMask) or the process runs under a global one.  About 0.2 us per call.
inline int stream_cu_count(hipStream_t stream) {
  uint32_t mask[32] = {};
  if (hipExtStreamGetCUMask(stream, 32, mask) != hipSuccess) {
    (void)hipGetLastError();
    return 1 << 30;  // unknown: treat as unrestricted
  }
  int n = 0;
  for (uint32_t w : mask) n += __builtin_popcount(w);
  return n;
}

// Launch the resident kernel if the tensor qualifies.  Returns DT_OK when it was launched, a
// negative value when the caller should take the two-kernel path instead.
constexpr int kResidentNotTaken = -1;
template <int IN, int OUT, bool ROUND_BF16, bool ROUND_SCALE, bool PAIR, bool OVERFLOW = false>
inline int launch_resident_impl(const void* x, int64_t numel, void* ws, void* out, void* out2, float* amax_out,
                                float* scale_out, float fmax0, float fmax1, hipStream_t stream) {
  if constexpr (PAIR && OUT != DT_E4M3FN) return kResidentNotTaken;  // the pair is (e4m3fn, e5m2)
  else {
  constexpr int kV = InTraits<IN>::kVec;
  constexpr size_t kStoreAlign = IN == DT_F32 ? 4 : 8;
  if (!aligned(x, 16) || !aligned(out, kStoreAlign) || (PAIR && !aligned(out2, kStoreAlign))) return kResidentNotTaken;
  const int cus = device_facts().cu_count;
  int64_t nvec = numel / kV;
  int tail = (int)(numel % kV);
  const int64_t capacity = (int64_t)cus * kBlock * kResVecs;
  if constexpr (!OVERFLOW) {
    if (nvec > capacity && nvec <= capacity * kResMaxOver && tuning("dynamic.resident_overflow"))
      return launch_resident_impl<IN, OUT, ROUND_BF16, ROUND_SCALE, PAIR, true>(x, numel, ws, out, out2, amax_out, scale_out,
                                                                                fmax0, fmax1, stream);
  }
  if (nvec < 1 || nvec > capacity * (OVERFLOW ? kResMaxOver : 1)) return kResidentNotTaken;
  int64_t grid = ceil_div(nvec, (int64_t)kBlock * 4);  // at least 4 vectors per lane before another workgroup joins
  if (grid > cus) grid = cus;
  if (grid < 1) grid = 1;
  auto kernel = resident_quant_kernel<IN, OUT, ROUND_BF16, ROUND_SCALE, PAIR, OVERFLOW>;
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev < 0 || dev >= ResidentGate::kMaxDevices) return kResidentNotTaken;
  // per instantiation and device (a function's attributes live with the device's copy of the code);
  // the call is idempotent, so a race between threads only repeats it
  static std::atomic<bool> configured[ResidentGate::kMaxDevices] = {};
  if (!configured[dev].load(std::memory_order_relaxed)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)kResLdsBytes) != hipSuccess) {
      (void)hipGetLastError();
      return kResidentNotTaken;
    }
    configured[dev].store(true, std::memory_order_relaxed);
  }
  uint8_t* w = static_cast<uint8_t*>(ws);
  uint8_t* o = static_cast<uint8_t*>(out);
  uint8_t* o2 = static_cast<uint8_t*>(out2);
  const uint32_t spin_limit = (uint32_t)tuning("dynamic.resident_spin_limit");
  // Two grids of this kernel in flight at once (two streams) could each hold part of the chip
  // and wait for the rest for ever: resident launches of a device are chained: one that arrives
  // on another stream than the previous one first waits for that stream's tail.  A stream under graph capture cannot take such a dependency.
  ResidentGate& gate = resident_gate();
  std::lock_guard<std::mutex> lock(gate.mu);
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return kResidentNotTaken;
  }
  // every workgroup waits for all the others: a stream that may not use as many CUs as the grid has
  // workgroups could never hold them all at once
  if (stream_cu_count(stream) < grid || cu_mask_in_environment()) return kResidentNotTaken;
  if (!resident_host_word_locked(gate, dev)) return kResidentNotTaken;  // without a way to report a give-up the path is not taken
  uint64_t* const log = phase_log((size_t)grid * 32);
  if (gate.used[dev] && gate.last_stream[dev] != stream) {
    // mark the tail of the stream that ran the previous resident kernel and wait for it here
    if (!gate.event[dev] && hipEventCreateWithFlags(&gate.event[dev], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      gate.event[dev] = nullptr;
      return kResidentNotTaken;
    }
    if (hipEventRecord(gate.event[dev], gate.last_stream[dev]) != hipSuccess) {
      (void)hipGetLastError();           // that stream is gone: its work may still be running
      (void)hipDeviceSynchronize();
    } else if (hipStreamWaitEvent(stream, gate.event[dev], 0) != hipSuccess) {
      (void)hipGetLastError();
      return kResidentNotTaken;
    }
  }
  kernel<<<(unsigned)grid, kBlock, kResLdsBytes, stream>>>(x, nvec, tail, w, o, o2, amax_out, scale_out, fmax0, fmax1,
                                                         spin_limit, gate.gave_up_dev[dev], log);
  const int st = launch_status();
  if (st == DT_OK) {
    gate.used[dev] = true;
    gate.last_stream[dev] = stream;
    gate.launches.fetch_add(1, std::memory_order_relaxed);
  }
  return st;
  }
}

template <bool PAIR>
inline int launch_resident(const void* x, int in_dtype, int64_t numel, int out_dtype, int round_mode, void* ws, void* out,
                           void* out2, float* amax_out, float* scale_out, float fmax0, float fmax1, hipStream_t stream) {
  // Where the two kernels win: below about 32 MiB the cast's second read of x comes out of the 256 MiB
  // last-level cache faster than this kernel's barrier and its launch with 144 KB of LDS cost (bf16, us,
  // this kernel against the two, both fp8 outputs / one: 8 MiB 12.9 vs 11.3 / 12.6 vs 10.6, 16 MiB 14.9 vs
  // 14.3 / 13.9 vs 13.1, 32 MiB 19.1 vs 19.7 / 17.4 vs 17.2, 48 MiB 22.8 vs 27.2 / 20.4 vs 23.1, 64 MiB
  // 27.5 vs 34.0 / 24.0 vs 29.2, 96 MiB 37.7 vs 48.1 / 32.1 vs 40.6, 128 MiB 44.4 vs 61.9).
  const int64_t bytes = numel * (in_dtype == DT_F32 ? 4 : 2);
  // An earlier launch of the one-kernel path on this device gave up waiting for the whole chip (its
  // outputs are NaN): say so once, and leave the path off for the rest of the process.
  if (resident_take_gave_up()) {
    (void)dt_set_tuning("dynamic.resident", 0);
    return DT_ERR_RESIDENT_GAVE_UP;
  }
  if (!tuning("dynamic.resident") || bytes < (int64_t)tuning("dynamic.resident_min_kib") * 1024) return kResidentNotTaken;
  if (bytes >= (int64_t)tuning("dynamic.resident_gap_lo_kib") * 1024 && bytes < (int64_t)tuning("dynamic.resident_gap_hi_kib") * 1024)
    return kResidentNotTaken;
#define DT_RES(IN, OUT, RB, RS) \
  return launch_resident_impl<IN, OUT, RB, RS, PAIR>(x, numel, ws, out, out2, amax_out, scale_out, fmax0, fmax1, stream)
  if (in_dtype == DT_F32) {
    if (out_dtype == DT_E4M3FN) DT_RES(DT_F32, DT_E4M3FN, false, false);
    DT_RES(DT_F32, DT_E5M2, false, false);
  }
  if (round_mode == DT_ROUND_F32) {
    if (out_dtype == DT_E4M3FN) DT_RES(DT_BF16, DT_E4M3FN, false, false);
    DT_RES(DT_BF16, DT_E5M2, false, false);
  }
  if (round_mode == DT_ROUND_BF16_PRODUCT) {
    if (out_dtype == DT_E4M3FN) DT_RES(DT_BF16, DT_E4M3FN, true, false);
    DT_RES(DT_BF16, DT_E5M2, true, false);
  }
  if (out_dtype == DT_E4M3FN) DT_RES(DT_BF16, DT_E4M3FN, true, true);
  DT_RES(DT_BF16, DT_E5M2, true, true);
#undef DT_RES
}

}  // namespace dt
