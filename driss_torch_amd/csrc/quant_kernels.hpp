// Kernel templates of the per-tensor path: the amax reduction and the saturating fp8 cast.
// Both stream the tensor with 16-byte loads from a persistent grid; they are shared by
// amax.hip, saturated_cast.hip and dynamic_scaled_quant.hip.
#pragma once

#include "dt_device.hpp"
#include "dt_host.hpp"

namespace dt {

constexpr int kBlock = 256;  // 4 waves

template <int IN>
struct InTraits;
template <>
struct InTraits<DT_F32> {
  static constexpr int kBytes = 4, kVec = 4;  // elements per 16-byte vector
};
template <>
struct InTraits<DT_BF16> {
  static constexpr int kBytes = 2, kVec = 8;
};
template <>
struct InTraits<DT_F16> {
  static constexpr int kBytes = 2, kVec = 8;
};

// How a flat tensor is cut for 16-byte access: `head` leading elements up to the first
// aligned address, `nvec` whole vectors, `tail` trailing elements.
struct Split {
  int64_t head, nvec, tail;
};
template <int IN>
inline Split split_for_vectors(const void* x, int64_t numel) {
  constexpr int kB = InTraits<IN>::kBytes, kV = InTraits<IN>::kVec;
  uintptr_t mis = reinterpret_cast<uintptr_t>(x) % 16;
  int64_t head = mis ? (int64_t)((16 - mis) / kB) : 0;
  if (head > numel) head = numel;
  int64_t nvec = (numel - head) / kV;
  return {head, nvec, numel - head - nvec * kV};
}

template <int IN>
__device__ __forceinline__ uint32_t absbits_of(const void* x, int64_t i) {
  if constexpr (IN == DT_F32)
    return static_cast<const uint32_t*>(x)[i] & 0x7FFFFFFFu;
  else
    return ((uint32_t)static_cast<const uint16_t*>(x)[i] & 0x7FFFu) << 16;  // bf16 -> f32 bits
}

// --------------------------------------------------------------------------- amax ----
// Every workgroup reduces a grid-strided share of the vectors to one unsigned magnitude,
// folds it into a running maximum in the workspace with one atomic and takes a ticket; the
// workgroup that draws the last ticket writes amax (and, when NSCALES > 0, the fp8 scales
// derived from it) and re-arms the workspace for the next launch.
template <int IN, int UNROLL, int NSCALES, bool NT>
__global__ __launch_bounds__(kBlock) void amax_kernel(const void* __restrict__ x, Split sp,
                                                      uint8_t* __restrict__ ws, float* __restrict__ amax_out,
                                                      float* __restrict__ scale_out, float fmax0, float fmax1,
                                                      uint64_t* __restrict__ phase_log) {
  constexpr int kB = InTraits<IN>::kBytes, kV = InTraits<IN>::kVec;
  __shared__ uint32_t lds[kBlock / kWave];
  const int tid = threadIdx.x;
  // phase_log (only in a build with DT_PHASE_LOG, and normally null there): readings of the constant-rate
  // 100 MHz counter per workgroup -- start, share loaded, workgroup's maximum known, atomics done -- for
  // the benchmark's per-phase report
  auto stamp = [&](int k) {
    if constexpr (kPhaseLog) {
      if (phase_log && tid == 0) phase_log[blockIdx.x * 4 + k] = wall_clock64();
    }
  };
  stamp(0);
  const u32x4* v = reinterpret_cast<const u32x4*>(static_cast<const uint8_t*>(x) + sp.head * kB);

  uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
  auto absorb = [&](u32x4 w) {
    if constexpr (IN == DT_F32) {
      a0 = umax(a0, absbits_f32(w.x)); a1 = umax(a1, absbits_f32(w.y));
      a2 = umax(a2, absbits_f32(w.z)); a3 = umax(a3, absbits_f32(w.w));
    } else {
      a0 = pk_absmax16(a0, w.x); a1 = pk_absmax16(a1, w.y);
      a2 = pk_absmax16(a2, w.z); a3 = pk_absmax16(a3, w.w);
    }
  };
  // Batches of P loads, software-pipelined over two register sets: the loads of the next batch are
  // issued before the current one is looked at, so P..2P loads per lane stay in flight and the memory
  // system never runs dry between batches.  (Every load of the steady state is unconditional: the wait
  // counts the compiler derives are exact only along straight-line code.)
  constexpr int P = UNROLL / 2;
  const int64_t stride = (int64_t)gridDim.x * kBlock, step = P * stride;
  int64_t i = (int64_t)blockIdx.x * kBlock + tid;
  auto whole_batch_at = [&](int64_t j) { return j + (P - 1) * stride < sp.nvec; };
  auto load_batch = [&](u32x4 (&w)[P], int64_t j) {
#pragma unroll
    for (int u = 0; u < P; ++u) w[u] = ld_maybe_stream<NT>(v + j + u * stride);
  };
  auto absorb_batch = [&](const u32x4 (&w)[P]) {
#pragma unroll
    for (int u = 0; u < P; ++u) absorb(w[u]);
  };
  if (whole_batch_at(i)) {
    u32x4 wa[P], wb[P];
    load_batch(wa, i);
    i += step;
    for (;;) {
      if (!whole_batch_at(i)) { absorb_batch(wa); break; }
      load_batch(wb, i);
      i += step;
      absorb_batch(wa);
      if (!whole_batch_at(i)) { absorb_batch(wb); break; }
      load_batch(wa, i);
      i += step;
      absorb_batch(wb);
    }
  }
  for (; i < sp.nvec; i += stride) absorb(ld_maybe_stream<NT>(v + i));
  stamp(1);

  uint32_t m;
  if constexpr (IN == DT_F32) {
    m = umax(umax(a0, a1), umax(a2, a3));
  } else {
    uint32_t p = pk_absmax16(pk_absmax16(a0, a1), pk_absmax16(a2, a3));
    m = umax(p & 0xFFFFu, p >> 16) << 16;
  }
  if (blockIdx.x == 0) {  // the few elements outside the aligned body
    if (tid < sp.head) m = umax(m, absbits_of<IN>(x, tid));
    if (tid < sp.tail) m = umax(m, absbits_of<IN>(x, sp.head + sp.nvec * kV + tid));
  }
  m = block_umax<kBlock / kWave>(m, lds);
  stamp(2);

  // Publishing the tensor's maximum: amax, the scales derived from it, into the workspace and to the caller
  auto publish = [&](uint32_t bits) {
    const float amax = as_f32(bits);
    *reinterpret_cast<float*>(ws + kWsAmax) = amax;
    if (amax_out) *amax_out = amax;
    if constexpr (NSCALES > 0) {
      float* wscale = reinterpret_cast<float*>(ws + kWsScale);
      const float s0 = amax_to_scale(amax, fmax0);
      wscale[0] = s0;
      if (scale_out) scale_out[0] = s0;
      if constexpr (NSCALES > 1) {
        const float s1 = amax_to_scale(amax, fmax1);
        wscale[1] = s1;
        if (scale_out) scale_out[1] = s1;
      }
    }
  };
  // One relaxed device-scope atomic max per workgroup carries the partial; a second one on the
  // ticket tells the last workgroup to arrive.  No fence is needed: the max is an atomic with
  // return, so it has been performed at the device's coherence point before the ticket is
  // taken, and ticket order is total.  (A release/acquire fence here costs a cache
  // write-back/invalidate per workgroup, which serialises: measured 10x the streaming time.)
  // (Leaving each workgroup's maximum in a slot of its own with a store that writes through, and letting
  // whoever then reads all slots marked publish the result, takes no read-modify-write at all, and is
  // slower: the store's acknowledgement and the cache-missing loads take about 2 us each where an
  // atomic with return takes 0.65 us.  8192 x 8192 bf16: 23.9 against 22.1 us; 1024 x 1024: 8.1 against 4.3.)
  uint32_t* ticket = reinterpret_cast<uint32_t*>(ws + kWsTicket);
  uint32_t* running = reinterpret_cast<uint32_t*>(ws + kWsRunning);
  if (tid == 0) {
    uint32_t before = __hip_atomic_fetch_max(running, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // make the ticket depend on the returned value so the two atomics cannot be reordered
    uint32_t one = 1u;
    asm volatile("v_and_or_b32 %0, %1, 0, %0" : "+v"(one) : "v"(before));
    uint32_t t = __hip_atomic_fetch_add(ticket, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t == gridDim.x - 1) {
      // last to arrive: every other workgroup's max is already in `running`
      const uint32_t r = __hip_atomic_exchange(running, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // re-arm
      __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);                          // re-arm
      publish(r);
    }
    stamp(3);
  }
}

inline int reduction_grid(int64_t nvec, int unroll, const char* knob) {
  int64_t want = ceil_div(nvec, (int64_t)kBlock * unroll);
  int64_t cap = (int64_t)device_facts().cu_count * tuning(knob);
  if (cap > kMaxPartials) cap = kMaxPartials;
  if (want > cap) want = cap;
  return want < 1 ? 1 : (int)want;
}

// Enqueue the amax reduction.  nscales: 0 = amax only, 1 = scale for fmax0, 2 = both.  With
// scales a cast pass over the same tensor follows, so the loads are left cacheable unless
// the "amax.stream_before_cast" knob says otherwise.
template <int IN>
inline int launch_amax(const void* x, int64_t numel, void* ws, float* amax_out, float* scale_out, int nscales,
                       float fmax0, float fmax1, hipStream_t stream) {
  constexpr int kUnroll = 8;
  Split sp = split_for_vectors<IN>(x, numel);
  int grid = reduction_grid(sp.nvec, kUnroll, "amax.blocks_per_cu");
  uint8_t* w = static_cast<uint8_t*>(ws);
  const bool nt = nscales == 0 || tuning("amax.stream_before_cast");
  uint64_t* const log = phase_log((size_t)grid * 32);
#define DT_AMAX(NS, NT) amax_kernel<IN, kUnroll, NS, NT><<<grid, kBlock, 0, stream>>>(x, sp, w, amax_out, scale_out, fmax0, fmax1, log)
  if (nscales == 0) DT_AMAX(0, true);
  else if (nscales == 1) { if (nt) DT_AMAX(1, true); else DT_AMAX(1, false); }
  else { if (nt) DT_AMAX(2, true); else DT_AMAX(2, false); }
#undef DT_AMAX
  return launch_status();
}

// --------------------------------------------------------------------------- cast ----
// ROUND_BF16: round the product to bf16 before the convert (modes 1 and 2 of
// dt_round_mode, bf16 input only); ROUND_SCALE: also round the scale itself (mode 2).
// CHECK_NAN = false is for callers that know no product can be a NaN (no NaN and no infinity in
// the tensor, finite scale): the result is the same, without the test.
//
// The converts saturate by themselves, so the calling kernel must have executed
// saturate_fp8_conversions(); bf16-rounded products go to the convert as the packed pairs the
// rounding instruction leaves.  Per 8 bf16 elements that is 8 unpacks, 8 multiplies, 4 roundings
// and 4 converts, against 48 instructions with unpacked clamps.
template <int IN, int OUT, bool ROUND_BF16>
__device__ __forceinline__ void products_to_fp8(const float (&p)[InTraits<IN>::kVec], uint32_t (&r)[InTraits<IN>::kVec / 4],
                                                float cvt_scale) {
  if constexpr (IN == DT_F32 || !ROUND_BF16) {
#pragma unroll
    for (int q = 0; q < InTraits<IN>::kVec / 4; ++q)
      r[q] = cvt_scaled_4x32<OUT>(as_u32(p[4 * q]), as_u32(p[4 * q + 1]), as_u32(p[4 * q + 2]), as_u32(p[4 * q + 3]), cvt_scale);
  } else {
#pragma unroll
    for (int q = 0; q < 2; ++q)
      r[q] = cvt_scaled_4x16<DT_BF16, OUT>(pack_bf16x2(p[4 * q], p[4 * q + 1]), pack_bf16x2(p[4 * q + 2], p[4 * q + 3]), cvt_scale);
  }
}
template <int IN>
__device__ __forceinline__ void products_of(u32x4 w, float s, float (&p)[InTraits<IN>::kVec]) {
  if constexpr (IN == DT_F32) {
    p[0] = as_f32(w.x) * s; p[1] = as_f32(w.y) * s; p[2] = as_f32(w.z) * s; p[3] = as_f32(w.w) * s;
  } else {
    p[0] = bf16_lo(w.x) * s; p[1] = bf16_hi(w.x) * s; p[2] = bf16_lo(w.y) * s; p[3] = bf16_hi(w.y) * s;
    p[4] = bf16_lo(w.z) * s; p[5] = bf16_hi(w.z) * s; p[6] = bf16_lo(w.w) * s; p[7] = bf16_hi(w.w) * s;
  }
}

// one 16-byte vector of x -> kV / 4 words of fp8 bytes
template <int IN, int OUT, bool ROUND_BF16, bool CHECK_NAN = true>
__device__ __forceinline__ void cast_vec_to_words(u32x4 w, float s, uint32_t (&r)[InTraits<IN>::kVec / 4]) {
  constexpr int kV = InTraits<IN>::kVec;
  float p[kV];
  products_of<IN>(w, s, p);
  products_to_fp8<IN, OUT, ROUND_BF16>(p, r, 1.0f);
  if constexpr (CHECK_NAN) {  // rounding to bf16 keeps a NaN a NaN and its sign
    bool any_nan = false;
#pragma unroll
    for (int k = 0; k < kV; k += 2) any_nan |= __builtin_isunordered(p[k], p[k + 1]);
    if (__builtin_expect(any_nan, 0)) {
#pragma unroll
      for (int q = 0; q < kV / 4; ++q) r[q] = nan_patch4(r[q], p[4 * q], p[4 * q + 1], p[4 * q + 2], p[4 * q + 3]);
    }
  }
}

template <int IN, int OUT, bool ROUND_BF16, bool CHECK_NAN = true>
__device__ __forceinline__ void cast_vec(u32x4 w, float s, uint8_t* __restrict__ out, int64_t vec_index) {
  uint32_t r[InTraits<IN>::kVec / 4];
  cast_vec_to_words<IN, OUT, ROUND_BF16, CHECK_NAN>(w, s, r);
  if constexpr (IN == DT_F32) st_stream(reinterpret_cast<uint32_t*>(out) + vec_index, r[0]);
  else st_stream(reinterpret_cast<u32x2*>(out) + vec_index, u32x2{r[0], r[1]});
}

template <int IN, int OUT, bool ROUND_BF16>
__device__ __forceinline__ uint8_t cast_one(const void* x, int64_t i, float s) {
  float xv;
  if constexpr (IN == DT_F32)
    xv = static_cast<const float*>(x)[i];
  else
    xv = as_f32((uint32_t)static_cast<const uint16_t*>(x)[i] << 16);
  return (uint8_t)(pack4<OUT>(scaled<ROUND_BF16>(xv, s), 0.f, 0.f, 0.f) & 0xFFu);
}

// Aligned streaming cast: x 16-byte aligned, out aligned to its packed store.  The tail
// (< one vector) is done by the first workgroup.  With PAIR the same read also feeds a
// second output of the other fp8 type with its own scale (scale[1], out2).
template <int IN, int OUT, bool ROUND_BF16, bool ROUND_SCALE, bool PAIR, int UNROLL>
__global__ __launch_bounds__(kBlock) void cast_kernel(const void* __restrict__ x, int64_t nvec, int64_t tail,
                                                      const float* __restrict__ scale, uint8_t* __restrict__ out,
                                                      uint8_t* __restrict__ out2) {
  constexpr int kV = InTraits<IN>::kVec;
  constexpr int OUT2 = OUT == DT_E4M3FN ? DT_E5M2 : DT_E4M3FN;
  saturate_fp8_conversions();
  float s = scale[0], s2 = PAIR ? scale[1] : 0.f;
  if constexpr (ROUND_SCALE) { s = round_to_bf16(s); s2 = round_to_bf16(s2); }
  const u32x4* v = static_cast<const u32x4*>(x);
  // batches of UNROLL loads, software-pipelined over two register sets (see amax_kernel)
  constexpr int P = UNROLL;
  const int64_t stride = (int64_t)gridDim.x * kBlock, step = P * stride;
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  auto whole_batch_at = [&](int64_t j) { return j + (P - 1) * stride < nvec; };
  auto load_batch = [&](u32x4 (&w)[P], int64_t j) {
#pragma unroll
    for (int u = 0; u < P; ++u) w[u] = ld_stream(v + j + u * stride);
  };
  auto cast_batch = [&](const u32x4 (&w)[P], int64_t j) {
#pragma unroll
    for (int u = 0; u < P; ++u) {
      cast_vec<IN, OUT, ROUND_BF16>(w[u], s, out, j + u * stride);
      if constexpr (PAIR) cast_vec<IN, OUT2, ROUND_BF16>(w[u], s2, out2, j + u * stride);
    }
  };
  if (whole_batch_at(i)) {
    u32x4 wa[P], wb[P];
    load_batch(wa, i);
    for (;;) {
      if (!whole_batch_at(i + step)) { cast_batch(wa, i); i += step; break; }
      load_batch(wb, i + step);
      cast_batch(wa, i);
      i += step;
      if (!whole_batch_at(i + step)) { cast_batch(wb, i); i += step; break; }
      load_batch(wa, i + step);
      cast_batch(wb, i);
      i += step;
    }
  }
  for (; i < nvec; i += stride) {
    u32x4 w = ld_stream(v + i);
    cast_vec<IN, OUT, ROUND_BF16>(w, s, out, i);
    if constexpr (PAIR) cast_vec<IN, OUT2, ROUND_BF16>(w, s2, out2, i);
  }
  if (blockIdx.x == 0 && threadIdx.x < tail) {
    const int64_t e = nvec * kV + threadIdx.x;
    out[e] = cast_one<IN, OUT, ROUND_BF16>(x, e, s);
    if constexpr (PAIR) out2[e] = cast_one<IN, OUT2, ROUND_BF16>(x, e, s2);
  }
}

// Any alignment (x aligned to its element, the outputs to a byte): the same 16-byte loads and packed
// stores, through vector types that claim no more alignment than that.  The device serves such
// accesses (unaligned access mode, the default for compute on ROCm); they cost the lines they
// straddle.  8192^2 bf16 with x one element off: 182 us with one element per lane and step.
typedef u32x4 u32x4_elem2 __attribute__((aligned(2)));
typedef u32x4 u32x4_elem4 __attribute__((aligned(4)));
typedef u32x2 u32x2_byte __attribute__((aligned(1)));
typedef uint32_t u32_byte __attribute__((aligned(1)));
template <int IN, int OUT, bool ROUND_BF16, bool ROUND_SCALE, bool PAIR>
__global__ __launch_bounds__(kBlock) void cast_kernel_unaligned(const void* __restrict__ x, int64_t numel,
                                                                const float* __restrict__ scale,
                                                                uint8_t* __restrict__ out, uint8_t* __restrict__ out2) {
  constexpr int kV = InTraits<IN>::kVec;
  constexpr int OUT2 = OUT == DT_E4M3FN ? DT_E5M2 : DT_E4M3FN;
  typedef typename std::conditional<IN == DT_F32, u32x4_elem4, u32x4_elem2>::type vec_t;
  saturate_fp8_conversions();
  float s = scale[0], s2 = PAIR ? scale[1] : 0.f;
  if constexpr (ROUND_SCALE) { s = round_to_bf16(s); s2 = round_to_bf16(s2); }
  const vec_t* v = static_cast<const vec_t*>(x);
  const int64_t nvec = numel / kV, tail = numel % kV;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  auto put = [](uint8_t* o, int64_t i, const uint32_t (&r)[kV / 4]) {
    if constexpr (IN == DT_F32) *reinterpret_cast<u32_byte*>(o + i * 4) = r[0];
    else *reinterpret_cast<u32x2_byte*>(o + i * 8) = u32x2{r[0], r[1]};
  };
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += stride) {
    const u32x4 w = v[i];
    uint32_t r[kV / 4];
    cast_vec_to_words<IN, OUT, ROUND_BF16>(w, s, r);
    put(out, i, r);
    if constexpr (PAIR) {
      cast_vec_to_words<IN, OUT2, ROUND_BF16>(w, s2, r);
      put(out2, i, r);
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < tail) {
    const int64_t e = nvec * kV + threadIdx.x;
    out[e] = cast_one<IN, OUT, ROUND_BF16>(x, e, s);
    if constexpr (PAIR) out2[e] = cast_one<IN, OUT2, ROUND_BF16>(x, e, s2);
  }
}

template <int IN, int OUT, bool ROUND_BF16, bool ROUND_SCALE, bool PAIR>
inline int launch_cast_impl(const void* x, int64_t numel, const float* scale, void* out, void* out2,
                            hipStream_t stream) {
  // Large tensors: batches of 4 loads per lane, software-pipelined (4..8 in flight), from ONE workgroup per
  // CU: the best point of the measured grid {1, 2, 4 workgroups per CU} (8192^2 bf16 32.5 / 32.9 / 36.0 us,
  // fp32 54.2 / 60.1 / 66 us, bf16 to both fp8 types 45.1 / 45.3 / 47.8 us); more in flight is slower.
  // Below 64 MiB of input, where the 3 us a launch costs whatever its size (launch, first round trip,
  // drain) weigh more: batches of 2 from three workgroups per CU, which reach their full rate sooner
  // (us, rotated buffers, batches of 4 and 1 workgroup per CU against this: bf16 4096^2 10.1 -> 9.6,
  // 2048^2 4.2 -> 3.9; no difference from 64 MiB on).  The knobs force either (0 = by size).
  constexpr size_t kStoreAlign = IN == DT_F32 ? 4 : 8;
  uint8_t* o = static_cast<uint8_t*>(out);
  uint8_t* o2 = static_cast<uint8_t*>(out2);
  const bool fast = aligned(x, 16) && aligned(out, kStoreAlign) && (!PAIR || aligned(out2, kStoreAlign));
  if (fast) {
    const int64_t nvec = numel / InTraits<IN>::kVec, tail = numel % InTraits<IN>::kVec;
    const bool small = nvec * 16 < (int64_t)64 << 20;
    const int unroll_knob = tuning("cast.unroll");
    const int unroll = unroll_knob == 2 || unroll_knob == 4 ? unroll_knob : (small && !PAIR ? 2 : 4);
    const char* const knob = PAIR ? "cast.pair_blocks_per_cu" : "cast.blocks_per_cu";
    const int per_cu = tuning(knob) > 0 ? tuning(knob) : (small && !PAIR ? 3 : 1);
    int64_t grid = ceil_div(nvec, (int64_t)kBlock * unroll);
    if (grid > (int64_t)device_facts().cu_count * per_cu) grid = (int64_t)device_facts().cu_count * per_cu;
    if (grid < 1) grid = 1;
    if (unroll == 2) cast_kernel<IN, OUT, ROUND_BF16, ROUND_SCALE, PAIR, 2><<<(unsigned)grid, kBlock, 0, stream>>>(x, nvec, tail, scale, o, o2);
    else cast_kernel<IN, OUT, ROUND_BF16, ROUND_SCALE, PAIR, 4><<<(unsigned)grid, kBlock, 0, stream>>>(x, nvec, tail, scale, o, o2);
  } else {
    int64_t grid = ceil_div(numel / InTraits<IN>::kVec, (int64_t)kBlock);
    if (grid > device_facts().cu_count) grid = device_facts().cu_count;
    if (grid < 1) grid = 1;
    cast_kernel_unaligned<IN, OUT, ROUND_BF16, ROUND_SCALE, PAIR><<<(unsigned)grid, kBlock, 0, stream>>>(x, numel, scale, o, o2);
  }
  return launch_status();
}

// Runtime (in_dtype, out_dtype, round_mode) -> template instance.  `pair` adds out2 of the
// other fp8 type with scale[1].
template <bool PAIR>
inline int launch_cast(const void* x, int in_dtype, int64_t numel, const float* scale, int out_dtype,
                       int round_mode, void* out, void* out2, hipStream_t stream) {
#define DT_CAST(IN, OUT, RB, RS) return launch_cast_impl<IN, OUT, RB, RS, PAIR>(x, numel, scale, out, out2, stream)
  if (in_dtype == DT_F32) {
    if (out_dtype == DT_E4M3FN) DT_CAST(DT_F32, DT_E4M3FN, false, false);
    DT_CAST(DT_F32, DT_E5M2, false, false);
  }
  if (round_mode == DT_ROUND_F32) {
    if (out_dtype == DT_E4M3FN) DT_CAST(DT_BF16, DT_E4M3FN, false, false);
    DT_CAST(DT_BF16, DT_E5M2, false, false);
  }
  if (round_mode == DT_ROUND_BF16_PRODUCT) {
    if (out_dtype == DT_E4M3FN) DT_CAST(DT_BF16, DT_E4M3FN, true, false);
    DT_CAST(DT_BF16, DT_E5M2, true, false);
  }
  if (out_dtype == DT_E4M3FN) DT_CAST(DT_BF16, DT_E4M3FN, true, true);
  DT_CAST(DT_BF16, DT_E5M2, true, true);
#undef DT_CAST
}

inline int check_cast_args(const void* x, int in_dtype, int64_t numel, int out_dtype, int round_mode, const void* out) {
  if (in_dtype != DT_F32 && in_dtype != DT_BF16) return DT_ERR_INVALID_DTYPE;
  if (out_dtype != DT_E4M3FN && out_dtype != DT_E5M2) return DT_ERR_INVALID_DTYPE;
  if (round_mode < DT_ROUND_BF16_PRODUCT || round_mode > DT_ROUND_F32) return DT_ERR_INVALID_MODE;
  if (numel < 0) return DT_ERR_INVALID_SHAPE;
  if (numel > 0 && (!x || !out)) return DT_ERR_NULL_POINTER;
  if (!aligned(x, in_dtype == DT_F32 ? 4 : 2)) return DT_ERR_MISALIGNED;
  return DT_OK;
}

inline int check_workspace(const void* ws, size_t bytes) {
  if (!ws) return DT_ERR_WORKSPACE;
  if (bytes < kWsBytes) return DT_ERR_WORKSPACE;
  if (!aligned(ws, 256)) return DT_ERR_MISALIGNED;
  return DT_OK;
}

}  // namespace dt
