// Device-side building blocks shared by the gfx950 kernels: 16-byte vector access, bf16/f16
// unpacking, OCP fp8 packing with the hardware converts, wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "driss_torch_hip.h"

namespace dt {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

__device__ __forceinline__ float as_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __float_as_uint(f); }

// ------------------------------------------------------------------ streaming access
// Non-temporal (streaming) global access: the tensors of this path are touched once, and on
// MI355X the nt hint is worth ~10% of achieved HBM bandwidth over plain loads and stores.
template <typename T>
__device__ __forceinline__ T ld_stream(const T* p) { return __builtin_nontemporal_load(p); }
template <typename T>
__device__ __forceinline__ void st_stream(T* p, T v) { __builtin_nontemporal_store(v, p); }
// NT selects between a streaming and a cached load (the latter when a second pass re-reads)
// One 4-byte store per lane (the fp8 bytes of four fp32 inputs): written back through L2, which
// merges the lanes' words into lines; measured 3-4 % faster than the streaming form for these
// (MX casts of fp32 8192 x 8192: 53.5 vs 55.5 us), while 8- and 16-byte stores are faster streamed --
// and so are the 4-byte stores of the per-tensor casts (two-kernel step 99 vs 120 us): measured per site.
__device__ __forceinline__ void st_words(uint32_t* p, uint32_t v) { *p = v; }

template <bool NT, typename T>
__device__ __forceinline__ T ld_maybe_stream(const T* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p); else return *p;
}

// ------------------------------------------------------------------ element unpacking
// A 32-bit word holds two bf16 / f16 values; lo = element with the lower address.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return as_f32(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return as_f32(w & 0xFFFF0000u); }
__device__ __forceinline__ float f16_lo(uint32_t w) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu));
}
__device__ __forceinline__ float f16_hi(uint32_t w) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
}

// fp32 -> bf16 -> fp32, round to nearest even, NaN stays NaN: v_cvt_pk_bf16_f32 (checked on
// gfx950 against torch's conversion over all bf16 patterns and a dense fp32 sweep).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
__device__ __forceinline__ float round_to_bf16(float f) { return as_f32(pack_bf16x2(f, 0.f) << 16); }
// round two products at once
__device__ __forceinline__ void round2_to_bf16(float& a, float& b) {
  const uint32_t d = pack_bf16x2(a, b);
  a = as_f32(d << 16);
  b = as_f32(d & 0xFFFF0000u);
}

// ------------------------------------------------------------------------ fp8 packing
template <int OUT>
__device__ __forceinline__ constexpr float fp8_max() {
  return OUT == DT_E5M2 ? 57344.0f : 448.0f;
}

// clamp to +-fmax with one v_med3_f32.  A NaN input does not survive med3, so callers that
// must keep NaN patch the converted byte afterwards (see pack2 below).
template <int OUT>
__device__ __forceinline__ float clamp_fp8(float p) {
  return __builtin_amdgcn_fmed3f(p, -fp8_max<OUT>(), fp8_max<OUT>());
}

// Two floats -> two fp8 bytes in the low (HI=false) or high (HI=true) half of `old`, using
// v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32 (round to nearest even, OCP encodings on gfx950).
template <int OUT, bool HI>
__device__ __forceinline__ uint32_t cvt_pk(float a, float b, uint32_t old) {
  if constexpr (OUT == DT_E5M2)
    return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, HI);
  else
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
}

// Saturating convert of four finite-or-infinite products to four packed fp8 bytes (byte i =
// p_i).  A NaN does not survive the med3 clamp: callers test for NaN and call nan_patch4.
template <int OUT>
__device__ __forceinline__ uint32_t pack4_clamped(float p0, float p1, float p2, float p3) {
  uint32_t w = cvt_pk<OUT, false>(clamp_fp8<OUT>(p0), clamp_fp8<OUT>(p1), 0u);
  return cvt_pk<OUT, true>(clamp_fp8<OUT>(p2), clamp_fp8<OUT>(p3), w);
}

// NaN products become the canonical fp8 NaN with the product's sign (0x7F / 0xFF), which is
// what `.to(torch.float8_*)` produces after the where-clamps leave a NaN in place.  (The
// hardware convert would give 0xFF / 0xFE whatever the sign.)  Rare path.
__device__ __noinline__ uint32_t nan_patch4(uint32_t w, float p0, float p1, float p2, float p3) {
  auto fix = [&](float p, int sh) {
    if (p != p) w = (w & ~(0xFFu << sh)) | ((0x7Fu | ((as_u32(p) >> 24) & 0x80u)) << sh);
  };
  fix(p0, 0); fix(p1, 8); fix(p2, 16); fix(p3, 24);
  return w;
}

template <int OUT>
__device__ __forceinline__ uint32_t pack4(float p0, float p1, float p2, float p3) {
  uint32_t w = pack4_clamped<OUT>(p0, p1, p2, p3);
  const bool any_nan = (p0 != p0) | (p1 != p1) | (p2 != p2) | (p3 != p3);
  if (__builtin_expect(any_nan, 0)) w = nan_patch4(w, p0, p1, p2, p3);
  return w;
}

// -------------------------------------------------------- scaled, saturating fp8 converts
// Conversions that apply a power-of-two scale themselves (v_cvt_scalef32_pk_{fp8,bf8}_{bf16,f16,f32}).
// One instruction turns two inputs into two fp8 bytes of x / 2^(b-127), rounded to nearest even.
// With MODE.FP16_OVFL set they saturate (infinity included) instead of producing NaN / infinity,
// which makes them bit-identical to multiply, clamp, convert for every non-NaN input and every
// scale byte 0..248 (checked exhaustively over all bf16 and f16 patterns and 9 x 65536 fp32
// patterns per byte on the hardware).  A NaN input gives a NaN code other than 0x7F / 0xFF, so
// callers that can meet a NaN patch or overwrite those bytes.  With a scale of 1.0f they are the
// plain saturating convert without the v_med3_f32 clamp, and bf16 products can be converted
// straight from the packed pair v_cvt_pk_bf16_f32 leaves.
typedef short v2s16 __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf16 __attribute__((ext_vector_type(2)));
typedef _Float16 v2f16 __attribute__((ext_vector_type(2)));

// every wave of a kernel that uses them calls this first (the mode register is per wave)
__device__ __forceinline__ void saturate_fp8_conversions() { __builtin_amdgcn_s_setreg(1 | (23 << 6), 1); }

// two 16-bit inputs packed in one word -> bytes 0-1 (HI false) or 2-3 (HI true) of old
template <int IN, int OUT, bool HI>
__device__ __forceinline__ uint32_t cvt_scaled_pair16(uint32_t old, uint32_t pair, float scale) {
  static_assert(IN == DT_BF16 || IN == DT_F16, "16-bit inputs");
  const v2s16 o = __builtin_bit_cast(v2s16, old);
  v2s16 r;
  if constexpr (IN == DT_BF16) {
    const v2bf16 x = __builtin_bit_cast(v2bf16, pair);
    if constexpr (OUT == DT_E5M2) r = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(o, x, scale, HI);
    else r = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o, x, scale, HI);
  } else {
    const v2f16 x = __builtin_bit_cast(v2f16, pair);
    if constexpr (OUT == DT_E5M2) r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(o, x, scale, HI);
    else r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(o, x, scale, HI);
  }
  return __builtin_bit_cast(uint32_t, r);
}
template <int OUT, bool HI>
__device__ __forceinline__ uint32_t cvt_scaled_pair32(uint32_t old, uint32_t a, uint32_t b, float scale) {
  const v2s16 o = __builtin_bit_cast(v2s16, old);
  v2s16 r;
  if constexpr (OUT == DT_E5M2) r = __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(o, as_f32(a), as_f32(b), scale, HI);
  else r = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, as_f32(a), as_f32(b), scale, HI);
  return __builtin_bit_cast(uint32_t, r);
}
// four 16-bit inputs in two words, or four fp32 words -> one word of fp8, all with one scale
template <int IN, int OUT>
__device__ __forceinline__ uint32_t cvt_scaled_4x16(uint32_t w0, uint32_t w1, float scale) {
  return cvt_scaled_pair16<IN, OUT, true>(cvt_scaled_pair16<IN, OUT, false>(w0, w0, scale), w1, scale);
}
template <int OUT>
__device__ __forceinline__ uint32_t cvt_scaled_4x32(uint32_t a, uint32_t b, uint32_t c, uint32_t d, float scale) {
  return cvt_scaled_pair32<OUT, true>(cvt_scaled_pair32<OUT, false>(a, a, b, scale), c, d, scale);
}
// e2m1 (fp4): v_cvt_scalef32_pk_fp4_* converts two values of x / 2^(e-127) into one byte (first value
// in the low nibble), round to nearest even, saturating at +-6; NaN becomes +-6, there being no NaN
// code.  Measured on gfx950 against a host restatement: every bf16 pattern and 2^20 fp32 values,
// scale bytes 0..254, bit-identical; the other three bytes of the word are left as they were.
constexpr int DT_E2M1 = 2;  // internal output code (the public out-dtype enum covers the fp8 types)
template <int IN>
__device__ __forceinline__ uint32_t cvt_fp4_8x16(u32x4 w, float scale) {  // 8 elements -> 4 bytes
  static_assert(IN == DT_BF16 || IN == DT_F16, "16-bit inputs");
  // Each word goes through an empty asm first: handed the words of a 16-byte vector directly, hipcc
  // (ROCm 7.2) selects the vector's FIRST word as the source of all four conversions.
  uint32_t x = w.x, y = w.y, z = w.z, v = w.w;
  asm("" : "+v"(x));
  asm("" : "+v"(y));
  asm("" : "+v"(z));
  asm("" : "+v"(v));
  uint32_t r = 0;
  if constexpr (IN == DT_BF16) {
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(v2bf16, x), scale, 0);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(v2bf16, y), scale, 1);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(v2bf16, z), scale, 2);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(v2bf16, v), scale, 3);
  } else {
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(v2f16, x), scale, 0);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(v2f16, y), scale, 1);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(v2f16, z), scale, 2);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(v2f16, v), scale, 3);
  }
  return r;
}
// one pair into byte `sel` (0..3) of `old`
template <int IN>
__device__ __forceinline__ uint32_t cvt_fp4_pair16(uint32_t old, uint32_t pair, float scale, int sel) {
  static_assert(IN == DT_BF16 || IN == DT_F16, "16-bit inputs");
  asm("" : "+v"(pair));  // see cvt_fp4_8x16
  if constexpr (IN == DT_BF16) {
    const v2bf16 x = __builtin_bit_cast(v2bf16, pair);
    return sel == 0 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, x, scale, 0)
         : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, x, scale, 1)
         : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, x, scale, 2)
                    : __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(old, x, scale, 3);
  } else {
    const v2f16 x = __builtin_bit_cast(v2f16, pair);
    return sel == 0 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, x, scale, 0)
         : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, x, scale, 1)
         : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, x, scale, 2)
                    : __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(old, x, scale, 3);
  }
}
__device__ __forceinline__ uint32_t cvt_fp4_pair32(uint32_t old, uint32_t a, uint32_t b, float scale, int sel) {
  const float x = as_f32(a), y = as_f32(b);
  return sel == 0 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, x, y, scale, 0)
       : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, x, y, scale, 1)
       : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, x, y, scale, 2)
                  : __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, x, y, scale, 3);
}
__device__ __forceinline__ uint32_t cvt_fp4_4x32(u32x4 w, float scale) {  // 4 elements -> 2 bytes (low half)
  uint32_t r = 0;
  r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, as_f32(w.x), as_f32(w.y), scale, 0);
  r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, as_f32(w.z), as_f32(w.w), scale, 1);
  return r;
}

// Product x*scale under the three rounding modes of dt_round_mode.  `sb` is the scale
// already rounded for the mode (bf16-rounded for mode 2), so modes 1 and 2 share code.
template <bool ROUND_PRODUCT_TO_BF16>
__device__ __forceinline__ float scaled(float x, float s) {
  float p = x * s;
  if constexpr (ROUND_PRODUCT_TO_BF16) p = round_to_bf16(p);
  return p;
}

// -------------------------------------------------------------------- wave reductions
// DPP cross-lane moves.  bound_ctrl=true makes invalid source lanes read 0, which is the
// identity for an unsigned max.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// max over the 4 lanes of a quad, result in all 4 lanes
__device__ __forceinline__ uint32_t quad_umax(uint32_t v) {
  v = umax(v, dpp<kDppQuadXor1>(v));
  v = umax(v, dpp<kDppQuadXor2>(v));
  return v;
}

// max over all 64 lanes, result in every lane: 4 DPP steps inside a row of 16, then two
// ds_swizzle/bpermute exchanges across rows.
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
  v = quad_umax(v);
  v = umax(v, dpp<kDppRowHalfMirror>(v));
  v = umax(v, dpp<kDppRowMirror>(v));
  v = umax(v, (uint32_t)__shfl_xor((int)v, 16, kWave));
  v = umax(v, (uint32_t)__shfl_xor((int)v, 32, kWave));
  return v;
}

// max over a workgroup of NWAVES waves through LDS; result valid in every thread.
template <int NWAVES>
__device__ __forceinline__ uint32_t block_umax(uint32_t v, uint32_t* lds /* >= NWAVES words */) {
  v = wave_umax(v);
  if constexpr (NWAVES == 1) return v;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  uint32_t r = lds[0];
#pragma unroll
  for (int i = 1; i < NWAVES; ++i) r = umax(r, lds[i]);
  __syncthreads();
  return r;
}

// ------------------------------------------------------------------- magnitudes as ints
// |x| of IEEE floats orders like its bit pattern read as an unsigned integer, and every
// NaN pattern sorts above infinity, so an integer max both finds the amax and propagates NaN.
__device__ __forceinline__ uint32_t absbits_f32(uint32_t w) { return w & 0x7FFFFFFFu; }

// max |.| of the two bf16/f16 halves of a word, as a 16-bit pattern in each half (v_pk_max_u16)
__device__ __forceinline__ uint32_t pk_absmax16(uint32_t acc, uint32_t w) {
  u16x2 a = __builtin_bit_cast(u16x2, acc);
  u16x2 b = __builtin_bit_cast(u16x2, w & 0x7FFF7FFFu);
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}

// amax -> scale exactly as f32(fmax / max(f64(amax), 1e-12)); NaN propagates.
__device__ __forceinline__ float amax_to_scale(float amax, float fmax) {
  double a = (double)amax;
  double c = (a != a) ? a : (a < 1e-12 ? 1e-12 : a);
  return (float)((double)fmax / c);
}

}  // namespace dt
