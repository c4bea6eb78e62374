// torch.ops.DrissTorch registration for PyTorch-ROCm.
//
// Keeps the operator schemas of the reference's src/register_ops.cpp:13-43 (same names,
// argument lists and dispatch key; on PyTorch-ROCm the CUDA key is the HIP device) and does
// what the reference's host functions do around their launches -- argument checks that
// raise RuntimeError, output allocation from the torch allocator, stream selection -- and
// nothing else: all device work goes through the C ABI in include/driss_torch_hip.h.
// Unlike the reference (legacy default stream, no guard: src/amax.cu:92,
// src/saturated_cast.cu:20, src/mx_cast.cu:238) every op runs on the current stream of the
// input's device.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DispatchKey.h>
#include <torch/library.h>

#include <map>
#include <mutex>
#include <tuple>

#include "driss_torch_hip.h"

namespace driss_torch {
using at::Tensor;

namespace {

struct Ctx {
  c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard;
  dt_stream_t stream;
  explicit Ctx(const Tensor& t) : guard(t.device()) {
    stream = reinterpret_cast<dt_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
  }
};

void check_status(int st, const char* what) {
  TORCH_CHECK(st == DT_OK, what, ": ", dt_status_string(st));
}

int in_code(const Tensor& t) {
  switch (t.scalar_type()) {
    case at::kFloat: return DT_F32;
    case at::kBFloat16: return DT_BF16;
    case at::kHalf: return DT_F16;
    default: TORCH_CHECK(false, "unsupported input dtype ", t.dtype());
  }
}

int out_code(at::ScalarType dtype) {  // src/saturated_cast.cu:155-164, src/dynamic_scaled_quant.cu:65-74
  switch (dtype) {
    case at::kFloat8_e4m3fn: return DT_E4M3FN;
    case at::kFloat8_e5m2: return DT_E5M2;
    default: TORCH_CHECK(false, "Invalid dtype");
  }
}

// One reduction workspace per (device, stream), zero-initialised once and then re-armed by
// the kernels themselves.  Leaked on purpose: tensors must not be destroyed after the HIP
// runtime has shut down.
Tensor& workspace_for(const Tensor& like, dt_stream_t stream) {
  static std::mutex mu;
  static auto* cache = new std::map<std::pair<int, void*>, Tensor>();
  std::lock_guard<std::mutex> lock(mu);
  auto key = std::make_pair((int)like.get_device(), (void*)stream);
  auto it = cache->find(key);
  if (it == cache->end()) {
    Tensor ws = at::zeros({(int64_t)dt_workspace_bytes()}, like.options().dtype(at::kByte));
    it = cache->emplace(key, ws).first;
  }
  return it->second;
}

// The same for the GEMM's split-K workspace (ticket counters that the kernel leaves zero, and
// parked accumulators).
Tensor& gemm_workspace_for(const Tensor& like, dt_stream_t stream) {
  static std::mutex mu;
  static auto* cache = new std::map<std::pair<int, void*>, Tensor>();
  std::lock_guard<std::mutex> lock(mu);
  auto key = std::make_pair((int)like.get_device(), (void*)stream);
  auto it = cache->find(key);
  if (it == cache->end()) {
    Tensor ws = at::zeros({(int64_t)dt_mx_gemm_workspace_bytes()}, like.options().dtype(at::kByte));
    it = cache->emplace(key, ws).first;
  }
  return it->second;
}

void check_hp_input(const Tensor& input) {
  TORCH_CHECK(input.is_cuda(), "Input tensor must be on the GPU");
  TORCH_CHECK(input.scalar_type() == at::kBFloat16 || input.scalar_type() == at::kFloat,
              "Input tensor must be of type BFloat16 or Float, but got ", input.dtype());
  TORCH_CHECK(input.dim() == 2, "Input tensor must be 2D, but got ", input.dim());
}

void check_fp8(at::ScalarType dtype) {
  TORCH_CHECK(dtype == at::kFloat8_e4m3fn || dtype == at::kFloat8_e5m2,
              "Output tensor must be of type Float8_e4m3fn or Float8_e5m2");
}

}  // namespace

// ------------------------------------------------------------------------------ amax
// src/amax.cu:106-119.  The even-numel restriction of :113 is lifted.
Tensor amax(const Tensor& input) {
  check_hp_input(input);
  TORCH_CHECK(input.numel() > 0, "amax of an empty tensor");
  Ctx ctx(input);
  Tensor x = input.is_non_overlapping_and_dense() ? input : input.contiguous();
  Tensor out = at::empty({1}, input.options().dtype(at::kFloat));
  Tensor& ws = workspace_for(input, ctx.stream);
  check_status(dt_amax(x.data_ptr(), in_code(x), x.numel(), out.data_ptr<float>(), ws.data_ptr(), ws.numel(), ctx.stream),
               "amax");
  return out;
}

// -------------------------------------------------------------------- saturated_cast
// src/saturated_cast.cu:227-252.  `mode` 0 picks the product rounding eager PyTorch would
// use for this scale tensor: 0-dim scale -> bf16 product with a bf16-rounded scale (which
// is also what the reference kernel computes, :66,81), rank >= 1 -> fp32 product.
Tensor saturated_cast_mode(const Tensor& input, const Tensor& scale, at::ScalarType dtype, bool transpose,
                           int64_t mode) {
  check_fp8(dtype);
  check_hp_input(input);
  TORCH_CHECK(scale.scalar_type() == at::kFloat, "Scale tensor must be of type Float, but got ", scale.dtype());
  TORCH_CHECK(scale.numel() == 1, "Scale tensor must be a scalar, but got ", scale.numel());
  TORCH_CHECK(scale.is_cuda() && scale.device() == input.device(), "Scale tensor must be on the input's device");
  TORCH_CHECK(!transpose, "Transpose is not supported yet");  // driss_torch/__init__.py:37
  TORCH_CHECK(mode >= 0 && mode <= 3, "invalid product rounding mode ", mode);
  // contiguous or column-major with zero offset is taken as is, in storage order (:243-247)
  auto strides = input.strides();
  const bool is_contiguous = input.is_contiguous();
  const bool is_transposed = strides[0] == 1 && strides[1] == input.size(0);
  const bool allowed = (is_contiguous || is_transposed) && input.storage_offset() == 0;
  Tensor x = allowed ? input : input.contiguous();
  Tensor out = at::empty_like(x, x.options().dtype(dtype));
  if (x.numel() == 0) return out;
  if (mode == 0) mode = scale.dim() == 0 ? DT_ROUND_BF16_SCALE_PRODUCT : DT_ROUND_F32;
  Ctx ctx(input);
  check_status(dt_saturated_cast(x.data_ptr(), in_code(x), x.numel(), scale.data_ptr<float>(), out_code(dtype), (int)mode,
                                 out.data_ptr(), ctx.stream),
               "saturated_cast");
  return out;
}

Tensor saturated_cast(const Tensor& input, const Tensor& scale, at::ScalarType dtype, bool transpose) {
  return saturated_cast_mode(input, scale, dtype, transpose, 0);
}

// -------------------------------------------------------------- dynamic_scaled_quant
// src/dynamic_scaled_quant.cu:157-176.  bf16 input follows eager with the 0-dim scale of
// tensor_to_scale (test/test_dynamic_quant.py:36): product and scale rounded to bf16.
std::tuple<Tensor, Tensor, Tensor> dynamic_scaled_quant_ex(const Tensor& input, at::ScalarType fp8_dtype, int64_t mode) {
  check_fp8(fp8_dtype);
  check_hp_input(input);
  TORCH_CHECK(input.is_contiguous());
  TORCH_CHECK(input.numel() > 0, "dynamic_scaled_quant of an empty tensor");
  TORCH_CHECK(mode >= 0 && mode <= 3, "invalid product rounding mode ", mode);
  if (mode == 0) mode = DT_ROUND_BF16_SCALE_PRODUCT;
  Ctx ctx(input);
  Tensor out = at::empty_like(input, input.options().dtype(fp8_dtype));
  Tensor amax_t = at::empty({1}, input.options().dtype(at::kFloat));
  Tensor scale_t = at::empty({}, input.options().dtype(at::kFloat));
  Tensor& ws = workspace_for(input, ctx.stream);
  check_status(dt_dynamic_scaled_quant(input.data_ptr(), in_code(input), input.numel(), out_code(fp8_dtype), (int)mode,
                                       out.data_ptr(), amax_t.data_ptr<float>(), scale_t.data_ptr<float>(),
                                       ws.data_ptr(), ws.numel(), ctx.stream),
               "dynamic_scaled_quant");
  return {out, amax_t, scale_t};
}

Tensor dynamic_scaled_quant(const Tensor& input, at::ScalarType fp8_dtype) {
  return std::get<0>(dynamic_scaled_quant_ex(input, fp8_dtype, 0));
}

// e4m3fn and e5m2 from one amax and one cast pass -> (e4m3fn, e5m2, amax[1], scale[2])
std::tuple<Tensor, Tensor, Tensor, Tensor> dynamic_scaled_quant_pair(const Tensor& input, int64_t mode) {
  check_hp_input(input);
  TORCH_CHECK(input.is_contiguous());
  TORCH_CHECK(input.numel() > 0, "dynamic_scaled_quant of an empty tensor");
  TORCH_CHECK(mode >= 0 && mode <= 3, "invalid product rounding mode ", mode);
  if (mode == 0) mode = DT_ROUND_BF16_SCALE_PRODUCT;
  Ctx ctx(input);
  Tensor o4 = at::empty_like(input, input.options().dtype(at::kFloat8_e4m3fn));
  Tensor o5 = at::empty_like(input, input.options().dtype(at::kFloat8_e5m2));
  Tensor amax_t = at::empty({1}, input.options().dtype(at::kFloat));
  Tensor scale_t = at::empty({2}, input.options().dtype(at::kFloat));
  Tensor& ws = workspace_for(input, ctx.stream);
  check_status(dt_dynamic_scaled_quant_pair(input.data_ptr(), in_code(input), input.numel(), (int)mode, o4.data_ptr(),
                                            o5.data_ptr(), amax_t.data_ptr<float>(), scale_t.data_ptr<float>(),
                                            ws.data_ptr(), ws.numel(), ctx.stream),
               "dynamic_scaled_quant_pair");
  return {o4, o5, amax_t, scale_t};
}

// per-row scales -> (fp8 [R,C], amax [R,1], scale [R,1])
std::tuple<Tensor, Tensor, Tensor> dynamic_scaled_quant_rowwise(const Tensor& input, at::ScalarType fp8_dtype) {
  check_fp8(fp8_dtype);
  check_hp_input(input);
  TORCH_CHECK(input.is_contiguous());
  TORCH_CHECK(input.size(0) == 0 || input.size(1) > 0, "rowwise amax over empty rows");
  Ctx ctx(input);
  const int64_t R = input.size(0), C = input.size(1);
  Tensor out = at::empty_like(input, input.options().dtype(fp8_dtype));
  Tensor amax_t = at::empty({R, 1}, input.options().dtype(at::kFloat));
  Tensor scale_t = at::empty({R, 1}, input.options().dtype(at::kFloat));
  check_status(dt_dynamic_scaled_quant_rowwise(input.data_ptr(), in_code(input), R, C, out_code(fp8_dtype), out.data_ptr(),
                                               amax_t.data_ptr<float>(), scale_t.data_ptr<float>(), ctx.stream),
               "dynamic_scaled_quant_rowwise");
  return {out, amax_t, scale_t};
}

// ------------------------------------------------------------------- mx_fp8_quantize
// src/mx_cast.cu:168-246.  The reference accepts block_size / axis / transpose / fp8_type
// and ignores them (:148,193,216,237); here they are honoured.  `blocked` writes the
// scales in the layout mx_fp8_bf16 reads.
std::tuple<Tensor, Tensor> mx_fp8_quantize_ex(const Tensor& input, int64_t block_size, int64_t axis, bool transpose,
                                              at::ScalarType fp8_type, bool blocked) {
  TORCH_CHECK(input.is_cuda(), "Input tensor must be a CUDA tensor");
  TORCH_CHECK(input.is_contiguous(), "Input tensor must be contiguous");
  TORCH_CHECK(input.scalar_type() == at::kHalf || input.scalar_type() == at::kFloat ||
                  input.scalar_type() == at::kBFloat16,
              "Input tensor must be float, half, or bfloat16");
  TORCH_CHECK(block_size > 0 && block_size <= 32, "Block size must be positive and <= 32");
  TORCH_CHECK(block_size == 32, "Only block size 32 is implemented");
  TORCH_CHECK(input.dim() == 2, "Only support 2d tensor for now");
  TORCH_CHECK(fp8_type == at::kFloat8_e4m3fn || fp8_type == at::kFloat8_e5m2,
              "FP8 type must be Float8_e4m3fn or Float8_e5m2");
  TORCH_CHECK(axis >= -2 && axis <= 1, "axis must be one of -2, -1, 0, 1");
  const int ax = (int)((axis + 2) % 2);
  const int64_t m = input.size(0), n = input.size(1);
  const int64_t blocked_dim = ax == 1 ? n : m, other_dim = ax == 1 ? m : n;
  TORCH_CHECK(blocked_dim % 32 == 0, "Need block shape to evenly divide the input tensor for now");
  TORCH_CHECK(!blocked || (ax == 1) != transpose,
              "blocked scales need the scale matrix as [outer, inner/32]: (axis 1, no transpose) or (axis 0, transpose)");
  Ctx ctx(input);
  Tensor data = transpose ? at::empty({n, m}, input.options().dtype(fp8_type))
                          : at::empty({m, n}, input.options().dtype(fp8_type));
  const int64_t total_blocks = other_dim * (blocked_dim / 32);
  const int64_t scale_elems = blocked ? dt_blocked_scale_bytes(other_dim, blocked_dim / 32) : total_blocks;
  Tensor scale = at::empty({scale_elems}, input.options().dtype(at::kFloat8_e8m0fnu));
  if (input.numel() == 0) return {data, scale};
  check_status(dt_mx_fp8_quantize(input.data_ptr(), in_code(input), m, n, ax, transpose ? 1 : 0, out_code(fp8_type),
                                  blocked ? DT_SCALE_BLOCKED : DT_SCALE_PLAIN, data.data_ptr(),
                                  static_cast<uint8_t*>(scale.data_ptr()), ctx.stream),
               "mx_fp8_quantize");
  return {data, scale};
}

// Both blockings of one tensor from a single read: (data [M,N], scale [M,N/32]) along the rows and
// (data [N,M], scale [N,M/32]) down the columns with the payload transposed.  Same checks as
// mx_fp8_quantize (src/mx_cast.cu:171-219) applied to both dimensions.
std::tuple<Tensor, Tensor, Tensor, Tensor> mx_fp8_quantize_dual(const Tensor& input, at::ScalarType fp8_type, bool blocked) {
  TORCH_CHECK(input.is_cuda(), "Input tensor must be a CUDA tensor");
  TORCH_CHECK(input.is_contiguous(), "Input tensor must be contiguous");
  TORCH_CHECK(input.scalar_type() == at::kHalf || input.scalar_type() == at::kFloat ||
                  input.scalar_type() == at::kBFloat16,
              "Input tensor must be float, half, or bfloat16");
  TORCH_CHECK(input.dim() == 2, "Only support 2d tensor for now");
  TORCH_CHECK(fp8_type == at::kFloat8_e4m3fn || fp8_type == at::kFloat8_e5m2,
              "FP8 type must be Float8_e4m3fn or Float8_e5m2");
  const int64_t m = input.size(0), n = input.size(1);
  TORCH_CHECK(m % 32 == 0 && n % 32 == 0, "Need block shape to evenly divide the input tensor for now");
  Ctx ctx(input);
  const auto fp8 = input.options().dtype(fp8_type);
  const auto e8 = input.options().dtype(at::kFloat8_e8m0fnu);
  Tensor data_r = at::empty({m, n}, fp8), data_c = at::empty({n, m}, fp8);
  Tensor scale_r = at::empty({blocked ? dt_blocked_scale_bytes(m, n / 32) : m * (n / 32)}, e8);
  Tensor scale_c = at::empty({blocked ? dt_blocked_scale_bytes(n, m / 32) : n * (m / 32)}, e8);
  if (input.numel() == 0) return {data_r, scale_r, data_c, scale_c};
  check_status(dt_mx_fp8_quantize_dual(input.data_ptr(), in_code(input), m, n, out_code(fp8_type),
                                       blocked ? DT_SCALE_BLOCKED : DT_SCALE_PLAIN, data_r.data_ptr(),
                                       static_cast<uint8_t*>(scale_r.data_ptr()), data_c.data_ptr(),
                                       static_cast<uint8_t*>(scale_c.data_ptr()), ctx.stream),
               "mx_fp8_quantize_dual");
  return {data_r, scale_r, data_c, scale_c};
}

std::tuple<Tensor, Tensor> mx_fp8_quantize(Tensor input, int64_t block_size, int64_t axis, bool transpose,
                                           at::ScalarType fp8_type) {
  return mx_fp8_quantize_ex(input, block_size, axis, transpose, fp8_type, false);
}

// plain [R, C] E8M0 scales -> blocked layout; stands in for to_blocked of test/test_mx.py:31-32
Tensor to_blocked(const Tensor& scale) {
  TORCH_CHECK(scale.is_cuda(), "scale must be on the GPU");
  TORCH_CHECK(scale.dim() == 2, "scale must be a matrix");
  TORCH_CHECK(scale.element_size() == 1, "scale must have a one-byte dtype");
  Tensor s = scale.contiguous();
  Ctx ctx(scale);
  const int64_t R = s.size(0), C = s.size(1);
  Tensor out = at::empty({dt_blocked_scale_bytes(R, C)}, s.options());
  check_status(dt_to_blocked(static_cast<const uint8_t*>(s.data_ptr()), R, C, static_cast<uint8_t*>(out.data_ptr()),
                             ctx.stream),
               "to_blocked");
  return out;
}

// -------------------------------------------------------------------- mx_fp4_quantize
// Operands for mx_fp4_bf16: packed e2m1 (uint8, first element of a pair in the low nibble) and E8M0
// scales per 32 elements: axis 1 along the rows -> [M, N/2]; axis 0 down the columns, transposed ->
// [N, M/2] (the axis-1 cast of input.t()).  No counterpart op in the reference, whose GEMM test takes them
// from torchao's MXTensor.to_mx(x, "fp4_e2m1", 32) (test/test_mx.py:17-21).
std::tuple<Tensor, Tensor> mx_fp4_quantize(const Tensor& input, bool blocked, int64_t axis) {
  TORCH_CHECK(input.is_cuda(), "Input tensor must be a CUDA tensor");
  TORCH_CHECK(input.is_contiguous(), "Input tensor must be contiguous");
  TORCH_CHECK(input.scalar_type() == at::kHalf || input.scalar_type() == at::kFloat ||
                  input.scalar_type() == at::kBFloat16,
              "Input tensor must be float, half, or bfloat16");
  TORCH_CHECK(input.dim() == 2, "Only support 2d tensor for now");
  TORCH_CHECK(axis >= -2 && axis < 2, "axis must be 0 or 1");
  const int ax = (int)((axis + 2) % 2);
  const int64_t m = input.size(0), n = input.size(1);
  const int64_t outer = ax == 1 ? m : n, inner = ax == 1 ? n : m;  // payload [outer, inner / 2]
  TORCH_CHECK(inner % 32 == 0, "Need block shape to evenly divide the input tensor for now");
  TORCH_CHECK(ax == 1 || n % 4 == 0, "The column-wise cast needs a multiple of 4 columns");
  Ctx ctx(input);
  Tensor data = at::empty({outer, inner / 2}, input.options().dtype(at::kByte));
  Tensor scale = at::empty({blocked ? dt_blocked_scale_bytes(outer, inner / 32) : outer * (inner / 32)},
                           input.options().dtype(at::kFloat8_e8m0fnu));
  if (input.numel() == 0) return {data, scale};
  TORCH_CHECK(reinterpret_cast<std::uintptr_t>(input.data_ptr()) % 16 == 0, "Input tensor must be 16-byte aligned");
  check_status(dt_mx_fp4_quantize(input.data_ptr(), in_code(input), m, n, ax, blocked ? DT_SCALE_BLOCKED : DT_SCALE_PLAIN,
                                  data.data_ptr(), static_cast<uint8_t*>(scale.data_ptr()), ctx.stream),
               "mx_fp4_quantize");
  return {data, scale};
}

// Both MXFP4 operands of one tensor from a single read: mx_fp4_quantize(input, blocked, 1) and
// mx_fp4_quantize(input, blocked, 0).  No counterpart op in the reference (see mx_fp4_quantize).
std::tuple<Tensor, Tensor, Tensor, Tensor> mx_fp4_quantize_dual(const Tensor& input, bool blocked) {
  TORCH_CHECK(input.is_cuda(), "Input tensor must be a CUDA tensor");
  TORCH_CHECK(input.is_contiguous(), "Input tensor must be contiguous");
  TORCH_CHECK(input.scalar_type() == at::kHalf || input.scalar_type() == at::kFloat ||
                  input.scalar_type() == at::kBFloat16,
              "Input tensor must be float, half, or bfloat16");
  TORCH_CHECK(input.dim() == 2, "Only support 2d tensor for now");
  const int64_t m = input.size(0), n = input.size(1);
  TORCH_CHECK(m % 32 == 0 && n % 32 == 0, "Need block shape to evenly divide the input tensor for now");
  Ctx ctx(input);
  const auto u8 = input.options().dtype(at::kByte);
  const auto e8 = input.options().dtype(at::kFloat8_e8m0fnu);
  Tensor data_r = at::empty({m, n / 2}, u8), data_c = at::empty({n, m / 2}, u8);
  Tensor scale_r = at::empty({blocked ? dt_blocked_scale_bytes(m, n / 32) : m * (n / 32)}, e8);
  Tensor scale_c = at::empty({blocked ? dt_blocked_scale_bytes(n, m / 32) : n * (m / 32)}, e8);
  if (input.numel() == 0) return {data_r, scale_r, data_c, scale_c};
  TORCH_CHECK(reinterpret_cast<std::uintptr_t>(input.data_ptr()) % 16 == 0, "Input tensor must be 16-byte aligned");
  check_status(dt_mx_fp4_quantize_dual(input.data_ptr(), in_code(input), m, n, blocked ? DT_SCALE_BLOCKED : DT_SCALE_PLAIN,
                                       data_r.data_ptr(), static_cast<uint8_t*>(scale_r.data_ptr()), data_c.data_ptr(),
                                       static_cast<uint8_t*>(scale_c.data_ptr()), ctx.stream),
               "mx_fp4_quantize_dual");
  return {data_r, scale_r, data_c, scale_c};
}

// ------------------------------------------------------------------------ mx_fp8_bf16
// src/mx_fp8_bf16.cu:168-241
Tensor mx_fp8_bf16(Tensor a, Tensor b, Tensor a_scale, Tensor b_scale) {
  TORCH_CHECK(a.is_cuda(), "a must be CUDA tensor");
  TORCH_CHECK(b.is_cuda(), "b must be CUDA tensor");
  TORCH_CHECK(a_scale.is_cuda(), "a_scale must be CUDA tensor");
  TORCH_CHECK(b_scale.is_cuda(), "b_scale must be CUDA tensor");
  TORCH_CHECK(a.dim() == 2, "a must be a matrix");
  TORCH_CHECK(b.dim() == 2, "b must be a matrix");
  TORCH_CHECK(a.scalar_type() == at::kFloat8_e4m3fn && b.scalar_type() == at::kFloat8_e4m3fn,
              "a and b must be float8_e4m3fn");
  TORCH_CHECK(a_scale.element_size() == 1 && b_scale.element_size() == 1, "scales must be E8M0 bytes");
  const int64_t M = a.size(0), K = a.size(1), N = b.size(1);
  TORCH_CHECK(b.size(0) == K, "Incompatible matrix dimensions: a is ", M, "x", K, " but b is ", b.size(0), "x", N);
  TORCH_CHECK(N % 8 == 0, "N must be a multiple of 16 but got, ", N);
  TORCH_CHECK(K % 32 == 0, "K must be a multiple of the MX block size 32 but got ", K);
  TORCH_CHECK(reinterpret_cast<std::uintptr_t>(a.data_ptr()) % 16 == 0, "Input tensor 'a' must be 16-byte aligned");
  TORCH_CHECK(reinterpret_cast<std::uintptr_t>(b.data_ptr()) % 16 == 0, "Input tensor 'b' must be 16-byte aligned");
  // the length of the blocked layout: 128 ceil(M / 128) rows of 4 ceil(K / 128) bytes, which is the
  // reference's 128 ceil(M / 128) ceil(K / 32) (:197-205) whenever K is a multiple of 128
  const int64_t expected_a = dt_blocked_scale_bytes(M, K / 32);
  TORCH_CHECK(a_scale.numel() == expected_a, "Expected a_scale_size to be ", expected_a, " but got ", a_scale.numel());
  const int64_t expected_b = dt_blocked_scale_bytes(N, K / 32);
  TORCH_CHECK(b_scale.numel() == expected_b, "Expected b_scale_size to be ", expected_b, " but got ", b_scale.numel());
  TORCH_CHECK(a.stride(1) == 1, "Input tensor 'a' must be contiguous in the K dimension (row-major)");
  TORCH_CHECK(b.stride(0) == 1, "Input tensor 'b' must be contiguous in the K dimension (column-major)");
  TORCH_CHECK(a_scale.is_contiguous() && b_scale.is_contiguous(), "scales must be contiguous");
  Ctx ctx(a);
  Tensor out = at::empty({M, N}, a.options().dtype(at::kBFloat16));
  if (M == 0 || N == 0) return out;
  const int64_t lda = M > 1 ? a.stride(0) : K, ldb = N > 1 ? b.stride(1) : K;
  Tensor& ws = gemm_workspace_for(a, ctx.stream);
  check_status(dt_mx_fp8_bf16_ws(a.data_ptr(), b.data_ptr(), static_cast<const uint8_t*>(a_scale.data_ptr()),
                                 static_cast<const uint8_t*>(b_scale.data_ptr()), M, N, K, lda, ldb, out.data_ptr(), N,
                                 ws.data_ptr(), ws.numel(), ctx.stream),
               "mx_fp8_bf16");
  return out;
}

// ------------------------------------------------------------------------ mx_fp4_bf16
// src/mx_fp8_bf16.cu:243-271.  a [M, K/2] and b [K/2, N] with stride(0) == 1 hold two e2m1
// values per byte, the even element in the low nibble (uint8 or float4_e2m1fn_x2 storage);
// K = 2 * a.size(1) as at :254.  The reference runs no operand checks here; these are the
// checks of mx_fp8_bf16 (:168-214) applied to the unpacked K.
Tensor mx_fp4_bf16(Tensor a, Tensor b, Tensor a_scale, Tensor b_scale) {
  TORCH_CHECK(a.is_cuda(), "a must be CUDA tensor");
  TORCH_CHECK(b.is_cuda(), "b must be CUDA tensor");
  TORCH_CHECK(a_scale.is_cuda(), "a_scale must be CUDA tensor");
  TORCH_CHECK(b_scale.is_cuda(), "b_scale must be CUDA tensor");
  TORCH_CHECK(a.dim() == 2, "a must be a matrix");
  TORCH_CHECK(b.dim() == 2, "b must be a matrix");
  auto packed = [](const Tensor& t) {
    return t.scalar_type() == at::kByte || t.scalar_type() == at::ScalarType::Float4_e2m1fn_x2;
  };
  TORCH_CHECK(packed(a) && packed(b), "a and b must hold packed e2m1 pairs (uint8 or float4_e2m1fn_x2)");
  TORCH_CHECK(a_scale.element_size() == 1 && b_scale.element_size() == 1, "scales must be E8M0 bytes");
  const int64_t M = a.size(0), Kp = a.size(1), K = 2 * Kp, N = b.size(1);
  TORCH_CHECK(b.size(0) == Kp, "Incompatible matrix dimensions: a is ", M, "x", Kp, " but b is ", b.size(0), "x", N);
  TORCH_CHECK(N % 8 == 0, "N must be a multiple of 16 but got, ", N);
  TORCH_CHECK(K % 32 == 0, "K must be a multiple of the MX block size 32 but got ", K);
  TORCH_CHECK(reinterpret_cast<std::uintptr_t>(a.data_ptr()) % 16 == 0, "Input tensor 'a' must be 16-byte aligned");
  TORCH_CHECK(reinterpret_cast<std::uintptr_t>(b.data_ptr()) % 16 == 0, "Input tensor 'b' must be 16-byte aligned");
  // the length of the blocked layout: 128 ceil(M / 128) rows of 4 ceil(K / 128) bytes, which is the
  // reference's 128 ceil(M / 128) ceil(K / 32) (:197-205) whenever K is a multiple of 128
  const int64_t expected_a = dt_blocked_scale_bytes(M, K / 32);
  TORCH_CHECK(a_scale.numel() == expected_a, "Expected a_scale_size to be ", expected_a, " but got ", a_scale.numel());
  const int64_t expected_b = dt_blocked_scale_bytes(N, K / 32);
  TORCH_CHECK(b_scale.numel() == expected_b, "Expected b_scale_size to be ", expected_b, " but got ", b_scale.numel());
  TORCH_CHECK(a.stride(1) == 1, "Input tensor 'a' must be contiguous in the K dimension (row-major)");
  TORCH_CHECK(b.stride(0) == 1, "Input tensor 'b' must be contiguous in the K dimension (column-major)");
  TORCH_CHECK(a_scale.is_contiguous() && b_scale.is_contiguous(), "scales must be contiguous");
  Ctx ctx(a);
  Tensor out = at::empty({M, N}, a.options().dtype(at::kBFloat16));
  if (M == 0 || N == 0) return out;
  const int64_t lda = M > 1 ? a.stride(0) : Kp, ldb = N > 1 ? b.stride(1) : Kp;
  Tensor& ws = gemm_workspace_for(a, ctx.stream);
  check_status(dt_mx_fp4_bf16_ws(a.data_ptr(), b.data_ptr(), static_cast<const uint8_t*>(a_scale.data_ptr()),
                                 static_cast<const uint8_t*>(b_scale.data_ptr()), M, N, K, lda, ldb, out.data_ptr(), N,
                                 ws.data_ptr(), ws.numel(), ctx.stream),
               "mx_fp4_bf16");
  return out;
}

// ----------------------------------------------------------- schemas kept, not built
Tensor keyed_random_uniform(Tensor, int64_t) { TORCH_CHECK(false, "Not built for this platform!"); }
Tensor sweep_mm(Tensor, Tensor, Tensor, Tensor, std::optional<Tensor>, at::ScalarType, bool, int64_t, int64_t, int64_t,
                bool, int64_t) {
  TORCH_CHECK(false, "sweep_mm was not built (BUILD_SWEEP_MM is OFF)");  // src/sweep_mm.cu:82-84
}

}  // namespace driss_torch

TORCH_LIBRARY(DrissTorch, m) {
  m.impl_abstract_pystub("driss_torch.abstract_impls");  // src/register_ops.cpp:14
  m.def("keyed_random_uniform(Tensor keys, int cols) -> Tensor");
  m.impl("keyed_random_uniform", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::keyed_random_uniform));
  m.def("saturated_cast(Tensor input, Tensor scale, ScalarType dtype, bool transpose) -> Tensor");
  m.impl("saturated_cast", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::saturated_cast));
  m.def("amax(Tensor input) -> Tensor");
  m.impl("amax", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::amax));
  m.def("dynamic_scaled_quant(Tensor input, ScalarType dtype) -> Tensor");
  m.impl("dynamic_scaled_quant", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::dynamic_scaled_quant));
  m.def(
      "sweep_mm(Tensor x, Tensor w, Tensor x_scale, Tensor w_scale, Tensor? bias , ScalarType out_dtype, bool "
      "use_fast_accum, int cluster_shape_x, int cluster_shape_y, int cluster_shape_z, bool transposed, int swizzle) -> "
      "Tensor");
  m.impl("sweep_mm", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::sweep_mm));
  m.def("mx_fp8_bf16(Tensor a, Tensor b, Tensor a_scale, Tensor b_scale) -> Tensor");
  m.impl("mx_fp8_bf16", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp8_bf16));
  m.def("mx_fp4_bf16(Tensor a, Tensor b, Tensor a_scale, Tensor b_scale) -> Tensor");
  m.impl("mx_fp4_bf16", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp4_bf16));
  m.def("mx_fp8_quantize(Tensor input, int block_size, int axis, bool transpose, ScalarType fp8_type) -> (Tensor, Tensor)");
  m.impl("mx_fp8_quantize", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp8_quantize));

  // additions beyond the reference's surface
  m.def("saturated_cast_mode(Tensor input, Tensor scale, ScalarType dtype, bool transpose, int mode) -> Tensor");
  m.impl("saturated_cast_mode", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::saturated_cast_mode));
  m.def("dynamic_scaled_quant_ex(Tensor input, ScalarType dtype, int mode) -> (Tensor, Tensor, Tensor)");
  m.impl("dynamic_scaled_quant_ex", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::dynamic_scaled_quant_ex));
  m.def("dynamic_scaled_quant_pair(Tensor input, int mode) -> (Tensor, Tensor, Tensor, Tensor)");
  m.impl("dynamic_scaled_quant_pair", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::dynamic_scaled_quant_pair));
  m.def("dynamic_scaled_quant_rowwise(Tensor input, ScalarType dtype) -> (Tensor, Tensor, Tensor)");
  m.impl("dynamic_scaled_quant_rowwise", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::dynamic_scaled_quant_rowwise));
  m.def(
      "mx_fp8_quantize_ex(Tensor input, int block_size, int axis, bool transpose, ScalarType fp8_type, bool blocked) -> "
      "(Tensor, Tensor)");
  m.impl("mx_fp8_quantize_ex", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp8_quantize_ex));
  m.def("mx_fp8_quantize_dual(Tensor input, ScalarType fp8_type, bool blocked) -> (Tensor, Tensor, Tensor, Tensor)");
  m.impl("mx_fp8_quantize_dual", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp8_quantize_dual));
  m.def("mx_fp4_quantize(Tensor input, bool blocked, int axis) -> (Tensor, Tensor)");
  m.impl("mx_fp4_quantize", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp4_quantize));
  m.def("mx_fp4_quantize_dual(Tensor input, bool blocked) -> (Tensor, Tensor, Tensor, Tensor)");
  m.impl("mx_fp4_quantize_dual", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::mx_fp4_quantize_dual));
  m.def("to_blocked(Tensor scale) -> Tensor");
  m.impl("to_blocked", c10::DispatchKey::CUDA, TORCH_FN(driss_torch::to_blocked));
}
