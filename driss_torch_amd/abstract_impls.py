"""Fake (meta) implementations so the ops trace under torch.compile / FakeTensor.

The reference registers them for saturated_cast and amax only
(driss_torch/abstract_impls.py:5-19); the remaining ops follow the same pattern.  The functions
are plain here; ``driss_torch/abstract_impls.py`` registers them, because the operator library
names that module as the home of its fake implementations (src/register_ops.cpp:14) and torch
checks the registering module against it.
"""
import torch


def _ceil_div(a, b):
    return (a + b - 1) // b


def _saturated_cast_out(x, out_dtype):
    # The op takes a contiguous or a column-major input with zero storage offset as it lies and
    # keeps its strides; anything else is made contiguous first (src/saturated_cast.cu:243-249).
    transposed = x.dim() == 2 and x.stride(0) == 1 and x.stride(1) == x.shape[0]
    if (x.is_contiguous() or transposed) and x.storage_offset() == 0:
        return torch.empty_like(x, dtype=out_dtype)
    return torch.empty(x.shape, dtype=out_dtype, device=x.device)


def saturated_cast_meta(x: torch.Tensor, scale: torch.Tensor, out_dtype: torch.dtype, transpose: bool = False):
    return _saturated_cast_out(x, out_dtype)


def saturated_cast_mode_meta(x, scale, out_dtype, transpose, mode):
    return _saturated_cast_out(x, out_dtype)


def amax_meta(x: torch.Tensor):
    return torch.empty(1, dtype=torch.float32, device=x.device)


def dynamic_scaled_quant_meta(x: torch.Tensor, dtype: torch.dtype):
    return torch.empty_like(x, dtype=dtype)


def dynamic_scaled_quant_ex_meta(x, dtype, mode):
    return (torch.empty_like(x, dtype=dtype), torch.empty(1, dtype=torch.float32, device=x.device),
            torch.empty((), dtype=torch.float32, device=x.device))


def dynamic_scaled_quant_pair_meta(x, mode):
    return (torch.empty_like(x, dtype=torch.float8_e4m3fn), torch.empty_like(x, dtype=torch.float8_e5m2),
            torch.empty(1, dtype=torch.float32, device=x.device), torch.empty(2, dtype=torch.float32, device=x.device))


def dynamic_scaled_quant_rowwise_meta(x, dtype):
    rows = x.shape[0]
    return (torch.empty_like(x, dtype=dtype), torch.empty((rows, 1), dtype=torch.float32, device=x.device),
            torch.empty((rows, 1), dtype=torch.float32, device=x.device))


def _mx_shapes(x, axis, transpose, blocked):
    m, n = x.shape
    ax = axis % 2
    blocked_dim, other = (n, m) if ax == 1 else (m, n)
    data_shape = (n, m) if transpose else (m, n)
    nblk = blocked_dim // 32
    scale_elems = 128 * _ceil_div(other, 128) * 4 * _ceil_div(nblk, 4) if blocked else other * nblk
    return data_shape, scale_elems


def mx_fp8_quantize_meta(x, block_size, axis, transpose, fp8_type):
    data_shape, scale_elems = _mx_shapes(x, axis, transpose, False)
    return (torch.empty(data_shape, dtype=fp8_type, device=x.device),
            torch.empty((scale_elems,), dtype=torch.float8_e8m0fnu, device=x.device))


def mx_fp8_quantize_ex_meta(x, block_size, axis, transpose, fp8_type, blocked):
    data_shape, scale_elems = _mx_shapes(x, axis, transpose, blocked)
    return (torch.empty(data_shape, dtype=fp8_type, device=x.device),
            torch.empty((scale_elems,), dtype=torch.float8_e8m0fnu, device=x.device))


def mx_fp8_quantize_dual_meta(x, fp8_type, blocked):
    shape_r, scale_r = _mx_shapes(x, 1, False, blocked)
    shape_c, scale_c = _mx_shapes(x, 0, True, blocked)
    e8 = torch.float8_e8m0fnu
    return (torch.empty(shape_r, dtype=fp8_type, device=x.device), torch.empty((scale_r,), dtype=e8, device=x.device),
            torch.empty(shape_c, dtype=fp8_type, device=x.device), torch.empty((scale_c,), dtype=e8, device=x.device))


def mx_fp4_quantize_meta(x, blocked, axis):
    m, n = x.shape
    outer, inner = (m, n) if axis % 2 == 1 else (n, m)
    nscale = 128 * _ceil_div(outer, 128) * 4 * _ceil_div(inner // 32, 4) if blocked else outer * (inner // 32)
    return (torch.empty((outer, inner // 2), dtype=torch.uint8, device=x.device),
            torch.empty((nscale,), dtype=torch.float8_e8m0fnu, device=x.device))


def mx_fp4_quantize_dual_meta(x, blocked):
    return mx_fp4_quantize_meta(x, blocked, 1) + mx_fp4_quantize_meta(x, blocked, 0)


def to_blocked_meta(scale):
    r, c = scale.shape
    return torch.empty((128 * _ceil_div(r, 128) * 4 * _ceil_div(c, 4),), dtype=scale.dtype, device=scale.device)


def mx_fp8_bf16_meta(a, b, a_scale, b_scale):
    return torch.empty((a.shape[0], b.shape[1]), dtype=torch.bfloat16, device=a.device)


def mx_fp4_bf16_meta(a, b, a_scale, b_scale):
    return torch.empty((a.shape[0], b.shape[1]), dtype=torch.bfloat16, device=a.device)


# operator -> fake implementation, registered by driss_torch.abstract_impls
FAKE_IMPLS = {
    "DrissTorch::saturated_cast": saturated_cast_meta,
    "DrissTorch::saturated_cast_mode": saturated_cast_mode_meta,
    "DrissTorch::amax": amax_meta,
    "DrissTorch::dynamic_scaled_quant": dynamic_scaled_quant_meta,
    "DrissTorch::dynamic_scaled_quant_ex": dynamic_scaled_quant_ex_meta,
    "DrissTorch::dynamic_scaled_quant_pair": dynamic_scaled_quant_pair_meta,
    "DrissTorch::dynamic_scaled_quant_rowwise": dynamic_scaled_quant_rowwise_meta,
    "DrissTorch::mx_fp8_quantize": mx_fp8_quantize_meta,
    "DrissTorch::mx_fp8_quantize_ex": mx_fp8_quantize_ex_meta,
    "DrissTorch::mx_fp8_quantize_dual": mx_fp8_quantize_dual_meta,
    "DrissTorch::mx_fp4_quantize": mx_fp4_quantize_meta,
    "DrissTorch::mx_fp4_quantize_dual": mx_fp4_quantize_dual_meta,
    "DrissTorch::to_blocked": to_blocked_meta,
    "DrissTorch::mx_fp8_bf16": mx_fp8_bf16_meta,
    "DrissTorch::mx_fp4_bf16": mx_fp4_bf16_meta,
}
