"""Fake (meta) implementations so the ops trace under torch.compile / FakeTensor.

The reference registers them for saturated_cast and amax only
(driss_torch/abstract_impls.py:5-19); the remaining ops follow the same pattern.
"""
import torch
from torch.library import register_fake


def _ceil_div(a, b):
    return (a + b - 1) // b


@register_fake("DrissTorch::saturated_cast")
def saturated_cast_meta(x: torch.Tensor, scale: torch.Tensor, out_dtype: torch.dtype, transpose: bool = False):
    return torch.empty_like(x, dtype=out_dtype)


@register_fake("DrissTorch::saturated_cast_mode")
def saturated_cast_mode_meta(x, scale, out_dtype, transpose, mode):
    return torch.empty_like(x, dtype=out_dtype)


@register_fake("DrissTorch::amax")
def amax_meta(x: torch.Tensor):
    return torch.empty(1, dtype=torch.float32, device=x.device)


@register_fake("DrissTorch::dynamic_scaled_quant")
def dynamic_scaled_quant_meta(x: torch.Tensor, dtype: torch.dtype):
    return torch.empty_like(x, dtype=dtype)


@register_fake("DrissTorch::dynamic_scaled_quant_ex")
def dynamic_scaled_quant_ex_meta(x, dtype, mode):
    return (torch.empty_like(x, dtype=dtype), torch.empty(1, dtype=torch.float32, device=x.device),
            torch.empty((), dtype=torch.float32, device=x.device))


@register_fake("DrissTorch::dynamic_scaled_quant_pair")
def dynamic_scaled_quant_pair_meta(x, mode):
    return (torch.empty_like(x, dtype=torch.float8_e4m3fn), torch.empty_like(x, dtype=torch.float8_e5m2),
            torch.empty(1, dtype=torch.float32, device=x.device), torch.empty(2, dtype=torch.float32, device=x.device))


@register_fake("DrissTorch::dynamic_scaled_quant_rowwise")
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


@register_fake("DrissTorch::mx_fp8_quantize")
def mx_fp8_quantize_meta(x, block_size, axis, transpose, fp8_type):
    data_shape, scale_elems = _mx_shapes(x, axis, transpose, False)
    return (torch.empty(data_shape, dtype=fp8_type, device=x.device),
            torch.empty((scale_elems,), dtype=torch.float8_e8m0fnu, device=x.device))


@register_fake("DrissTorch::mx_fp8_quantize_ex")
def mx_fp8_quantize_ex_meta(x, block_size, axis, transpose, fp8_type, blocked):
    data_shape, scale_elems = _mx_shapes(x, axis, transpose, blocked)
    return (torch.empty(data_shape, dtype=fp8_type, device=x.device),
            torch.empty((scale_elems,), dtype=torch.float8_e8m0fnu, device=x.device))


@register_fake("DrissTorch::mx_fp8_quantize_dual")
def mx_fp8_quantize_dual_meta(x, fp8_type, blocked):
    shape_r, scale_r = _mx_shapes(x, 1, False, blocked)
    shape_c, scale_c = _mx_shapes(x, 0, True, blocked)
    e8 = torch.float8_e8m0fnu
    return (torch.empty(shape_r, dtype=fp8_type, device=x.device), torch.empty((scale_r,), dtype=e8, device=x.device),
            torch.empty(shape_c, dtype=fp8_type, device=x.device), torch.empty((scale_c,), dtype=e8, device=x.device))


@register_fake("DrissTorch::mx_fp4_quantize")
def mx_fp4_quantize_meta(x, blocked, axis):
    m, n = x.shape
    outer, inner = (m, n) if axis % 2 == 1 else (n, m)
    nscale = 128 * _ceil_div(outer, 128) * 4 * _ceil_div(inner // 32, 4) if blocked else outer * (inner // 32)
    return (torch.empty((outer, inner // 2), dtype=torch.uint8, device=x.device),
            torch.empty((nscale,), dtype=torch.float8_e8m0fnu, device=x.device))


@register_fake("DrissTorch::to_blocked")
def to_blocked_meta(scale):
    r, c = scale.shape
    return torch.empty((128 * _ceil_div(r, 128) * 4 * _ceil_div(c, 4),), dtype=scale.dtype, device=scale.device)


@register_fake("DrissTorch::mx_fp8_bf16")
def mx_fp8_bf16_meta(a, b, a_scale, b_scale):
    return torch.empty((a.shape[0], b.shape[1]), dtype=torch.bfloat16, device=a.device)


@register_fake("DrissTorch::mx_fp4_bf16")
def mx_fp4_bf16_meta(a, b, a_scale, b_scale):
    return torch.empty((a.shape[0], b.shape[1]), dtype=torch.bfloat16, device=a.device)
