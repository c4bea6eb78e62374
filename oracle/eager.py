"""Eager-PyTorch restatement of the math the reference's tests compare with.
TEST INFRASTRUCTURE ONLY -- never imported by the product.

The reference has no CPU implementation; its tests check each op against an eager
computation (and against torchao / transformer_nuggets helpers that are not in the
reference tree and not installed here -- those are restated from their published
algorithms and pinned by closed forms in tests/).

Citations are relative to the reference tree.
"""
from __future__ import annotations

import torch

FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)
EPS = 1e-12  # torchao float8_utils.EPS


def eager_amax(a: torch.Tensor) -> torch.Tensor:
    """test/test_amax.py:6-7"""
    return torch.abs(a).max().to(torch.float32).expand(1)


def amax_to_scale(amax: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    """torchao.float8.float8_utils.amax_to_scale as reached through tensor_to_scale
    (test/test_sat_cast.py:35): float64 divide, clamp at EPS, result as float32."""
    amax64 = amax.to(torch.float64)
    res = torch.finfo(fp8_dtype).max / torch.clamp(amax64, min=EPS)
    return res.to(torch.float32)


def tensor_to_scale(a: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    """0-dim fp32 scale of a tensor (torchao tensor_to_scale with per-tensor granularity)."""
    return amax_to_scale(torch.max(torch.abs(a)), fp8_dtype)


def eager_scaled_quant(a: torch.Tensor, scale: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    """test/test_sat_cast.py:7-24 (same body at test/test_dynamic_quant.py:8-25).

    For a bf16 ``a`` the product's precision follows torch's type promotion:
      * ``scale`` 0-dim            -> result stays bf16 (the product is rounded to bf16)
      * ``scale`` of rank >= 1     -> promoted to fp32 (single rounding, at the fp8 convert)
    """
    fmax = torch.finfo(fp8_dtype).max
    out = a * scale
    out = torch.where(out > fmax, fmax, out)
    out = torch.where(out < -1 * fmax, -1 * fmax, out)
    return out.to(fp8_dtype)


def scaled_quant_mode(a: torch.Tensor, scale: torch.Tensor, fp8_dtype: torch.dtype, mode: int) -> torch.Tensor:
    """eager_scaled_quant with the product rounding spelled out explicitly, device independent:
    1: bf16(f32(a)*s)   2: bf16(f32(a)*f32(bf16(s)))   3: f32(a)*s.   fp32 input: all equal."""
    s = scale.reshape(()).to(torch.float32)
    if a.dtype == torch.bfloat16 and mode == 1:
        prod = (a.to(torch.float32) * s).to(torch.bfloat16)
    elif a.dtype == torch.bfloat16 and mode == 2:
        prod = (a.to(torch.float32) * s.to(torch.bfloat16).to(torch.float32)).to(torch.bfloat16)
    else:
        prod = a.to(torch.float32) * s
    fmax = torch.finfo(fp8_dtype).max
    prod = torch.where(prod > fmax, fmax, prod)
    prod = torch.where(prod < -fmax, -fmax, prod)
    return prod.to(fp8_dtype)


def dynamic_scaled_quant(a: torch.Tensor, fp8_dtype: torch.dtype):
    """test/test_dynamic_quant.py:36-44 -> (fp8, amax[1], scale 0-dim)"""
    scale = tensor_to_scale(a, fp8_dtype)
    return eager_scaled_quant(a, scale, fp8_dtype), eager_amax(a), scale


def dynamic_scaled_quant_rowwise(a: torch.Tensor, fp8_dtype: torch.dtype):
    """Row-wise variant (no reference implementation): amax(dim=-1, keepdim=True) and a
    [rows,1] scale, which eager promotes to fp32 before the multiply."""
    amax = torch.amax(torch.abs(a), dim=-1, keepdim=True).to(torch.float32)
    scale = amax_to_scale(amax, fp8_dtype)
    return eager_scaled_quant(a, scale, fp8_dtype), amax, scale


# ------------------------------------------------------------------ MX ----------------

def mx_ceil_exponent(max_abs_f32: torch.Tensor) -> torch.Tensor:
    """ceil(log2(v)) read off the fp32 exponent field, src/mx_cast.cu:50-65."""
    bits = max_abs_f32.contiguous().view(torch.int32) & 0x7FFFFFFF
    be = bits >> 23
    mant = bits & 0x7FFFFF
    normal = be - 127 + (mant != 0).to(torch.int32)
    sub = torch.where(bits == 0, torch.full_like(be, -128), torch.full_like(be, -126))
    return torch.where(be == 0, sub, normal)


def to_mx(a: torch.Tensor, fp8_dtype: torch.dtype = torch.float8_e4m3fn, block: int = 32):
    """MX CEIL-mode cast along the last dim (torchao ``to_mx(..., ScaleCalculationMode.CEIL)``
    as used at test/test_mx.py:90, restated with the integer formula of src/mx_cast.cu:44-86).
    -> (scale uint8 [R, C/block], data fp8 [R, C])."""
    R, Cc = a.shape
    assert Cc % block == 0
    x = a.to(torch.float32).reshape(R, Cc // block, block)
    has_nan = torch.isnan(x).any(dim=-1)
    max_abs = torch.where(torch.isnan(x), torch.zeros_like(x), x.abs()).amax(dim=-1)
    e = mx_ceil_exponent(max_abs)
    target = 8 if fp8_dtype == torch.float8_e4m3fn else 15
    byte = torch.clamp(e - target + 127, 0, 254)
    # payload = x * 2^(127-byte), exact: do it in float64 and round once to fp32
    k = (127 - byte).to(torch.float64).unsqueeze(-1)
    p = (x.to(torch.float64) * torch.exp2(k)).to(torch.float32)
    fmax = torch.finfo(fp8_dtype).max
    p = torch.clamp(p, -fmax, fmax)
    data = p.to(fp8_dtype)
    nan_code = torch.full((), 0x7F, dtype=torch.uint8).view(fp8_dtype)
    data = torch.where(has_nan.unsqueeze(-1), nan_code, data)
    byte = torch.where(has_nan, torch.full_like(byte, 255), byte)
    return byte.to(torch.uint8), data.reshape(R, Cc)


def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def to_blocked(scale: torch.Tensor) -> torch.Tensor:
    """transformer_nuggets.mx.to_blocked (test/test_mx.py:31-32): the cuBLAS block-scaling
    layout: pad to [128*rb, 4*cb], view (rb,128,cb,4) -> permute -> 32x16 interleave."""
    rows, cols = scale.shape
    rb, cb = ceil_div(rows, 128), ceil_div(cols, 4)
    padded = scale
    if (rows, cols) != (rb * 128, cb * 4):
        padded = torch.zeros((rb * 128, cb * 4), dtype=scale.dtype)
        padded[:rows, :cols] = scale
    blocks = padded.view(rb, 128, cb, 4).permute(0, 2, 1, 3)
    rearranged = blocks.reshape(-1, 4, 32, 4).transpose(1, 2).reshape(-1, 32, 16)
    return rearranged.flatten()


def mx_dequant(data: torch.Tensor, scale_u8: torch.Tensor, block: int = 32) -> torch.Tensor:
    """fp32 value of an MX tensor (torchao MXTensor.to_dtype restated): data * 2^(scale-127)."""
    R, Cc = data.shape
    s = torch.exp2(scale_u8.to(torch.float64) - 127.0).reshape(R, Cc // block, 1)
    s = torch.where(scale_u8.reshape(R, Cc // block, 1) == 255, torch.full_like(s, float("nan")), s)
    x = data.to(torch.float64).reshape(R, Cc // block, block) * s
    return x.reshape(R, Cc).to(torch.float32)


def mx_gemm_ref(a_data, a_scale_u8, b_data, b_scale_u8) -> torch.Tensor:
    """test/test_mx.py:34-36 in fp32: dequant(a) @ dequant(b)^T, a [M,K], b [N,K]."""
    return mx_dequant(a_data, a_scale_u8) @ mx_dequant(b_data, b_scale_u8).T


def compute_error(ref: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """torchao compute_error (test/test_mx.py:6,39): SQNR in dB."""
    ref, out = ref.to(torch.float64), out.to(torch.float64)
    return 20 * torch.log10(torch.linalg.norm(ref) / torch.linalg.norm(ref - out))


# ------------------------------------------------------------------------- MXFP4 (e2m1)
# OCP Microscaling Formats v1.0, FP4 E2M1 element table: code -> value
E2M1_VALUES = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def fp4_unpack(packed_u8: torch.Tensor) -> torch.Tensor:
    """[R, C/2] uint8 -> fp32 [R, C]; element 2j is the low nibble of byte j (the packing of the
    MXTensor data the reference's test passes to mx_fp4_bf16, test/test_mx.py:23-26)."""
    lut = torch.tensor(E2M1_VALUES + [-v for v in E2M1_VALUES], dtype=torch.float32)
    lo = lut[(packed_u8 & 15).long()]
    hi = lut[(packed_u8 >> 4).long()]
    return torch.stack([lo, hi], dim=-1).reshape(packed_u8.shape[0], -1)


def mx_fp4_quantize(x: torch.Tensor, block: int = 32):
    """MXFP4 cast in eager form: torchao's ``to_mx(x, "fp4_e2m1", 32)`` in its default (floor) scale mode,
    as called at test/test_mx.py:20-21, restated with torch ops (torchao is not importable here).
    -> (packed e2m1 [R, C/2] uint8, E8M0 [R, C/32] uint8).  Special blocks as in oracle/dt_oracle.c."""
    R, Cc = x.shape
    v = x.to(torch.float32).reshape(R, Cc // block, block)
    has_nan = torch.isnan(v).any(-1)
    amax = torch.where(torch.isnan(v), torch.zeros_like(v), v.abs()).amax(-1)
    field = (amax.view(torch.int32) >> 23) & 0xFF            # floor(log2) + 127 for normal numbers
    byte = torch.clamp(field - 2, 0, 254)
    scaled = v.double() * torch.exp2((127 - byte).double()).unsqueeze(-1)   # exact in float64
    grid = torch.tensor(E2M1_VALUES, dtype=torch.float64)
    mids = (grid[:-1] + grid[1:]) / 2
    a = scaled.abs()
    code = torch.bucketize(a, mids, right=False)             # a == mid goes to the lower code ...
    tie_up = torch.zeros_like(code, dtype=torch.bool)
    for i, m in enumerate(mids.tolist()):                    # ... unless the lower code is odd
        tie_up |= (a == m) & (i % 2 == 1)
    code = torch.where(tie_up, code + 1, code)
    code = torch.where(torch.isnan(a), torch.full_like(code, 7), code)
    code = (code | torch.where(torch.signbit(scaled), 8, 0)).to(torch.uint8)
    code = torch.where(has_nan.unsqueeze(-1), torch.full_like(code, 7), code).reshape(R, Cc)
    packed = code[:, 0::2] | (code[:, 1::2] << 4)
    return packed, torch.where(has_nan, torch.full_like(byte, 255), byte).to(torch.uint8)


def mx_fp4_dequant(packed_u8: torch.Tensor, scale_u8: torch.Tensor, block: int = 32) -> torch.Tensor:
    v = fp4_unpack(packed_u8)
    R, Cc = v.shape
    s = torch.exp2(scale_u8.view(R, Cc // block, 1).double() - 127.0)
    return (v.view(R, Cc // block, block).double() * s).view(R, Cc)
