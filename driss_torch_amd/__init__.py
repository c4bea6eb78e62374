"""driss_torch on MI355X: FP8 / MX quantization ops behind ``torch.ops.DrissTorch``.

The wrapper names, signatures and defaults follow the reference's
``driss_torch/__init__.py:20-122``; the work is done by hand-written gfx950 kernels in
``lib/libdriss_torch_hip.so`` (C ABI: ``include/driss_torch_hip.h``) reached through the
registration shim ``lib/libdriss_torch.so``.  There is no fallback path: importing this
package fails if the libraries have not been built (``python driss_torch_amd/_build.py``).
"""
from pathlib import Path
from typing import Optional, Tuple

import torch

_LIB_DIR = Path(__file__).parent / "lib"
hip_lib_path = _LIB_DIR / "libdriss_torch_hip.so"
lib_path = _LIB_DIR / "libdriss_torch.so"
for _p in (hip_lib_path, lib_path):
    if not _p.exists():
        raise ImportError(f"{_p} is missing: build it with `python driss_torch_amd/_build.py`")
torch.ops.load_library(str(lib_path.resolve()))

ops = torch.ops.DrissTorch
Tensor = torch.Tensor

# product rounding of x*scale for bf16 inputs (see include/driss_torch_hip.h: dt_round_mode)
ROUND_AUTO, ROUND_BF16_PRODUCT, ROUND_BF16_SCALE_PRODUCT, ROUND_F32 = 0, 1, 2, 3


def list_ops():
    """Kept from the reference, which raises here too (driss_torch/__init__.py:15-17)."""
    raise NotImplementedError("This function does not do what I think it should.")


def set_exclusive_gpu(exclusive: bool = True) -> None:
    """Tell the library that this process has the GPU to itself.  ``dynamic_scaled_quant`` of a tensor that
    fits the chip (up to 128 MiB) then runs as ONE kernel that keeps the tensor in registers and LDS
    between the reduction and the cast and waits inside for all of its workgroups (1.4 x faster at
    8192 x 8192 bf16).  Off by default -- another process on the GPU could make that wait give up and the
    call return NaN -- and also switched on by ``DRISS_TORCH_RESIDENT=1`` in the environment at import.
    The reference gets the same guarantee from a cooperative launch (src/dynamic_scaled_quant.cu:144-150)."""
    from . import cabi

    cabi.set_exclusive_gpu(exclusive)


def saturated_cast(x: Tensor, scale: Tensor, out_dtype: torch.dtype, transpose: bool = False) -> Tensor:
    """fp8 saturated cast of ``x * scale`` (reference: driss_torch/__init__.py:20-38).

    ``scale`` is a one-element fp32 tensor on the device.  For bf16 ``x`` the product is
    rounded the way eager PyTorch rounds it for that scale tensor: a 0-dim scale keeps the
    product (and the scale) in bf16, a scale of rank >= 1 promotes the product to fp32.
    """
    assert not transpose, "Transpose is not supported yet"
    return ops.saturated_cast(x, scale, out_dtype, transpose)


def saturated_cast_mode(x: Tensor, scale: Tensor, out_dtype: torch.dtype, mode: int) -> Tensor:
    """``saturated_cast`` with the product rounding mode given explicitly (ROUND_*)."""
    return ops.saturated_cast_mode(x, scale, out_dtype, False, mode)


def amax(x: Tensor) -> Tensor:
    """max(abs(x)) as an fp32 tensor of shape [1] (reference: driss_torch/__init__.py:41-43)."""
    return ops.amax(x)


def dynamic_scaled_quant(inpt: Tensor, dtype: torch.dtype) -> Tensor:
    """amax -> scale -> saturated cast in one call (reference: driss_torch/__init__.py:46-47)."""
    return ops.dynamic_scaled_quant(inpt, dtype)


def dynamic_scaled_quant_ex(inpt: Tensor, dtype: torch.dtype, mode: int = ROUND_AUTO) -> Tuple[Tensor, Tensor, Tensor]:
    """As ``dynamic_scaled_quant`` but also returns (amax [1], scale 0-dim)."""
    return ops.dynamic_scaled_quant_ex(inpt, dtype, mode)


def dynamic_scaled_quant_pair(inpt: Tensor, mode: int = ROUND_AUTO) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """e4m3fn and e5m2 casts from one amax and one read: (e4m3fn, e5m2, amax [1], scale [2])."""
    return ops.dynamic_scaled_quant_pair(inpt, mode)


def dynamic_scaled_quant_rowwise(inpt: Tensor, dtype: torch.dtype) -> Tuple[Tensor, Tensor, Tensor]:
    """Per-row scales: (fp8 [R,C], amax [R,1], scale [R,1]); the product is taken in fp32."""
    return ops.dynamic_scaled_quant_rowwise(inpt, dtype)


def sweep_mm(x: Tensor, w: Tensor, x_scale: Tensor, w_scale: Tensor, bias: Optional[Tensor], out_dtype: torch.dtype,
             use_fast_accum: bool, cluster_shape_x: int, cluster_shape_y: int, cluster_shape_z: int, transposed: bool,
             swizzle: int) -> Tensor:
    """Schema kept from the reference (driss_torch/__init__.py:50-77); not built, raises."""
    return ops.sweep_mm(x, w, x_scale, w_scale, bias, out_dtype, use_fast_accum, cluster_shape_x, cluster_shape_y,
                        cluster_shape_z, transposed, swizzle)


def mx_fp8_bf16(a: Tensor, b: Tensor, a_scale: Tensor, b_scale: Tensor) -> Tensor:
    """bf16 = (a * 2^a_scale) @ (b * 2^b_scale) for e4m3fn operands with E8M0 block-32 scales
    in the blocked 128x4 layout (reference: driss_torch/__init__.py:80-94).

    a: [M, K] row-major; b: [K, N] with stride(0) == 1 (an [N, K] tensor transposed).
    """
    return ops.mx_fp8_bf16(a, b, a_scale, b_scale)


def mx_fp4_bf16(a: Tensor, b: Tensor, a_scale: Tensor, b_scale: Tensor) -> Tensor:
    """bf16 = (a * 2^a_scale) @ (b * 2^b_scale) for e2m1 operands with E8M0 block-32 scales in
    the blocked 128x4 layout (reference: driss_torch/__init__.py:97-111).

    a: [M, K/2] row-major, b: [K/2, N] with stride(0) == 1; two e2m1 values per byte (uint8 or
    float4_e2m1fn_x2 storage), the even element in the low nibble.
    """
    return ops.mx_fp4_bf16(a, b, a_scale, b_scale)


def mx_fp8_quantize(input: Tensor, block_size: int = 32, axis: int = 1, transpose: bool = False,
                    ScalarType: torch.dtype = torch.float8_e4m3fn) -> Tuple[Tensor, Tensor]:
    """MXFP8 cast (reference: driss_torch/__init__.py:114-122): (payload, E8M0 scales, 1-D).

    axis 1 blocks along rows, axis 0 down columns.  Payload is [M, N], or [N, M] with
    ``transpose``; the flat scale tensor is the row-major scale matrix [M, N/32] (axis 1),
    [M/32, N] (axis 0), [N/32, M] (axis 1, transpose) or [N, M/32] (axis 0, transpose).
    """
    return ops.mx_fp8_quantize(input, block_size, axis, transpose, ScalarType)


mx_cast = mx_fp8_quantize


def mx_fp8_quantize_blocked(input: Tensor, axis: int = 1, ScalarType: torch.dtype = torch.float8_e4m3fn
                            ) -> Tuple[Tensor, Tensor]:
    """MXFP8 cast whose scales come out in the blocked layout ``mx_fp8_bf16`` reads, with K as
    the contiguous payload dimension: axis 1 -> payload [M, N]; axis 0 -> payload [N, M]."""
    return ops.mx_fp8_quantize_ex(input, 32, axis, axis % 2 == 0, ScalarType, True)


def mx_fp8_quantize_dual(input: Tensor, ScalarType: torch.dtype = torch.float8_e4m3fn, blocked: bool = False
                         ) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Both MXFP8 blockings of ``input`` [M, N] from one read: ``(data [M, N], scale, data_t [N, M],
    scale_t)``.  The first pair equals ``mx_fp8_quantize(input)``, the second
    ``mx_fp8_quantize(input.t().contiguous())``: the operand for a forward product and the one for the
    weight-gradient product.  ``blocked`` selects the scale layout ``mx_fp8_bf16`` reads."""
    return ops.mx_fp8_quantize_dual(input, ScalarType, blocked)


def mx_fp4_quantize(input: Tensor, blocked: bool = False, axis: int = 1) -> Tuple[Tensor, Tensor]:
    """MXFP4 cast of ``input`` [M, N]: ``(packed e2m1 pairs as uint8, E8M0 scales)``, the operands
    ``mx_fp4_bf16`` takes (the reference's test builds them with torchao's
    ``MXTensor.to_mx(x, "fp4_e2m1", 32)``, test/test_mx.py:17-21).  axis 1: blocks of 32 along the rows,
    payload [M, N/2], scale matrix [M, N/32]; axis 0: blocks down the columns with the payload
    transposed, [N, M/2] and [N, M/32], which equals the axis-1 cast of ``input.t().contiguous()``.
    ``blocked`` selects the scale layout the GEMM reads; otherwise the flat scale tensor is row-major."""
    return ops.mx_fp4_quantize(input, blocked, axis)


def mx_fp4_quantize_dual(input: Tensor, blocked: bool = False) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Both MXFP4 operands of ``input`` [M, N] from one read: ``(data [M, N/2], scale, data_t [N, M/2],
    scale_t)``, equal to ``mx_fp4_quantize(input, blocked, 1) + mx_fp4_quantize(input, blocked, 0)``."""
    return ops.mx_fp4_quantize_dual(input, blocked)


def to_blocked(scale: Tensor) -> Tensor:
    """[R, C] E8M0 scale matrix -> flat blocked 128x4 layout (zero padded)."""
    return ops.to_blocked(scale)


# The fake implementations register from the module the operator library names as their home
# (the reference's: src/register_ops.cpp:14).  Imported last: that package re-exports the wrappers above.
torch.ops.import_module("driss_torch.abstract_impls")
