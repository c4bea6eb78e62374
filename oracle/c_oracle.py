"""ctypes binding of ``dt_oracle.c`` -- the bit-level CPU oracle.  TEST INFRASTRUCTURE ONLY.

Arguments and results are CPU torch tensors (fp8 results come back as uint8 codes unless
stated otherwise) so that tests can compare them bit for bit with the HIP path.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libdt_oracle.so"

F32, BF16, F16 = 0, 1, 2
E4M3FN, E5M2 = 0, 1
ROUND_V1, ROUND_V2, ROUND_V3 = 1, 2, 3

_IN_DTYPE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_OUT_DTYPE = {torch.float8_e4m3fn: E4M3FN, torch.float8_e5m2: E5M2}


def build(force: bool = False) -> Path:
    """Compile the C oracle with the Makefile beside it (building the checker is not using it)."""
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < (_HERE / "dt_oracle.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(_HERE), "-B", "libdt_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(str(_LIB_PATH))
        i64, i32, f32, vp, u8 = C.c_int64, C.c_int, C.c_float, C.c_void_p, C.c_uint8
        L.dto_bf16_to_f32.restype, L.dto_bf16_to_f32.argtypes = f32, [C.c_uint16]
        L.dto_f32_to_bf16.restype, L.dto_f32_to_bf16.argtypes = C.c_uint16, [f32]
        L.dto_f32_to_e4m3fn.restype, L.dto_f32_to_e4m3fn.argtypes = u8, [f32]
        L.dto_f32_to_e5m2.restype, L.dto_f32_to_e5m2.argtypes = u8, [f32]
        L.dto_e4m3fn_to_f32.restype, L.dto_e4m3fn_to_f32.argtypes = f32, [u8]
        L.dto_e5m2_to_f32.restype, L.dto_e5m2_to_f32.argtypes = f32, [u8]
        L.dto_e8m0_to_f32.restype, L.dto_e8m0_to_f32.argtypes = f32, [u8]
        L.dto_amax.restype, L.dto_amax.argtypes = f32, [vp, i32, i64]
        L.dto_amax_rows.restype, L.dto_amax_rows.argtypes = None, [vp, i32, i64, i64, vp]
        L.dto_amax_to_scale.restype, L.dto_amax_to_scale.argtypes = f32, [f32, i32]
        L.dto_scaled_quant_one.restype, L.dto_scaled_quant_one.argtypes = u8, [f32, i32, f32, i32, i32]
        L.dto_saturated_cast.restype, L.dto_saturated_cast.argtypes = None, [vp, i32, i64, f32, i32, i32, vp]
        L.dto_dynamic_scaled_quant.restype = None
        L.dto_dynamic_scaled_quant.argtypes = [vp, i32, i64, i32, i32, vp, vp, vp]
        L.dto_dynamic_scaled_quant_rowwise.restype = None
        L.dto_dynamic_scaled_quant_rowwise.argtypes = [vp, i32, i64, i64, i32, vp, vp, vp]
        L.dto_mx_ceil_log2.restype, L.dto_mx_ceil_log2.argtypes = i32, [f32]
        L.dto_mx_scale_byte.restype, L.dto_mx_scale_byte.argtypes = u8, [i32, i32]
        L.dto_mx_quantize.restype, L.dto_mx_quantize.argtypes = i32, [vp, i32, i64, i64, i32, i32, i32, vp, vp]
        L.dto_blocked_offset.restype, L.dto_blocked_offset.argtypes = i64, [i64, i64, i64]
        L.dto_blocked_size.restype, L.dto_blocked_size.argtypes = i64, [i64, i64]
        L.dto_to_blocked.restype, L.dto_to_blocked.argtypes = None, [vp, i64, i64, vp]
        L.dto_mx_gemm_ref.restype = None
        L.dto_mx_gemm_ref.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]
        L.dto_mx_dequant.restype, L.dto_mx_dequant.argtypes = None, [vp, vp, i64, i64, i32, vp]
        L.dto_e2m1_to_f32.restype, L.dto_e2m1_to_f32.argtypes = C.c_float, [C.c_uint8]
        L.dto_f32_to_e2m1.restype, L.dto_f32_to_e2m1.argtypes = C.c_uint8, [C.c_float]
        L.dto_fp4_unpack.restype, L.dto_fp4_unpack.argtypes = None, [vp, i64, i64, vp]
        L.dto_mx_fp4_quantize.restype, L.dto_mx_fp4_quantize.argtypes = None, [vp, i64, i64, vp, vp]
        L.dto_mx_fp4_gemm_ref.restype = None
        L.dto_mx_fp4_gemm_ref.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]
        _lib = L
    return _lib


def _cpu(x: torch.Tensor) -> torch.Tensor:
    assert x.device.type == "cpu", "the oracle works on CPU tensors"
    return x.contiguous()


def _p(t: torch.Tensor):
    return C.c_void_p(t.data_ptr())


def amax(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x)
    v = lib().dto_amax(_p(x), _IN_DTYPE[x.dtype], x.numel())
    return torch.tensor([v], dtype=torch.float32)


def amax_to_scale(amax_value: float, out_dtype: torch.dtype) -> float:
    return lib().dto_amax_to_scale(float(amax_value), _OUT_DTYPE[out_dtype])


def saturated_cast(x: torch.Tensor, scale: float, out_dtype: torch.dtype, mode: int) -> torch.Tensor:
    """uint8 fp8 codes of eager_scaled_quant(x, scale) under product rounding ``mode``."""
    x = _cpu(x)
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().dto_saturated_cast(_p(x), _IN_DTYPE[x.dtype], x.numel(), float(scale), _OUT_DTYPE[out_dtype], mode, _p(out))
    return out


def dynamic_scaled_quant(x: torch.Tensor, out_dtype: torch.dtype, mode: int):
    """-> (uint8 codes, amax fp32[1], scale fp32[1])"""
    x = _cpu(x)
    out = torch.empty(x.shape, dtype=torch.uint8)
    a = torch.empty(1, dtype=torch.float32)
    s = torch.empty(1, dtype=torch.float32)
    lib().dto_dynamic_scaled_quant(_p(x), _IN_DTYPE[x.dtype], x.numel(), _OUT_DTYPE[out_dtype], mode, _p(out), _p(a), _p(s))
    return out, a, s


def dynamic_scaled_quant_rowwise(x: torch.Tensor, out_dtype: torch.dtype):
    """-> (uint8 codes [R,C], amax fp32 [R,1], scale fp32 [R,1])"""
    x = _cpu(x)
    R, Cc = x.shape
    out = torch.empty((R, Cc), dtype=torch.uint8)
    a = torch.empty((R, 1), dtype=torch.float32)
    s = torch.empty((R, 1), dtype=torch.float32)
    lib().dto_dynamic_scaled_quant_rowwise(_p(x), _IN_DTYPE[x.dtype], R, Cc, _OUT_DTYPE[out_dtype], _p(out), _p(a), _p(s))
    return out, a, s


def mx_quantize(x: torch.Tensor, axis: int = 1, transpose: bool = False,
                out_dtype: torch.dtype = torch.float8_e4m3fn):
    """-> (uint8 payload codes, uint8 E8M0 bytes); shapes as documented in dt_oracle.c"""
    x = _cpu(x)
    R, Cc = x.shape
    axis = axis % 2
    if axis == 1:
        dshape, sshape = ((Cc, R), (Cc // 32, R)) if transpose else ((R, Cc), (R, Cc // 32))
    else:
        dshape, sshape = ((Cc, R), (Cc, R // 32)) if transpose else ((R, Cc), (R // 32, Cc))
    data = torch.empty(dshape, dtype=torch.uint8)
    scale = torch.empty(sshape, dtype=torch.uint8)
    rc = lib().dto_mx_quantize(_p(x), _IN_DTYPE[x.dtype], R, Cc, axis, int(transpose), _OUT_DTYPE[out_dtype], _p(data), _p(scale))
    if rc != 0:
        raise ValueError("blocked dimension must be a multiple of 32")
    return data, scale


def to_blocked(scale: torch.Tensor) -> torch.Tensor:
    """[R, C] uint8 E8M0 bytes -> flat blocked 128x4 layout (zero padded)."""
    scale = _cpu(scale)
    R, Cc = scale.shape
    out = torch.empty(lib().dto_blocked_size(R, Cc), dtype=torch.uint8)
    lib().dto_to_blocked(_p(scale), R, Cc, _p(out))
    return out


def mx_gemm_ref(a: torch.Tensor, bt: torch.Tensor, sfa_blocked: torch.Tensor, sfb_blocked: torch.Tensor) -> torch.Tensor:
    """a [M,K], bt [N,K] uint8 e4m3 codes, blocked scales -> fp32 [M,N] (float64 accumulation)."""
    a, bt = _cpu(a), _cpu(bt)
    M, K = a.shape
    N = bt.shape[0]
    out = torch.empty((M, N), dtype=torch.float32)
    lib().dto_mx_gemm_ref(_p(a), _p(bt), _p(_cpu(sfa_blocked)), _p(_cpu(sfb_blocked)), M, N, K, K, K, _p(out))
    return out


def mx_dequant(data: torch.Tensor, scale: torch.Tensor, out_dtype: torch.dtype = torch.float8_e4m3fn) -> torch.Tensor:
    data, scale = _cpu(data), _cpu(scale)
    R, Cc = data.shape
    out = torch.empty((R, Cc), dtype=torch.float32)
    lib().dto_mx_dequant(_p(data), _p(scale), R, Cc, _OUT_DTYPE[out_dtype], _p(out))
    return out


def e2m1_to_f32(code: int) -> float:
    return lib().dto_e2m1_to_f32(code)


def f32_to_e2m1(x: float) -> int:
    return lib().dto_f32_to_e2m1(x)


def fp4_unpack(packed: torch.Tensor) -> torch.Tensor:
    """[R, C/2] uint8 (even element in the low nibble) -> fp32 [R, C]"""
    packed = _cpu(packed)
    R, Ch = packed.shape
    out = torch.empty((R, 2 * Ch), dtype=torch.float32)
    lib().dto_fp4_unpack(_p(packed), R, 2 * Ch, _p(out))
    return out


def mx_fp4_quantize(x: torch.Tensor):
    """MXFP4 cast of [R, C] (any float dtype; widened to fp32, which is exact) -> (packed e2m1 [R, C/2]
    uint8, E8M0 [R, C/32] uint8)."""
    x = _cpu(x.float())
    R, Cc = x.shape
    data = torch.empty((R, Cc // 2), dtype=torch.uint8)
    scale = torch.empty((R, Cc // 32), dtype=torch.uint8)
    lib().dto_mx_fp4_quantize(_p(x), R, Cc, _p(data), _p(scale))
    return data, scale


def mx_fp4_gemm_ref(a: torch.Tensor, bt: torch.Tensor, sfa_blocked: torch.Tensor, sfb_blocked: torch.Tensor) -> torch.Tensor:
    """a [M,K/2], bt [N,K/2] packed e2m1, blocked scales -> fp32 [M,N] (float64 accumulation)."""
    a, bt = _cpu(a), _cpu(bt)
    M, Kp = a.shape
    N = bt.shape[0]
    out = torch.empty((M, N), dtype=torch.float32)
    lib().dto_mx_fp4_gemm_ref(_p(a), _p(bt), _p(_cpu(sfa_blocked)), _p(_cpu(sfb_blocked)), M, N, 2 * Kp, Kp, Kp, _p(out))
    return out
