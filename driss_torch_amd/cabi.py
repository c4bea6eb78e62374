"""ctypes view of the C ABI in ``include/driss_torch_hip.h``.

This is what a host language binding looks like: plain pointers, sizes and a stream handle.
It is used by the parity tests and the benchmark to call the kernels without going through
the torch dispatcher.  torch is only the owner of the device buffers here.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).parent / "lib" / "libdriss_torch_hip.so"
# the same kernels built with -DDT_PHASE_LOG (python driss_torch_amd/_build.py --phase-log): per-workgroup
# clock readings for the benchmark's phase report, switched on with dt_set_phase_log
_PHASES_LIB_PATH = Path(__file__).parent / "lib" / "libdriss_torch_hip_phases.so"

OK = 0
F32, BF16, F16 = 0, 1, 2
E4M3FN, E5M2 = 0, 1
ROUND_BF16_PRODUCT, ROUND_BF16_SCALE_PRODUCT, ROUND_F32 = 1, 2, 3
SCALE_PLAIN, SCALE_BLOCKED = 0, 1

IN_DTYPE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
OUT_DTYPE = {torch.float8_e4m3fn: E4M3FN, torch.float8_e5m2: E5M2}

# every symbol the header declares, with its ctypes signature
_i64, _i32, _vp, _sz, _cp = C.c_int64, C.c_int, C.c_void_p, C.c_size_t, C.c_char_p
SIGNATURES = {
    "dt_status_string": (_cp, [_i32]),
    "dt_abi_version": (_i32, []),
    "dt_workspace_bytes": (_sz, []),
    "dt_workspace_init": (_i32, [_vp, _sz, _vp]),
    "dt_amax": (_i32, [_vp, _i32, _i64, _vp, _vp, _sz, _vp]),
    "dt_saturated_cast": (_i32, [_vp, _i32, _i64, _vp, _i32, _i32, _vp, _vp]),
    "dt_dynamic_scaled_quant": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dt_dynamic_scaled_quant_noalloc": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _vp]),
    "dt_dynamic_scaled_quant_pair": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dt_amax_scales": (_i32, [_vp, _i32, _i64, _vp, _vp, _vp, _sz, _vp]),
    "dt_saturated_cast_pair": (_i32, [_vp, _i32, _i64, _vp, _i32, _vp, _vp, _vp]),
    "dt_dynamic_scaled_quant_rowwise": (_i32, [_vp, _i32, _i64, _i64, _i32, _vp, _vp, _vp, _vp]),
    "dt_mx_fp8_quantize": (_i32, [_vp, _i32, _i64, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "dt_mx_fp8_quantize_dual": (_i32, [_vp, _i32, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "dt_mx_fp4_quantize": (_i32, [_vp, _i32, _i64, _i64, _i32, _i32, _vp, _vp, _vp]),
    "dt_mx_fp4_quantize_dual": (_i32, [_vp, _i32, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp]),
    "dt_blocked_scale_bytes": (_i64, [_i64, _i64]),
    "dt_to_blocked": (_i32, [_vp, _i64, _i64, _vp, _vp]),
    "dt_mx_fp8_bf16": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "dt_mx_fp4_bf16": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "dt_mx_gemm_workspace_bytes": (_sz, []),
    "dt_mx_gemm_workspace_init": (_i32, [_vp, _sz, _vp]),
    "dt_mx_fp8_bf16_ws": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "dt_mx_fp4_bf16_ws": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "dt_dynamic_quant_gave_up": (_i32, []),
    "dt_set_exclusive_gpu": (_i32, [_i32]),
    "dt_get_exclusive_gpu": (_i32, []),
    "dt_dynamic_quant_resident_launches": (C.c_uint64, []),
    "dt_set_tuning": (_i32, [_cp, _i32]),
    "dt_get_tuning": (_i32, [_cp, C.POINTER(_i32)]),
}

_lib = None


def _load(path: Path, extra=None) -> C.CDLL:
    if not path.exists():
        raise ImportError(f"{path} is missing: build it with `python driss_torch_amd/_build.py`")
    L = C.CDLL(str(path))
    for name, (res, args) in {**SIGNATURES, **(extra or {})}.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    return L


def lib() -> C.CDLL:
    """The kernel library.  Raises if it has not been built -- there is no fallback."""
    global _lib
    if _lib is None:
        _lib = _load(_LIB_PATH)
    return _lib


def use_phase_log_build() -> C.CDLL:
    """Switch this module's wrappers to the instrumented build of the kernels (benchmark only)."""
    global _lib
    _lib = _load(_PHASES_LIB_PATH, {"dt_set_phase_log": (_i32, [_vp, _sz])})
    return _lib


def set_exclusive_gpu(on: bool) -> None:
    """Say that this process has the GPU to itself (or no longer): per-tensor dynamic quantization of a
    tensor that fits the chip then runs as one kernel that waits inside for all of its workgroups."""
    _check(lib().dt_set_exclusive_gpu(1 if on else 0), "dt_set_exclusive_gpu")


class DtError(RuntimeError):
    def __init__(self, status: int, what: str):
        self.status = status
        super().__init__(f"{what}: {lib().dt_status_string(status).decode()} (status {status})")


def _check(status: int, what: str) -> None:
    if status != OK:
        raise DtError(status, what)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


_workspaces = {}


def workspace(device=None) -> torch.Tensor:
    """A zero-initialised reduction workspace for the current (device, stream)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if dev.index is None:  # "cuda" means the current device: same workspace as "cuda:<current>"
        dev = torch.device("cuda", torch.cuda.current_device())
    key = (dev.index, _stream())
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.empty(lib().dt_workspace_bytes(), dtype=torch.uint8, device=dev)
        _check(lib().dt_workspace_init(ws.data_ptr(), ws.numel(), _stream()), "dt_workspace_init")
        _workspaces[key] = ws
    return ws


_gemm_workspaces = {}


def gemm_workspace(device=None) -> torch.Tensor:
    """A split-K workspace (zeroed once) for the current (device, stream)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    key = (dev.index, _stream())
    ws = _gemm_workspaces.get(key)
    if ws is None:
        ws = torch.empty(lib().dt_mx_gemm_workspace_bytes(), dtype=torch.uint8, device=dev)
        _check(lib().dt_mx_gemm_workspace_init(ws.data_ptr(), ws.numel(), _stream()), "dt_mx_gemm_workspace_init")
        _gemm_workspaces[key] = ws
    return ws


def set_tuning(key: str, value: int) -> None:
    _check(lib().dt_set_tuning(key.encode(), value), f"dt_set_tuning({key})")


def get_tuning(key: str) -> int:
    v = C.c_int(0)
    _check(lib().dt_get_tuning(key.encode(), C.byref(v)), f"dt_get_tuning({key})")
    return v.value


def amax(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    out = torch.empty(1, dtype=torch.float32, device=x.device) if out is None else out
    ws = workspace(x.device)
    _check(lib().dt_amax(x.data_ptr(), IN_DTYPE[x.dtype], x.numel(), out.data_ptr(), ws.data_ptr(), ws.numel(), _stream()),
           "dt_amax")
    return out


def saturated_cast(x: torch.Tensor, scale: torch.Tensor, out_dtype: torch.dtype, mode: int,
                   out: torch.Tensor | None = None) -> torch.Tensor:
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) if out is None else out
    _check(lib().dt_saturated_cast(x.data_ptr(), IN_DTYPE[x.dtype], x.numel(), scale.data_ptr(), OUT_DTYPE[out_dtype], mode,
                                   out.data_ptr(), _stream()), "dt_saturated_cast")
    return out


def dynamic_scaled_quant(x: torch.Tensor, out_dtype: torch.dtype, mode: int, out=None, amax_out=None, scale_out=None):
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) if out is None else out
    amax_out = torch.empty(1, dtype=torch.float32, device=x.device) if amax_out is None else amax_out
    scale_out = torch.empty(1, dtype=torch.float32, device=x.device) if scale_out is None else scale_out
    ws = workspace(x.device)
    _check(lib().dt_dynamic_scaled_quant(x.data_ptr(), IN_DTYPE[x.dtype], x.numel(), OUT_DTYPE[out_dtype], mode,
                                         out.data_ptr(), amax_out.data_ptr(), scale_out.data_ptr(), ws.data_ptr(),
                                         ws.numel(), _stream()), "dt_dynamic_scaled_quant")
    return out, amax_out, scale_out


def dynamic_scaled_quant_pair(x: torch.Tensor, mode: int, out4=None, out5=None, amax_out=None, scale_out=None):
    out4 = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device) if out4 is None else out4
    out5 = torch.empty(x.shape, dtype=torch.float8_e5m2, device=x.device) if out5 is None else out5
    amax_out = torch.empty(1, dtype=torch.float32, device=x.device) if amax_out is None else amax_out
    scale_out = torch.empty(2, dtype=torch.float32, device=x.device) if scale_out is None else scale_out
    ws = workspace(x.device)
    _check(lib().dt_dynamic_scaled_quant_pair(x.data_ptr(), IN_DTYPE[x.dtype], x.numel(), mode, out4.data_ptr(),
                                              out5.data_ptr(), amax_out.data_ptr(), scale_out.data_ptr(), ws.data_ptr(),
                                              ws.numel(), _stream()), "dt_dynamic_scaled_quant_pair")
    return out4, out5, amax_out, scale_out


def amax_scales(x: torch.Tensor, amax_out=None, scale_out=None):
    amax_out = torch.empty(1, dtype=torch.float32, device=x.device) if amax_out is None else amax_out
    scale_out = torch.empty(2, dtype=torch.float32, device=x.device) if scale_out is None else scale_out
    ws = workspace(x.device)
    _check(lib().dt_amax_scales(x.data_ptr(), IN_DTYPE[x.dtype], x.numel(), amax_out.data_ptr(), scale_out.data_ptr(),
                                ws.data_ptr(), ws.numel(), _stream()), "dt_amax_scales")
    return amax_out, scale_out


def saturated_cast_pair(x: torch.Tensor, scale2: torch.Tensor, mode: int, out4=None, out5=None):
    out4 = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device) if out4 is None else out4
    out5 = torch.empty(x.shape, dtype=torch.float8_e5m2, device=x.device) if out5 is None else out5
    _check(lib().dt_saturated_cast_pair(x.data_ptr(), IN_DTYPE[x.dtype], x.numel(), scale2.data_ptr(), mode,
                                        out4.data_ptr(), out5.data_ptr(), _stream()), "dt_saturated_cast_pair")
    return out4, out5


def dynamic_scaled_quant_rowwise(x: torch.Tensor, out_dtype: torch.dtype, out=None, amax_out=None, scale_out=None):
    R, Cc = x.shape
    out = torch.empty((R, Cc), dtype=out_dtype, device=x.device) if out is None else out
    amax_out = torch.empty((R, 1), dtype=torch.float32, device=x.device) if amax_out is None else amax_out
    scale_out = torch.empty((R, 1), dtype=torch.float32, device=x.device) if scale_out is None else scale_out
    _check(lib().dt_dynamic_scaled_quant_rowwise(x.data_ptr(), IN_DTYPE[x.dtype], R, Cc, OUT_DTYPE[out_dtype],
                                                 out.data_ptr(), amax_out.data_ptr(), scale_out.data_ptr(), _stream()),
           "dt_dynamic_scaled_quant_rowwise")
    return out, amax_out, scale_out


def mx_shapes(rows: int, cols: int, axis: int, transpose: bool, layout: int):
    blocked_dim, other = (cols, rows) if axis == 1 else (rows, cols)
    nblk = blocked_dim // 32
    data_shape = (cols, rows) if transpose else (rows, cols)
    if layout == SCALE_BLOCKED:
        scale_shape = (lib().dt_blocked_scale_bytes(other, nblk),)
    elif (axis == 1) != bool(transpose):
        scale_shape = (other, nblk)
    else:
        scale_shape = (nblk, other)
    return data_shape, scale_shape


def mx_fp8_quantize(x: torch.Tensor, axis: int = 1, transpose: bool = False, out_dtype: torch.dtype = torch.float8_e4m3fn,
                    layout: int = SCALE_PLAIN, data=None, scale=None):
    R, Cc = x.shape
    dshape, sshape = mx_shapes(R, Cc, axis, transpose, layout)
    data = torch.empty(dshape, dtype=out_dtype, device=x.device) if data is None else data
    scale = torch.empty(sshape, dtype=torch.uint8, device=x.device) if scale is None else scale
    _check(lib().dt_mx_fp8_quantize(x.data_ptr(), IN_DTYPE[x.dtype], R, Cc, axis, int(transpose), OUT_DTYPE[out_dtype],
                                    layout, data.data_ptr(), scale.data_ptr(), _stream()), "dt_mx_fp8_quantize")
    return data, scale


def mx_fp8_quantize_dual(x: torch.Tensor, out_dtype: torch.dtype = torch.float8_e4m3fn, layout: int = SCALE_PLAIN, outs=None):
    """(data_rows, scale_rows, data_cols_t, scale_cols_t): the (axis 1) cast of x and the (axis 1) cast of x^T
    from one read of x.  `outs`: the four output tensors, to reuse them."""
    R, Cc = x.shape
    if outs is None:
        dr_shape, sr_shape = mx_shapes(R, Cc, 1, False, layout)
        dc_shape, sc_shape = mx_shapes(R, Cc, 0, True, layout)
        outs = (torch.empty(dr_shape, dtype=out_dtype, device=x.device), torch.empty(sr_shape, dtype=torch.uint8, device=x.device),
                torch.empty(dc_shape, dtype=out_dtype, device=x.device), torch.empty(sc_shape, dtype=torch.uint8, device=x.device))
    dr, sr, dc, sc = outs
    _check(lib().dt_mx_fp8_quantize_dual(x.data_ptr(), IN_DTYPE[x.dtype], R, Cc, OUT_DTYPE[out_dtype], layout, dr.data_ptr(),
                                         sr.data_ptr(), dc.data_ptr(), sc.data_ptr(), _stream()), "dt_mx_fp8_quantize_dual")
    return dr, sr, dc, sc


def mx_fp4_quantize(x: torch.Tensor, layout: int = 0, data=None, scale=None, axis: int = 1):
    """x [R, C] -> (packed e2m1 uint8, E8M0 bytes plain or flat blocked): axis 1 -> [R, C/2] and [R, C/32],
    axis 0 -> the cast of x^T, [C, R/2] and [C, R/32]"""
    R, Cc = x.shape
    outer, inner = (R, Cc) if axis == 1 else (Cc, R)
    data = torch.empty((outer, inner // 2), dtype=torch.uint8, device=x.device) if data is None else data
    if scale is None:
        n = lib().dt_blocked_scale_bytes(outer, inner // 32) if layout == SCALE_BLOCKED else outer * (inner // 32)
        scale = torch.empty((n,), dtype=torch.uint8, device=x.device)
    _check(lib().dt_mx_fp4_quantize(x.data_ptr(), IN_DTYPE[x.dtype], R, Cc, axis, layout, data.data_ptr(), scale.data_ptr(),
                                    _stream()), "dt_mx_fp4_quantize")
    return data, scale


def mx_fp4_quantize_dual(x: torch.Tensor, layout: int = SCALE_PLAIN, outs=None):
    """(data_rows [R, C/2], scale_rows, data_cols_t [C, R/2], scale_cols_t): the axis-1 and the axis-0 MXFP4
    cast of x from one read of x.  `outs`: the four output tensors, to reuse them."""
    R, Cc = x.shape
    if outs is None:
        n_r = lib().dt_blocked_scale_bytes(R, Cc // 32) if layout == SCALE_BLOCKED else R * (Cc // 32)
        n_c = lib().dt_blocked_scale_bytes(Cc, R // 32) if layout == SCALE_BLOCKED else Cc * (R // 32)
        outs = (torch.empty((R, Cc // 2), dtype=torch.uint8, device=x.device), torch.empty((n_r,), dtype=torch.uint8, device=x.device),
                torch.empty((Cc, R // 2), dtype=torch.uint8, device=x.device), torch.empty((n_c,), dtype=torch.uint8, device=x.device))
    dr, sr, dc, sc = outs
    _check(lib().dt_mx_fp4_quantize_dual(x.data_ptr(), IN_DTYPE[x.dtype], R, Cc, layout, dr.data_ptr(), sr.data_ptr(),
                                         dc.data_ptr(), sc.data_ptr(), _stream()), "dt_mx_fp4_quantize_dual")
    return dr, sr, dc, sc


def to_blocked(scale: torch.Tensor) -> torch.Tensor:
    R, Cc = scale.shape
    out = torch.empty(lib().dt_blocked_scale_bytes(R, Cc), dtype=torch.uint8, device=scale.device)
    _check(lib().dt_to_blocked(scale.data_ptr(), R, Cc, out.data_ptr(), _stream()), "dt_to_blocked")
    return out


def mx_fp8_bf16(a: torch.Tensor, bt: torch.Tensor, sfa: torch.Tensor, sfb: torch.Tensor, out=None,
                workspace: bool = True) -> torch.Tensor:
    """a [M,K], bt [N,K] (both K-contiguous), blocked scales -> bf16 [M,N].  ``workspace=False`` calls
    the entry point without a split-K workspace."""
    M, K = a.shape
    N = bt.shape[0]
    out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device) if out is None else out
    if workspace:
        ws = gemm_workspace(a.device)
        _check(lib().dt_mx_fp8_bf16_ws(a.data_ptr(), bt.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), M, N, K, a.stride(0),
                                       bt.stride(0), out.data_ptr(), out.stride(0), ws.data_ptr(), ws.numel(), _stream()),
               "dt_mx_fp8_bf16_ws")
    else:
        _check(lib().dt_mx_fp8_bf16(a.data_ptr(), bt.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), M, N, K, a.stride(0),
                                    bt.stride(0), out.data_ptr(), out.stride(0), _stream()), "dt_mx_fp8_bf16")
    return out


def mx_fp4_bf16(a: torch.Tensor, bt: torch.Tensor, sfa: torch.Tensor, sfb: torch.Tensor, out=None,
                workspace: bool = True) -> torch.Tensor:
    """a [M,K/2], bt [N,K/2] packed e2m1 pairs (both K-contiguous), blocked scales -> bf16 [M,N]."""
    M, Kp = a.shape
    N = bt.shape[0]
    out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device) if out is None else out
    if workspace:
        ws = gemm_workspace(a.device)
        _check(lib().dt_mx_fp4_bf16_ws(a.data_ptr(), bt.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), M, N, 2 * Kp, a.stride(0),
                                       bt.stride(0), out.data_ptr(), out.stride(0), ws.data_ptr(), ws.numel(), _stream()),
               "dt_mx_fp4_bf16_ws")
    else:
        _check(lib().dt_mx_fp4_bf16(a.data_ptr(), bt.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), M, N, 2 * Kp, a.stride(0),
                                    bt.stride(0), out.data_ptr(), out.stride(0), _stream()), "dt_mx_fp4_bf16")
    return out
