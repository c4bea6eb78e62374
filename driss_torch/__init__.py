"""The reference's import name for the MI355X build.

``from driss_torch import saturated_cast, amax, dynamic_scaled_quant, mx_fp8_quantize,
mx_fp8_bf16, mx_fp4_bf16`` (the imports of the reference's tests and benchmark,
test/test_*.py, benchmarks/benchmark_saturated_casting.py:8) resolve to the wrappers of
``driss_torch_amd``, which mirror driss_torch/__init__.py:20-122.
"""
import driss_torch_amd as _impl
from driss_torch_amd import *  # noqa: F401,F403
from driss_torch_amd import (amax, dynamic_scaled_quant, lib_path, mx_cast, mx_fp4_bf16, mx_fp8_bf16,  # noqa: F401
                             mx_fp8_quantize, ops, saturated_cast, sweep_mm)

__all__ = [n for n in dir(_impl) if not n.startswith("_")]
