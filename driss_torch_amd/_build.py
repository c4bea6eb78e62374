"""Builds the two in-tree shared libraries of the package for gfx950.

* ``lib/libdriss_torch_hip.so`` -- the HIP kernels behind the C ABI of
  ``include/driss_torch_hip.h`` (no torch dependency), compiled with hipcc.
* ``lib/libdriss_torch.so``     -- the ``torch.ops.DrissTorch`` registration shim, host C++
  only, linked against torch and the kernel library.

Run ``python driss_torch_amd/_build.py`` (or ``__graft_entry__.build()``).  The GPU is not
needed: hipcc cross-compiles.  ``python driss_torch_amd/_build.py --phase-log`` makes a third library,
``lib/libdriss_torch_hip_phases.so``: the kernels with their per-workgroup clock readings compiled in,
which only ``bench.py --phases`` loads.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB = PKG / "lib"
OBJ = LIB / "obj"
INCLUDE = ROOT / "include"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

HIP_LIB = LIB / "libdriss_torch_hip.so"
TORCH_LIB = LIB / "libdriss_torch.so"
PHASES_HIP_LIB = LIB / "libdriss_torch_hip_phases.so"  # made on request only (--phase-log)

HIP_SOURCES = ["mx_fp8_bf16.hip", "mx_fp4_bf16.hip", "mx_few_rows.hip", "abi_common.hip", "amax.hip", "saturated_cast.hip",
               "dynamic_scaled_quant.hip", "mx_cast.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-fno-fast-math",
    "-ffp-contract=off",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    # hipcc's host pass warns that it does not know the -packed-fp32-ops feature: harmless
    noise = [l for l in proc.stderr.splitlines() if l and "packed-fp32-ops" not in l]
    if noise and os.environ.get("DT_BUILD_VERBOSE"):
        sys.stderr.write("\n".join(noise) + "\n")


def build_hip_library(jobs: int = 6, phase_log: bool = False) -> Path:
    """The kernel library; with ``phase_log`` the instrumented build of the same sources
    (-DDT_PHASE_LOG: per-workgroup clock readings and dt_set_phase_log, for ``bench.py --phases``)."""
    obj_dir = OBJ / "phases" if phase_log else OBJ
    target = PHASES_HIP_LIB if phase_log else HIP_LIB
    obj_dir.mkdir(parents=True, exist_ok=True)
    hipcc = str(ROCM / "bin" / "hipcc")
    flags = HIPCC_FLAGS + (["-DDT_PHASE_LOG"] if phase_log else [])
    objs = []

    def compile_one(src: str) -> str:
        obj = obj_dir / (Path(src).stem + ".o")
        _run([hipcc, *flags, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / src), "-o", str(obj)])
        return str(obj)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wno-unused-command-line-argument", *objs, "-o",
          str(target)])
    return target


def build_torch_shim() -> Path:
    import torch
    from torch.utils import cpp_extension as ce

    torch_lib = Path(torch.__file__).parent / "lib"
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{INCLUDE}", f"-I{ROCM / 'include'}"]
    cmd += [f"-isystem{p}" for p in ce.include_paths()]
    cmd += [str(CSRC / "register_ops.cpp"), "-o", str(TORCH_LIB),
            f"-L{LIB}", "-ldriss_torch_hip", f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch", "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"]
    _run(cmd)
    return TORCH_LIB


def build_all() -> None:
    build_hip_library()
    build_torch_shim()


if __name__ == "__main__":
    if "--phase-log" in sys.argv[1:]:
        print("built", build_hip_library(phase_log=True))
    else:
        build_all()
        print("built", HIP_LIB, TORCH_LIB)
