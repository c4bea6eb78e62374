#!/usr/bin/env python3
"""Saturated-cast benchmark over the reference's shape table.

Mirrors benchmarks/benchmark_saturated_casting.py:52-64 of the reference (same eleven
(rows, cols) shapes incl. the degenerate (1, 3232), (2048, 1) and the wide (2048, 109760), bf16
input, e4m3fn and e5m2 output; correctness check with rtol = atol = 1e-3 as lines 100-110),
timing the HIP kernel against the eager formulation on the same device.  The reference's helpers
from transformer_nuggets and jsonargparse are replaced by a few local lines.

    python -m driss_torch_amd.benchmarks.benchmark_saturated_casting [--csv out.csv] [--compiled]
"""
from __future__ import annotations

import argparse
import csv
import itertools
import sys

import torch

SHAPES = [(512, 512), (1024, 1024), (2048, 2048), (1024, 8192), (8192, 1280), (8192, 7168), (3584, 8192),
          (2048, 109760), (1, 3232), (2048, 1), (14144, 2048)]
LOW_PRECISION = [torch.float8_e4m3fn, torch.float8_e5m2]


def amax_to_scale(amax: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    """fp32 scale = fmax / max(amax, 1e-12), computed in float64 as the reference's tests do."""
    return (torch.finfo(fp8_dtype).max / torch.clamp(amax.double(), min=1e-12)).float()


def eager_scaled_quant(a: torch.Tensor, scale: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    fmax = torch.finfo(fp8_dtype).max
    return (a * scale).clamp(min=-fmax, max=fmax).to(fp8_dtype)


def time_us(fn, *args, min_run_s: float = 0.05) -> float:
    """Median-free simple timer: events around enough back-to-back calls to run for min_run_s."""
    for _ in range(3):
        fn(*args)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 10
    while True:
        start.record()
        for _ in range(n):
            fn(*args)
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end)
        if ms >= min_run_s * 1e3 or n >= 100000:
            return ms * 1e3 / n
        n *= 4


def run(compiled: bool, timed: bool = True, on_checked=None):
    """One row per (shape, fp8 dtype): the correctness check of the reference's harness
    (benchmarks/benchmark_saturated_casting.py:100-108), then, if `timed`, the timings (:110-128).
    `on_checked(x, scale, fp8_dtype, out)` is called after each check (a test hooks in there)."""
    from driss_torch import saturated_cast  # the reference's import (benchmarks/benchmark_saturated_casting.py:8)

    rows = []
    for (r, c), lp in itertools.product(SHAPES, LOW_PRECISION):
        x = torch.randn(r, c, dtype=torch.bfloat16, device="cuda")
        scale = amax_to_scale(x.abs().max().float(), lp)  # 0-dim device scale, as in the reference
        out = saturated_cast(x, scale, lp)
        ref = eager_scaled_quant(x, scale, lp)
        torch.testing.assert_close(out.to(torch.bfloat16), ref.to(torch.bfloat16), rtol=1e-3, atol=1e-3)
        if on_checked is not None:
            on_checked(x, scale, lp, out)
        row = {"num_rows": r, "num_cols": c, "high_precision_dtype": "bfloat16", "low_precision_dtype": str(lp).split(".")[-1]}
        if timed:
            hip_us = time_us(saturated_cast, x, scale, lp)
            eager_us = time_us(eager_scaled_quant, x, scale, lp)
            row.update({"hip_time_us": round(hip_us, 2), "pytorch_time_us": round(eager_us, 2),
                        "hip_GBps": round(r * c * 3 / hip_us / 1e3, 1), "speedup_vs_eager": round(eager_us / hip_us, 2)})
            if compiled:
                fn = torch.compile(eager_scaled_quant, fullgraph=True)
                row["compiled_pytorch_time_us"] = round(time_us(fn, x, scale, lp), 2)
        rows.append(row)
        del x, out, ref
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--csv", help="also write the table to this file")
    ap.add_argument("--compiled", action="store_true", help="also time torch.compile of the eager formulation "
                                                            "(needs a working inductor/triton install)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("this benchmark needs a GPU", file=sys.stderr)
        return 2
    rows = run(args.compiled)
    headers = list(rows[0].keys())
    widths = [max(len(h), *(len(str(r[h])) for r in rows)) for h in headers]
    print("  ".join(h.ljust(w) for h, w in zip(headers, widths)))
    for r in rows:
        print("  ".join(str(r[h]).ljust(w) for h, w in zip(headers, widths)))
    if args.csv:
        with open(args.csv, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=headers)
            w.writeheader()
            w.writerows(rows)
    return 0


if __name__ == "__main__":
    sys.exit(main())
