#!/usr/bin/env python3
"""Benchmark of the FP8 / MX quantization path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

A step is one pass of the per-tensor dynamic quantization over one 8192 x 8192 bf16 tensor
(amax -> scales -> e4m3fn and e5m2 casts, reached through the C ABI entry point
dt_dynamic_scaled_quant_pair: one kernel that keeps the tensor on the chip between the
reduction and the cast; the two-kernel path of larger tensors is timed beside it).  Inputs are resident in HBM before the timed
region; steps rotate over enough buffer sets that no step finds its input in the 256 MB
memory-side cache.  One JSON line is printed: the step throughput in algorithmic GB/s,
the roofline figures of the dominant kernel (timed with events on the launch stream), a table of every other kernel of the path (`kernels`), and the
eager CPU formulation timed on this host's cores (`cpu_baseline`).
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
FP8_PEAK_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
FP4_PEAK_TFLOPS = 10100.0   # MI355X dense fp4 MFMA
MALL_BYTES = 256 << 20
# HBM-side bytes per launch of the step's kernels, from rocprofv3 FETCH_SIZE / WRITE_SIZE, each scaled
# by what the same counter reads for a plain 128 MiB device copy: the summary of those two counter
# runs is a text file, read at run time (its commands are in its header)
TRAFFIC_PROFILE = ROOT / "profiles" / "dynamic_quant_pair_config2_hbm_traffic.txt"


def traffic_from_profile(kernel_prefix):
    """HBM bytes per launch of the kernel whose name starts with `kernel_prefix`, or None."""
    try:
        for line in TRAFFIC_PROFILE.read_text().splitlines():
            if line.startswith(kernel_prefix):
                return float(line.split()[-1]) * 1e6  # last column: traffic in MB
    except (OSError, ValueError):
        pass
    return None


def normal_with_outliers(torch, shape, seed, frac=1e-3, factor=100.0):
    """config 2's input: N(0,1) drawn in fp32 on the CPU, 0.1 % of the positions multiplied by 100, as bf16"""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    idx = torch.randperm(x.numel(), generator=g)[:max(1, round(frac * x.numel()))]
    x.view(-1)[idx] *= factor
    return x.to(torch.bfloat16)


def _events(n):
    import torch

    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def time_launches(fn, nsets, steps, warmup):
    """Average device time of fn(set_index) in microseconds: events around `steps` launches."""
    import torch

    for i in range(warmup):
        fn(i % nsets)
    torch.cuda.synchronize()
    start, end = _events(2)
    start.record()
    for i in range(steps):
        fn(i % nsets)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) * 1e3 / steps


_NOT_LAUNCHES = {"dt_workspace_bytes", "dt_blocked_scale_bytes", "dt_mx_gemm_workspace_bytes", "dt_status_string",
                 "dt_get_tuning", "dt_set_tuning", "dt_workspace_init", "dt_mx_gemm_workspace_init", "dt_abi_version",
                 "dt_set_phase_log", "dt_dynamic_quant_gave_up"}


class _Recorder:
    """Stands in for the C-ABI library handle while one call of a wrapper is noted down."""

    def __init__(self, lib):
        self._lib, self.calls = lib, []

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if name in _NOT_LAUNCHES or not name.startswith("dt_"):
            return fn

        def noted(*args):
            self.calls.append((fn, args))
            return fn(*args)

        return noted


def bind(cabi, run, *args):
    """run(*args) once, noting the C-ABI entry points it reaches with their plain arguments (pointers,
    sizes, stream); returns a callable that repeats exactly those calls.  The Python wrappers in cabi.py
    cost 10-20 us per call (tensor attribute look-ups), more than some kernels take: the timed loops call
    the C ABI the way a compiled host would."""
    rec, saved = _Recorder(cabi.lib()), cabi._lib
    cabi._lib = rec
    try:
        kept = run(*args)  # what the wrapper allocated itself stays alive as long as the replays may write to it
    finally:
        cabi._lib = saved
    calls = rec.calls
    assert calls, "the wrapper made no C-ABI call"
    if len(calls) == 1:
        fn, a = calls[0]

        def replay_one(_kept=kept):
            if fn(*a):
                raise RuntimeError("C-ABI call failed in the timed loop")

        return replay_one

    def replay(_kept=kept):
        for f, a_ in calls:
            if f(*a_):
                raise RuntimeError("C-ABI call failed in the timed loop")

    return replay


def nsets_for(bytes_per_set):
    """buffer sets needed so a set is evicted from the memory-side cache before it is reused"""
    return max(2, -(-2 * MALL_BYTES // bytes_per_set) + 1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (the timed region of `value` is bracketed by host synchronisations that cost it about 0.2 ms whatever
    # its length: 1000 steps of 44 us keep that to half a percent)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-extra", action="store_true", help="skip the per-kernel table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--gemm-only", action="store_true",
                    help="run only the block-scaled GEMM rows of the per-kernel table (for profiling) and print them")
    ap.add_argument("--gemm-ramp", action="store_true",
                    help="print how the 8192^3 block-scaled GEMM's launch time settles after a pause (windows of 25 launches)")
    ap.add_argument("--phases", action="store_true",
                    help="also report the per-phase times of the step's kernel (shader clock counter readings it dumps)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain device copies of 128 MiB (to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every op of this path is a single-device kernel "
              "(sharding is by rows with at most a 4-byte max-reduce); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from driss_torch_amd import cabi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.phases:
        # the per-phase report needs the kernels' clock readings, which only the instrumented build of the
        # library has (python driss_torch_amd/_build.py --phase-log); everything below then runs on that build
        cabi.use_phase_log_build()
    # The benchmark has the GPU to itself and says so: per-tensor dynamic quantization of a tensor that fits
    # the chip then runs as one kernel (the library's default, for callers that have not said so, is the
    # reduction kernel followed by the cast kernel: `two_kernel_path` below)
    cabi.set_exclusive_gpu(True)
    K, W = args.steps, args.warmup
    # the per-kernel rows, the event-bracketed trains and the comparison legs: at most 200 launches each
    KX, WX = min(K, 200), min(W, 20)
    if args.gemm_ramp:
        print(json.dumps(gemm_ramp(torch, cabi, dev)))
        return
    if args.gemm_only:
        ph = {} if args.phases else None
        rows = extra_kernels(torch, cabi, dev, KX, WX, gemm_only=True, phases=ph)
        print(json.dumps({"kernels": rows, "phases": ph} if ph else {"kernels": rows}))
        return

    # ------------------------------------------------------------ headline step: config 2
    R = C = 8192
    numel = R * C
    # Bytes of the step.  A two-kernel formulation of the path reads x twice (once for the
    # reduction, once for the cast: 6 B per element with two fp8 outputs); the step's one kernel keeps
    # x on the chip between its passes, so what it must move -- and what the counters see -- is one
    # read of x and the two fp8 outputs: 4 B per element.  `value` and the roofline are quoted on
    # those 4 B; the 6 B figure is reported beside them as the two-pass equivalent.
    two_pass_bytes = numel * (2 + 2 + 1 + 1)
    step_bytes = numel * (2 + 1 + 1)
    cast_bytes = numel * (2 + 1 + 1)              # the cast of the two-kernel path: one read, two writes
    ns = nsets_for(numel * 4)
    x_cpu = normal_with_outliers(torch, (R, C), 1002)
    xs = [x_cpu.to(dev) if i == 0 else torch.roll(x_cpu, i, 0).to(dev) for i in range(ns)]
    o4 = [torch.empty((R, C), dtype=torch.float8_e4m3fn, device=dev) for _ in range(ns)]
    o5 = [torch.empty((R, C), dtype=torch.float8_e5m2, device=dev) for _ in range(ns)]
    amax_out = torch.empty(1, dtype=torch.float32, device=dev)
    scale_out = torch.empty(2, dtype=torch.float32, device=dev)
    mode = cabi.ROUND_BF16_SCALE_PRODUCT

    steps_bound = [bind(cabi, lambda s=s: cabi.dynamic_scaled_quant_pair(xs[s], mode, o4[s], o5[s], amax_out, scale_out))
                   for s in range(ns)]
    amax_bound = [bind(cabi, lambda s=s: cabi.amax_scales(xs[s], amax_out, scale_out)) for s in range(ns)]
    cast_bound = [bind(cabi, lambda s=s: cabi.saturated_cast_pair(xs[s], scale_out, mode, o4[s], o5[s])) for s in range(ns)]

    def step(i):
        steps_bound[i % ns]()

    def step_staged(i, ev):
        # the same two kernels through the staged entry points, with events around the second
        amax_bound[i % ns]()
        ev[0].record()
        cast_bound[i % ns]()
        ev[1].record()

    # timed region 1: K whole steps, nothing between the launches -> `value`
    for i in range(W):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        step(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / K
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # timed region 2: the step is one kernel (the tensor fits the chip, see resident_kernels.hpp):
    # K launches between one pair of HIP events on the launch stream -> `roofline`
    # (the median of five such trains: a train of K launches lasts about 2 ms, and one hiccup of the launching
    # thread in it shifts its average by several percent)
    step_us = statistics.median(time_launches(step, ns, KX, WX) for _ in range(5))
    step_gbs = step_bytes / (step_us * 1e-6) / 1e9

    phases = None
    if args.phases:
        phases = {"resident_quant_kernel (the step)": kernel_phases(
            torch, cabi, step, ["load and reduce", "grid barrier", "convert and store"])}
        amax_tmp = torch.empty(1, dtype=torch.float32, device=dev)
        phases["amax_kernel, bf16 [8192,8192]"] = kernel_phases(
            torch, cabi, lambda i: cabi.amax(xs[i % ns], amax_tmp), ["load", "workgroup reduce", "atomics"])
        del amax_tmp

    # for comparison: the two-kernel path every larger tensor takes (amax, then cast), the cast
    # bracketed by an event pair per launch (adds about 4 us of dispatch latency to it)
    cabi.set_exclusive_gpu(False)
    two_kernel_us = time_launches(step, ns, KX, WX)
    evs = [_events(2) for _ in range(KX)]
    torch.cuda.synchronize()
    for i in range(KX):
        step_staged(i, evs[i])
    torch.cuda.synchronize()
    cast_us = statistics.fmean(e[0].elapsed_time(e[1]) for e in evs) * 1e3
    cabi.set_exclusive_gpu(True)

    traffic = traffic_from_profile("dt::resident_quant_kernel")
    cast_traffic = traffic_from_profile("dt::cast_kernel")
    result = {
        "metric": "cast/amax HBM GB/s (% of 8 TB/s) at 8192² bf16; MXFP8 GEMM TFLOPS",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16->fp8 (fp32 arithmetic)",
        "data": "synthetic",
        "config": {"workload": "config 2: amax + dynamic_scaled_quant per tensor, bf16 [8192,8192] N(0,1) with 0.1% x100 "
                               "outliers -> fp32 amax, scales, e4m3fn and e5m2; value counts the 268.4 MB the step must "
                               "move (x once, two fp8 outputs)",
                   "buffer_sets": ns, "product_rounding": "bf16 product, bf16-rounded scale (eager with a 0-dim scale)",
                   "exclusive_gpu": "opted in (dt_set_exclusive_gpu): the step is the one-kernel path; the default for callers "
                                    "that have not opted in is two_kernel_path"},
        # achieved = the bytes the kernel must move (x once + two fp8 outputs: 4 B per element, its lower
        # bound) / average launch time, so frac is a fraction of the HBM peak and cannot exceed 1.  `traffic`
        # is what rocprofv3 FETCH_SIZE + WRITE_SIZE saw per launch (scaled by a plain copy), read from the
        # committed summary of those runs.  The two-pass figure of 6 B per element (x read by the reduction and again
        # by the cast, as two kernels would) over the same time is two_pass_equivalent_GBs.
        "roofline": {"kernel": "resident_quant_kernel<bf16, e4m3fn+e5m2 pair>", "bound": "hbm", "achieved": round(step_gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(step_gbs / HBM_PEAK_GBS, 4),
                     "avg_launch_us": round(step_us, 2), "algorithmic_bytes_per_launch": step_bytes,
                     "min_traffic_bytes": step_bytes, "frac_of_min_traffic": round(step_gbs / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": str(TRAFFIC_PROFILE.relative_to(ROOT)) if traffic else None,
                     "traffic_rate_GBs": round(traffic / (step_us * 1e-6) / 1e9, 1) if traffic else None,
                     "two_pass_algorithmic_bytes": two_pass_bytes,
                     "two_pass_equivalent_GBs": round(two_pass_bytes / (step_us * 1e-6) / 1e9, 1)},
        "two_kernel_path": {"step_us": round(two_kernel_us, 2),
                            "GBs of the 6 B per element its two kernels read and write": round(two_pass_bytes / (two_kernel_us * 1e-6) / 1e9, 1),
                            "cast_kernel(pair) inside the step, event pair per launch, us": round(cast_us, 2),
                            "cast_kernel(pair) GBs (4 B per element)": round(cast_bytes / (cast_us * 1e-6) / 1e9, 1),
                            "cast_kernel(pair) traffic": cast_traffic},
    }
    if args.calibrate_copy:
        src = xs[0]
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # 128 MiB read + 128 MiB written per launch
        torch.cuda.synchronize()
        del dst
    del xs, o4, o5
    torch.cuda.empty_cache()

    if not args.no_extra:
        result["kernels"] = extra_kernels(torch, cabi, dev, KX, WX, phases=phases)
    if phases:
        result["phases"] = phases
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, x_cpu, step_bytes)
    print(json.dumps(result))


def kernel_phases(torch, cabi, launch, names, launches=20):
    """Where a kernel spends its time: with a phase log set (dt_set_phase_log) every workgroup of the
    one-kernel dynamic quantization and of the amax reduction writes four readings of the 100 MHz
    constant-rate counter (start and three phase ends, `names`), collected here over `launches`
    launches of `launch(i)` with a synchronisation after each.  All figures in microseconds, medians
    over the launches; t = 0 is the first workgroup's start."""
    L = cabi.lib()
    log = torch.zeros((1024, 4), dtype=torch.int64, device="cuda")
    assert L.dt_set_phase_log(log.data_ptr(), log.numel() * 8) == 0
    rows = []
    try:
        for i in range(launches + 3):
            log.zero_()
            launch(i)
            torch.cuda.synchronize()
            t = log.cpu().double()
            t = t[t[:, 0] > 0]  # workgroups of the grid
            if i < 3 or t.numel() == 0:
                continue
            t = (t - t[:, 0].min()) / 100.0  # 100 MHz -> us
            med = lambda v: float(v.median())  # noqa: E731
            row = {"workgroups": int(t.shape[0]), "last_workgroup_starts_at": float(t[:, 0].max())}
            for k, name in enumerate(names, start=1):
                row[f"{name}: per workgroup, median"] = med(t[:, k] - t[:, k - 1])
                row[f"{name}: first workgroup done at"] = float(t[:, k].min())
                row[f"{name}: median workgroup done at"] = med(t[:, k])
                row[f"{name}: last workgroup done at"] = float(t[:, k].max())
            # by XCD (workgroup b runs on XCD b % 8): when each XCD's slowest workgroup is done with everything
            if t.shape[0] % 8 == 0:
                row["last phase done at, slowest workgroup of each XCD"] = [float(t[x::8, 3].max()) for x in range(8)]
            rows.append(row)
    finally:
        L.dt_set_phase_log(None, 0)
    if not rows:
        return None
    out = {}
    for k in rows[0]:
        if isinstance(rows[0][k], list):
            out[k] = [round(statistics.median(r[k][x] for r in rows), 2) for x in range(len(rows[0][k]))]
        else:
            out[k] = round(statistics.median(r[k] for r in rows), 2)
    out["launches"] = len(rows)
    out["unit"] = "us (100 MHz counter, 0.01 us resolution)"
    return out


def gemm_ramp(torch, cabi, dev, windows=24, per_window=25):
    """Launch time of the config-5 GEMM in consecutive windows of `per_window` launches, first after a
    stretch of HBM-bound kernels (what precedes the GEMM rows in the default run), then after two seconds
    of idling: the shader clock under sustained MFMA load needs on the order of a hundred launches to
    settle, which is why the GEMM rows of the per-kernel table warm up with 150 launches."""
    import time

    e4, bf16 = torch.float8_e4m3fn, torch.bfloat16
    M = N = Kd = 8192
    g = torch.Generator().manual_seed(7)
    a = torch.randn((M, Kd), generator=g).to(bf16).to(dev)
    b = torch.randn((N, Kd), generator=g).to(bf16).to(dev)
    a_data, sfa = cabi.mx_fp8_quantize(a, 1, False, e4, cabi.SCALE_BLOCKED)
    b_data, sfb = cabi.mx_fp8_quantize(b, 1, False, e4, cabi.SCALE_BLOCKED)
    out = torch.empty((M, N), dtype=bf16, device=dev)
    gemm = bind(cabi, lambda: cabi.mx_fp8_bf16(a_data, b_data, sfa, sfb, out))
    amax = bind(cabi, lambda: cabi.amax(a))

    def train():
        ev = _events(windows + 1)
        ev[0].record()
        for w in range(windows):
            for _ in range(per_window):
                gemm()
            ev[w + 1].record()
        torch.cuda.synchronize()
        return [round(ev[w].elapsed_time(ev[w + 1]) * 1e3 / per_window, 1) for w in range(windows)]

    gemm()
    for _ in range(300):
        amax()
    torch.cuda.synchronize()
    after_hbm = train()
    time.sleep(2.0)
    after_idle = train()
    return {"kernel": "mx_fp8_bf16", "workload": "config 5: 8192^3 e4m3, N(0,1)-derived operands", "launches_per_window": per_window,
            "us_per_launch_after_300_amax_launches": after_hbm, "us_per_launch_after_2s_idle": after_idle}


def gemm_timeline(torch, cabi, launch, launches=5):
    """Where the block-scaled GEMM spends its time: with a phase log set every workgroup (= output tile)
    writes four readings of the 100 MHz constant-rate counter (start, K loop entered, K loop left, output
    stored) and the XCD and CU it ran on.  Medians over `launches` launches, each in a train of warm
    launches (the clocks need tens of launches to settle); microseconds."""
    import collections

    L = cabi.lib()
    log = torch.zeros((8192, 8), dtype=torch.int64, device="cuda")
    rows = []
    for _ in range(launches):
        for _ in range(30):
            launch()
        assert L.dt_set_phase_log(log.data_ptr(), log.numel() * 8) == 0
        try:
            log.zero_()
            launch()
            torch.cuda.synchronize()
        finally:
            L.dt_set_phase_log(None, 0)
        d = log.cpu()
        d = d[d[:, 0] > 0]
        if d.numel() == 0:
            return None
        t = (d[:, :4] - d[:, 0].min()).double() / 100.0
        xcc = (d[:, 4] & 0xF).tolist()
        hw = d[:, 5].tolist()
        per_cu = collections.defaultdict(list)
        for i in range(t.shape[0]):
            per_cu[(xcc[i], (hw[i] >> 8) & 0xF, (hw[i] >> 12) & 1, (hw[i] >> 13) & 7)].append(t[i].tolist())
        gaps = []
        for v in per_cu.values():
            v.sort()
            gaps += [b[0] - a[3] for a, b in zip(v, v[1:])]
        med = lambda v: float(torch.as_tensor(v, dtype=torch.float64).median())  # noqa: E731
        loop = t[:, 2] - t[:, 1]
        by_xcd = lambda col: [round(med([col[i] for i in range(len(xcc)) if xcc[i] == x]), 2) for x in sorted(set(xcc))]  # noqa: E731
        rows.append({
            "tiles": int(t.shape[0]), "CUs": len(per_cu), "kernel span (first start to last store)": float(t[:, 3].max()),
            "per tile: prologue (first stages and fragments in)": med(t[:, 1] - t[:, 0]),
            "per tile: K loop": med(loop), "per tile: epilogue (convert, stage, stores issued and performed)": med(t[:, 3] - t[:, 2]),
            "per CU: gap between a tile's end and the next one's start": med(gaps) if gaps else 0.0,
            "K loop by XCD": by_xcd(loop.tolist()),
            "last store by XCD": [round(max(t[i, 3].item() for i in range(len(xcc)) if xcc[i] == x), 2) for x in sorted(set(xcc))],
        })
    out = {}
    for k in rows[0]:
        if isinstance(rows[0][k], list):
            out[k] = [round(statistics.median(r[k][x] for r in rows), 2) for x in range(len(rows[0][k]))]
        else:
            out[k] = round(statistics.median(r[k] for r in rows), 2)
    out["launches"] = len(rows)
    out["unit"] = "us (100 MHz counter)"
    return out


def extra_kernels(torch, cabi, dev, K, W, gemm_only=False, phases=None):
    """Every other kernel of the path at its benchmark config: rotated (HBM) and hot-cache."""
    rows = []

    def hbm_row(name, workload, nbytes, make_set, run):
        one = make_set(0)
        set_bytes = sum(t.numel() * t.element_size() for t in one if isinstance(t, torch.Tensor))
        ns = nsets_for(set_bytes)
        sets = [one] + [make_set(i) for i in range(1, ns)]
        bound = [bind(cabi, run, *st) for st in sets]
        us = time_launches(lambda i: bound[i](), ns, K, W)
        us_hot = time_launches(lambda i: bound[0](), 1, K, W)
        gbs = nbytes / (us * 1e-6) / 1e9
        rows.append({"kernel": name, "workload": workload, "bound": "hbm", "avg_us": round(us, 2),
                     "achieved_GBs": round(gbs, 1), "frac_of_8TBs": round(gbs / HBM_PEAK_GBS, 4),
                     "hot_cache_us": round(us_hot, 2), "hot_cache_GBs": round(nbytes / (us_hot * 1e-6) / 1e9, 1),
                     "algorithmic_bytes": nbytes, "buffer_sets": ns})
        del sets
        torch.cuda.empty_cache()

    bf16, f32 = torch.bfloat16, torch.float32
    e4, e5 = torch.float8_e4m3fn, torch.float8_e5m2
    scale1 = torch.full((1,), 37.0, device=dev)

    def rnd(shape, dtype, i):
        g = torch.Generator(device=dev).manual_seed(77 + i)
        return torch.randn(shape, generator=g, device=dev, dtype=torch.float32).to(dtype)

    def hbm_rows():
        n = 8192 * 8192
        hbm_row("amax", "bf16 [8192,8192]", n * 2, lambda i: (rnd((8192, 8192), bf16, i), torch.empty(1, device=dev)),
                lambda x, o: cabi.amax(x, o))
        hbm_row("amax", "fp32 [8192,8192]", n * 4, lambda i: (rnd((8192, 8192), f32, i), torch.empty(1, device=dev)),
                lambda x, o: cabi.amax(x, o))
        for od, nm in ((e4, "e4m3fn"), (e5, "e5m2")):
            hbm_row("saturated_cast", f"bf16 [8192,8192] -> {nm}", n * 3,
                    lambda i, od=od: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=od, device=dev)),
                    lambda x, o, od=od: cabi.saturated_cast(x, scale1, od, cabi.ROUND_BF16_SCALE_PRODUCT, o))
        n1 = 4096 * 4096
        hbm_row("saturated_cast", "config 1: bf16 [4096,4096] -> e4m3fn", n1 * 3,
                lambda i: (rnd((4096, 4096), bf16, i), torch.empty((4096, 4096), dtype=e4, device=dev)),
                lambda x, o: cabi.saturated_cast(x, scale1, e4, cabi.ROUND_BF16_SCALE_PRODUCT, o))
        hbm_row("saturated_cast", "fp32 [8192,8192] -> e4m3fn", n * 5,
                lambda i: (rnd((8192, 8192), f32, i), torch.empty((8192, 8192), dtype=e4, device=dev)),
                lambda x, o: cabi.saturated_cast(x, scale1, e4, cabi.ROUND_F32, o))
        # bytes of the dynamic rows: what the kernel must move (x once for the part the chip holds)
        hbm_row("dynamic_scaled_quant (one resident kernel)", "bf16 [8192,8192] -> amax, scale, e4m3fn", n * 3,
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty(1, device=dev), torch.empty(1, device=dev)),
                lambda x, o, a, s_: cabi.dynamic_scaled_quant(x, e4, cabi.ROUND_BF16_SCALE_PRODUCT, o, a, s_))
        # twice what the chip holds: 128 MiB stays in registers and LDS, the other 128 MiB is read twice
        n2 = 16384 * 8192
        hbm_row("dynamic_scaled_quant pair, 2 x the chip's capacity", "bf16 [16384,8192] -> amax, scales, e4m3fn and e5m2", n2 * 5,
                lambda i: (rnd((16384, 8192), bf16, i), torch.empty((16384, 8192), dtype=e4, device=dev),
                           torch.empty((16384, 8192), dtype=e5, device=dev), torch.empty(1, device=dev), torch.empty(2, device=dev)),
                lambda x, o4, o5, a, s_: cabi.dynamic_scaled_quant_pair(x, cabi.ROUND_BF16_SCALE_PRODUCT, o4, o5, a, s_))
        nr = 16384 * 4096
        for dt_, nm, b in ((f32, "fp32", 4), (bf16, "bf16", 2)):
            hbm_row("dynamic_scaled_quant_rowwise", f"config 3: {nm} [16384,4096] -> e4m3fn", nr * (b + 1) + 16384 * 8,
                    lambda i, dt_=dt_: (rnd((16384, 4096), dt_, i), torch.empty((16384, 4096), dtype=e4, device=dev),
                                        torch.empty((16384, 1), device=dev), torch.empty((16384, 1), device=dev)),
                    lambda x, o, a, s: cabi.dynamic_scaled_quant_rowwise(x, e4, o, a, s))
        mxb = n * 2 + n + n // 32
        hbm_row("mx_fp8_quantize rows", "config 4: bf16 [8192,8192], blocks along rows", mxb,
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty((8192, 256), dtype=torch.uint8, device=dev)),
                lambda x, dd, s: cabi.mx_fp8_quantize(x, 1, False, e4, cabi.SCALE_PLAIN, dd, s))
        nblk = cabi.lib().dt_blocked_scale_bytes(8192, 256)
        hbm_row("mx_fp8_quantize rows, blocked scales", "config 4: bf16 [8192,8192], scales in the GEMM's layout", mxb,
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty((nblk,), dtype=torch.uint8, device=dev)),
                lambda x, dd, s: cabi.mx_fp8_quantize(x, 1, False, e4, cabi.SCALE_BLOCKED, dd, s))
        hbm_row("mx_fp8_quantize_dual (rows + transposed columns from one read)",
                "config 4: bf16 [8192,8192], blocked scales", n * 2 + 2 * (n + n // 32),
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty((nblk,), dtype=torch.uint8, device=dev), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty((nblk,), dtype=torch.uint8, device=dev)),
                lambda x, dr, sr, dc, sc: cabi.mx_fp8_quantize_dual(x, e4, cabi.SCALE_BLOCKED, (dr, sr, dc, sc)))
        hbm_row("mx_fp8_quantize cols (transposed out)", "config 4: bf16 [8192,8192], blocks down columns", mxb,
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty((8192, 256), dtype=torch.uint8, device=dev)),
                lambda x, dd, s: cabi.mx_fp8_quantize(x, 0, True, e4, cabi.SCALE_PLAIN, dd, s))
        hbm_row("mx_fp8_quantize cols (in place)", "config 4: bf16 [8192,8192], blocks down columns", mxb,
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 8192), dtype=e4, device=dev),
                           torch.empty((256, 8192), dtype=torch.uint8, device=dev)),
                lambda x, dd, s: cabi.mx_fp8_quantize(x, 0, False, e4, cabi.SCALE_PLAIN, dd, s))
        # the cast that makes mx_fp4_bf16's operands: 2 B in, 1/2 B + 1/32 B out per element
        hbm_row("mx_fp4_quantize rows, blocked scales", "bf16 [8192,8192] -> packed e2m1 + E8M0, scales in the GEMM's layout",
                8192 * 8192 * (2 + 0.5 + 1 / 32),
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 4096), dtype=torch.uint8, device=dev),
                           torch.empty((nblk,), dtype=torch.uint8, device=dev)),
                lambda x, dd, sc: cabi.mx_fp4_quantize(x, cabi.SCALE_BLOCKED, dd, sc))

        nblk_c = cabi.lib().dt_blocked_scale_bytes(8192, 256)
        hbm_row("mx_fp4_quantize_dual (rows + transposed columns from one read)",
                "bf16 [8192,8192] -> two packed e2m1 payloads + E8M0, blocked scales", 8192 * 8192 * (2 + 2 * (0.5 + 1 / 32)),
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 4096), dtype=torch.uint8, device=dev),
                           torch.empty((nblk,), dtype=torch.uint8, device=dev), torch.empty((8192, 4096), dtype=torch.uint8, device=dev),
                           torch.empty((nblk_c,), dtype=torch.uint8, device=dev)),
                lambda x, dr, sr, dc, sc: cabi.mx_fp4_quantize_dual(x, cabi.SCALE_BLOCKED, (dr, sr, dc, sc)))
        hbm_row("mx_fp4_quantize cols (transposed out), blocked scales", "bf16 [8192,8192] -> packed e2m1 [8192,4096] + E8M0",
                8192 * 8192 * (2 + 0.5 + 1 / 32),
                lambda i: (rnd((8192, 8192), bf16, i), torch.empty((8192, 4096), dtype=torch.uint8, device=dev),
                           torch.empty((nblk_c,), dtype=torch.uint8, device=dev)),
                lambda x, dd, sc: cabi.mx_fp4_quantize(x, cabi.SCALE_BLOCKED, dd, sc, 0))

    if not gemm_only:
        hbm_rows()

    # MXFP8 GEMM, config 5
    M = N = Kd = 8192
    a = rnd((M, Kd), bf16, 1)
    b = rnd((N, Kd), bf16, 2)
    a_data, sfa = cabi.mx_fp8_quantize(a, 1, False, e4, cabi.SCALE_BLOCKED)
    b_data, sfb = cabi.mx_fp8_quantize(b, 1, False, e4, cabi.SCALE_BLOCKED)
    out = torch.empty((M, N), dtype=bf16, device=dev)
    del a, b
    # The clock under sustained MFMA load settles over some 50 ms (30 warm-up launches and 25 timed ones read
    # 5 % slower than the steady state that 150 + 100 launches reach): the GEMM rows report the steady state.
    GEMM_WARMUP, GEMM_STEPS = max(150, W), max(100, K // 2)
    gemm8 = bind(cabi, lambda: cabi.mx_fp8_bf16(a_data, b_data, sfa, sfb, out))
    # The row's figure is the usual GEMM measurement, the same launch over and over on one operand set
    # (the kernel is bound by the MFMA pipe and the power limit, not by HBM).  Beside it: rotating over
    # three operand sets that together exceed the 256 MB memory-side cache (3 x 260 MB of operands, scales
    # and output), so that every launch takes its operands from HBM (rotated_us, 2-3 % slower).
    more = []
    for sset in (3, 5):
        a2, sa2 = cabi.mx_fp8_quantize(rnd((M, Kd), bf16, sset), 1, False, e4, cabi.SCALE_BLOCKED)
        b2, sb2 = cabi.mx_fp8_quantize(rnd((N, Kd), bf16, sset + 1), 1, False, e4, cabi.SCALE_BLOCKED)
        more.append((a2, b2, sa2, sb2, torch.empty((M, N), dtype=bf16, device=dev)))
    gemm_sets = [gemm8] + [bind(cabi, lambda t=t: cabi.mx_fp8_bf16(*t)) for t in more]
    us_rot = time_launches(lambda i: gemm_sets[i](), len(gemm_sets), GEMM_STEPS, GEMM_WARMUP)
    us = time_launches(lambda i: gemm8(), 1, GEMM_STEPS, GEMM_WARMUP)
    del more, gemm_sets
    flops = 2.0 * M * N * Kd
    tf = flops / (us * 1e-6) / 1e12
    if phases is not None:
        phases["mx_gemm_kernel, config 5 (8192^3 e4m3)"] = gemm_timeline(
            torch, cabi, gemm8)
    rows.append({"kernel": "mx_fp8_bf16", "workload": "config 5: 8192^3 e4m3 x e4m3, E8M0 block-32 scales -> bf16",
                 "bound": "mfma", "avg_us": round(us, 2), "achieved_TFLOPs": round(tf, 1),
                 "frac_of_fp8_peak": round(tf / FP8_PEAK_TFLOPS, 4), "flops": flops, "buffer_sets": 1,
                 "rotated_us": round(us_rot, 2), "rotated_TFLOPs": round(flops / (us_rot * 1e-6) / 1e12, 1), "rotated_buffer_sets": 3})
    # The same launch on operands of ones (payload 0x38, scale bytes 127): the same schedule and the same
    # data movement with almost no switching in the multipliers.  The difference to the row above is the
    # shader clock the power management allows (cycles per launch are the same, see profiles/).
    ones_a = torch.full((M, Kd), 0x38, dtype=torch.uint8, device=dev).view(e4)
    ones_s = torch.full_like(sfa, 127)
    gemm1 = bind(cabi, lambda: cabi.mx_fp8_bf16(ones_a, ones_a, ones_s, ones_s, out))
    us1 = time_launches(lambda i: gemm1(), 1, GEMM_STEPS, GEMM_WARMUP)
    rows.append({"kernel": "mx_fp8_bf16", "workload": "8192^3, every operand element 1.0 (same schedule and traffic, little switching power)",
                 "bound": "mfma", "avg_us": round(us1, 2), "achieved_TFLOPs": round(flops / (us1 * 1e-6) / 1e12, 1),
                 "frac_of_fp8_peak": round(flops / (us1 * 1e-6) / 1e12 / FP8_PEAK_TFLOPS, 4), "flops": flops})
    del ones_a, ones_s
    # shapes off the 8192^3 grid, on row slices of the same operands (blocked scales are stored by 128-row
    # chunks, so a row prefix of the operand owns a prefix of its scales).  Each is warmed up for 40 ms first:
    # under MFMA load the shader clock needs tens of milliseconds to settle, whatever the launch's length
    def mfma_row(kernel, fn, ops, m_rows, n_rows, k_dim, what, peak, key):
        g_ = bind(cabi, lambda: fn(*ops))
        one = time_launches(lambda i: g_(), 1, 5, 2)
        us_ = time_launches(lambda i: g_(), 1, max(50, K // 2), max(20, int(40e3 / max(one, 1.0))))
        fl = 2.0 * m_rows * n_rows * k_dim
        rows.append({"kernel": kernel, "workload": f"{m_rows}x{n_rows}x{k_dim} {what}", "bound": "mfma", "avg_us": round(us_, 2),
                     "achieved_TFLOPs": round(fl / (us_ * 1e-6) / 1e12, 1), key: round(fl / (us_ * 1e-6) / 1e12 / peak, 4), "flops": fl})

    for m_rows, n_rows, k_dim, what in ((1024, 8192, 8192, "e4m3 (128 tiles of 256x256 on 256 CUs: runs as 256 tiles of 256x128)"),
                                        (4096, 4096, 4096, "e4m3 (256 tiles of 256x256: exactly one round of the chip)"),
                                        (5120, 5120, 5120, "e4m3 (400 tiles: one round of 256x256 tiles, the other 144 as 256x128 halves or a second round)"),
                                        (2048, 8192, 8192, "e4m3 (256 tiles, one round)")):
        sa_rows = -(-m_rows // 128) * 128 * (Kd // 32)
        sb_rows = -(-n_rows // 128) * 128 * (Kd // 32)
        if k_dim == Kd:
            ops = (a_data[:m_rows], b_data[:n_rows], sfa[:sa_rows], sfb[:sb_rows], out[:m_rows, :n_rows])
        else:  # a shorter K: operands of their own (the blocked scale layout depends on K)
            a_s, sa_s = cabi.mx_fp8_quantize(rnd((m_rows, k_dim), bf16, 11), 1, False, e4, cabi.SCALE_BLOCKED)
            b_s, sb_s = cabi.mx_fp8_quantize(rnd((n_rows, k_dim), bf16, 12), 1, False, e4, cabi.SCALE_BLOCKED)
            ops = (a_s, b_s, sa_s, sb_s, torch.empty((m_rows, n_rows), dtype=bf16, device=dev))
        mfma_row("mx_fp8_bf16", cabi.mx_fp8_bf16, ops, m_rows, n_rows, k_dim, what, FP8_PEAK_TFLOPS, "frac_of_fp8_peak")

    # Few rows (decode shapes): one pass over B, whose payload and scale bytes are the algorithmic bytes.  B rotates
    # over enough operand sets to leave the 256 MB memory-side cache, so that every launch reads it from HBM;
    # hot_cache_us is the same launch on one set.
    def few_rows_row(kernel, fp4, m_rows):
        nb = N * Kd // (2 if fp4 else 1) + N * Kd // 32
        ns_ = nsets_for(nb)
        sets_ = []
        for i in range(ns_):
            src = rnd((N, Kd), bf16, 20 + i)
            sets_.append(cabi.mx_fp4_quantize(src, cabi.SCALE_BLOCKED) if fp4 else cabi.mx_fp8_quantize(src, 1, False, e4, cabi.SCALE_BLOCKED))
            del src
        a_src = rnd((m_rows, Kd), bf16, 1)
        a_q, sa_q = cabi.mx_fp4_quantize(a_src, cabi.SCALE_BLOCKED) if fp4 else cabi.mx_fp8_quantize(a_src, 1, False, e4, cabi.SCALE_BLOCKED)
        o_ = torch.empty((m_rows, N), dtype=bf16, device=dev)
        fn = cabi.mx_fp4_bf16 if fp4 else cabi.mx_fp8_bf16
        bound_ = [bind(cabi, lambda bq=bq, sq=sq: fn(a_q, bq, sa_q, sq, o_)) for bq, sq in sets_]
        us_ = time_launches(lambda i: bound_[i](), ns_, max(50, K // 2), 20)
        hot_ = time_launches(lambda i: bound_[0](), 1, max(50, K // 2), 20)
        rows.append({"kernel": kernel, "workload": f"{m_rows}x{N}x{Kd} {'e2m1' if fp4 else 'e4m3'} (few rows, one pass over B; the library picks "
                     "the kernel: B straight from memory into the MFMA's registers and A through LDS, or, for e4m3 with more than 32 "
                     "rows at this size, 128x128 tiles with K shared between workgroups)", "bound": "hbm", "avg_us": round(us_, 2),
                     "achieved_GBs": round(nb / us_ / 1e3, 1), "frac_of_8TBs": round(nb / us_ / 1e3 / HBM_PEAK_GBS, 4),
                     "hot_cache_us": round(hot_, 2), "algorithmic_bytes": nb, "buffer_sets": ns_})
        del sets_, bound_
        torch.cuda.empty_cache()

    few_rows_row("mx_fp8_bf16", False, 16)
    few_rows_row("mx_fp8_bf16", False, 64)
    # MXFP4 GEMM, same shape: the MXFP4 cast of the same N(0,1) operands, scales blocked by the cast
    del a_data, b_data
    a4, s4a = cabi.mx_fp4_quantize(rnd((M, Kd), bf16, 1), cabi.SCALE_BLOCKED)
    b4, s4b = cabi.mx_fp4_quantize(rnd((N, Kd), bf16, 2), cabi.SCALE_BLOCKED)
    gemm4 = bind(cabi, lambda: cabi.mx_fp4_bf16(a4, b4, s4a, s4b, out))
    us = time_launches(lambda i: gemm4(), 1, GEMM_STEPS, GEMM_WARMUP)
    tf = flops / (us * 1e-6) / 1e12
    rows.append({"kernel": "mx_fp4_bf16", "workload": "8192^3 e2m1 x e2m1, E8M0 block-32 scales -> bf16",
                 "bound": "mfma", "avg_us": round(us, 2), "achieved_TFLOPs": round(tf, 1),
                 "frac_of_fp4_peak": round(tf / FP4_PEAK_TFLOPS, 4), "flops": flops})
    del a4, b4, s4a, s4b
    torch.cuda.empty_cache()
    few_rows_row("mx_fp4_bf16", True, 16)
    return rows


def cpu_baseline(torch, x_cpu, step_bytes):
    """The eager formulation the reference's tests use, on this host's cores."""
    from oracle import eager

    cores = os.cpu_count() or 1
    # worker pools are sized to the box's CPU share, whatever cpu_count says
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)

    def once():
        t0 = time.perf_counter()
        for od in (torch.float8_e4m3fn, torch.float8_e5m2):
            eager.dynamic_scaled_quant(x_cpu, od)
        return time.perf_counter() - t0

    once()
    ts, t_start = [], time.perf_counter()
    while len(ts) < 3 or (time.perf_counter() - t_start < 10.0 and len(ts) < 500):  # about 10 s of CPU work
        ts.append(once())
    t = statistics.median(ts)
    model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": round(step_bytes / t / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "the whole config-2 tensor (bf16 8192x8192), eager amax -> scale -> cast for e4m3fn and e5m2, "
                      f"median of {len(ts)} passes (about 10 s) after one warm-up",
            "seconds": round(t, 3), "cpu": model}


if __name__ == "__main__":
    main()
