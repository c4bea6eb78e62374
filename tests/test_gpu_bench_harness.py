"""The saturated-cast benchmark harness under test: its correctness leg over the reference's
eleven shapes x two fp8 types (benchmarks/benchmark_saturated_casting.py:46-76,100-108), incl. the
degenerate (1, 3232) and (2048, 1) and the wide (2048, 109760), and every output bit for bit against
the CPU oracle in the rounding mode a 0-dim device scale selects."""
import pytest
import torch

from oracle import c_oracle as co
from tests import util

pytestmark = pytest.mark.gpu


def test_harness_correctness_leg_matches_the_oracle(gpu_device):
    from driss_torch_amd.benchmarks import benchmark_saturated_casting as bench

    seen = []

    def on_checked(x, scale, lp, out):
        assert out.shape == x.shape and out.dtype == lp
        want = co.saturated_cast(x.cpu(), scale.item(), lp, co.ROUND_V2)
        assert torch.equal(util.codes(out), want), (tuple(x.shape), lp)
        seen.append((tuple(x.shape), lp))

    torch.manual_seed(46)
    rows = bench.run(False, timed=False, on_checked=on_checked)
    assert len(rows) == len(seen) == len(bench.SHAPES) * len(bench.LOW_PRECISION) == 22
    assert {s for s, _ in seen} >= {(1, 3232), (2048, 1), (2048, 109760)}


def test_harness_timed_table(gpu_device, capsys):
    """the timed leg and the printed table on two of the shapes (the whole table is what
    `python -m driss_torch_amd.benchmarks.benchmark_saturated_casting` prints)"""
    from driss_torch_amd.benchmarks import benchmark_saturated_casting as bench

    saved = bench.SHAPES
    bench.SHAPES = [(512, 512), (1, 3232)]
    try:
        # with the column of the reference's harness that times torch.compile of the eager formulation
        # (benchmarks/benchmark_saturated_casting.py:122-133)
        assert bench.main(["--compiled"]) == 0
    finally:
        bench.SHAPES = saved
    text = capsys.readouterr().out
    assert "hip_GBps" in text and "speedup_vs_eager" in text and text.count("bfloat16") == 4
    header, *table = [line.split() for line in text.strip().splitlines()]
    col = header.index("compiled_pytorch_time_us")
    assert len(table) == 4 and all(float(row[col]) > 0 for row in table)
