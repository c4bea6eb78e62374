"""GPU parity on seeded random shapes: every cast of the path against the CPU oracle, bit for bit,
on shapes that are not multiples of any tile or vector size (within what each op accepts)."""
import random

import pytest
import torch

from oracle import c_oracle as co
from tests import util

pytestmark = pytest.mark.gpu

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


@pytest.fixture(scope="module")
def d(gpu_device):
    import driss_torch_amd

    return driss_torch_amd


def _shapes(seed, n, row_mult=1, col_mult=1, max_rows=700, max_cols=1500):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        r = rng.randint(1, max_rows // row_mult) * row_mult
        c = rng.randint(1, max_cols // col_mult) * col_mult
        out.append((r, c))
    return out


def _data(shape, seed, dtype):
    g = util.gen(seed)
    x = torch.randn(shape, generator=g) * torch.exp(2.5 * torch.randn(shape, generator=g))
    flat = x.flatten()
    if flat.numel() > 7:  # a few exact zeros and one large value somewhere
        flat[torch.randint(0, flat.numel(), (3,), generator=g)] = 0.0
        flat[torch.randint(0, flat.numel(), (1,), generator=g)] = 3.0e4
    return x.to(dtype)


@pytest.mark.parametrize("shape", _shapes(1, 12), ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_per_tensor_ops_random_shapes(d, shape, in_dtype):
    x = _data(shape, shape[0] * 31 + shape[1], in_dtype)
    g = x.cuda()
    assert d.amax(g).item() == co.amax(x).item()
    for fp8 in (E4, E5):
        modes = (1, 2, 3) if in_dtype == torch.bfloat16 else (3,)
        for mode in modes:
            out, amax, scale = d.dynamic_scaled_quant_ex(g, fp8, mode)
            ref, ramax, rscale = co.dynamic_scaled_quant(x, fp8, mode)
            assert torch.equal(util.codes(out), ref) and amax.item() == ramax.item() and scale.item() == rscale.item()
            got = d.saturated_cast_mode(g, scale.reshape(1), fp8, mode)
            assert torch.equal(util.codes(got), co.saturated_cast(x, rscale.item(), fp8, mode))
        out, amax, scale = d.dynamic_scaled_quant_rowwise(g, fp8)
        ref, ramax, rscale = co.dynamic_scaled_quant_rowwise(x, fp8)
        assert torch.equal(util.codes(out), ref) and torch.equal(amax.cpu(), ramax) and torch.equal(scale.cpu(), rscale)


@pytest.mark.parametrize("shape", _shapes(2, 6, 1, 32) + _shapes(3, 6, 32, 4) + _shapes(4, 6, 32, 32), ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_mx_casts_random_shapes(d, shape, in_dtype):
    x = _data(shape, shape[0] * 17 + shape[1], in_dtype)
    g = x.cuda()
    rows, cols = shape
    if cols % 32 == 0:  # the MXFP4 cast, plain and blocked scales
        fd, fs = co.mx_fp4_quantize(x)
        for blocked in (False, True):
            data, scale = d.mx_fp4_quantize(g, blocked)
            assert torch.equal(data.cpu(), fd) and torch.equal(util.codes(scale), (co.to_blocked(fs) if blocked else fs).flatten())
    if rows % 32 == 0 and cols % 4 == 0:  # ... and down the columns (the cast of x^T)
        fd, fs = co.mx_fp4_quantize(x.t().contiguous())
        for blocked in (False, True):
            data, scale = d.mx_fp4_quantize(g, blocked, 0)
            assert torch.equal(data.cpu(), fd) and torch.equal(util.codes(scale), (co.to_blocked(fs) if blocked else fs).flatten())
    for fp8 in (E4, E5):
        if cols % 32 == 0:
            rd, rs = co.mx_quantize(x, axis=1, transpose=False, out_dtype=fp8)
            data, scale = d.mx_fp8_quantize(g, 32, 1, False, fp8)
            assert torch.equal(util.codes(data), rd) and torch.equal(util.codes(scale), rs.flatten())
            data, scale = d.mx_fp8_quantize_blocked(g, 1, fp8)
            assert torch.equal(util.codes(data), rd) and torch.equal(util.codes(scale), co.to_blocked(rs))
        if rows % 32 == 0:
            cd, cs = co.mx_quantize(x, axis=0, transpose=True, out_dtype=fp8)
            data, scale = d.mx_fp8_quantize(g, 32, 0, True, fp8)
            assert torch.equal(util.codes(data), cd) and torch.equal(util.codes(scale), cs.flatten())
            data, scale = d.mx_fp8_quantize(g, 32, 0, False, fp8)
            assert torch.equal(util.codes(data), cd.t()) and torch.equal(util.codes(scale).view(cs.shape[1], cs.shape[0]), cs.t())
            data, scale = d.mx_fp8_quantize_blocked(g, 0, fp8)
            assert torch.equal(util.codes(data), cd) and torch.equal(util.codes(scale), co.to_blocked(cs))
        if rows % 32 == 0 and cols % 32 == 0:
            for blocked in (False, True):
                dr, sr, dc, sc = d.mx_fp8_quantize_dual(g, fp8, blocked)
                assert torch.equal(util.codes(dr), rd) and torch.equal(util.codes(dc), cd)
                assert torch.equal(util.codes(sr), (co.to_blocked(rs) if blocked else rs).flatten())
                assert torch.equal(util.codes(sc), (co.to_blocked(cs) if blocked else cs).flatten())
