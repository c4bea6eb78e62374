"""GPU parity of the one-read MXFP8 cast that emits both blockings (rows, and columns with a
transposed payload), bit for bit against the CPU oracle and against two single casts; plus the
row-wise cast's 4-row pass for blocked scales."""
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


@pytest.fixture()
def cabi(gpu_device):
    from driss_torch_amd import cabi as c

    keep = {k: c.get_tuning(k) for k in ("mx.dual", "mx.row_band4", "mx.colt_via_dual")}
    yield c
    for k, v in keep.items():
        c.set_tuning(k, v)


def _wide_range(shape, seed, dtype):
    g = util.gen(seed)
    x = torch.randn(shape, generator=g) * torch.exp(3.0 * torch.randn(shape, generator=g))
    return x.to(dtype)


@pytest.mark.parametrize("shape", [(32, 32), (128, 256), (160, 96), (96, 160), (992, 1312), (1024, 2048)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("out_dtype", [E4, E5])
@pytest.mark.parametrize("blocked", [False, True])
def test_dual_matches_oracle(d, shape, in_dtype, out_dtype, blocked):
    x = _wide_range(shape, 11 + shape[1], in_dtype)
    dr, sr, dc, sc = d.mx_fp8_quantize_dual(x.cuda(), out_dtype, blocked)
    rd, rs = co.mx_quantize(x, axis=1, transpose=False, out_dtype=out_dtype)
    cd, cs = co.mx_quantize(x, axis=0, transpose=True, out_dtype=out_dtype)
    assert dr.shape == shape and dc.shape == (shape[1], shape[0]) and dr.dtype == dc.dtype == out_dtype
    assert torch.equal(util.codes(dr), rd) and torch.equal(util.codes(dc), cd)
    if blocked:
        rs, cs = co.to_blocked(rs), co.to_blocked(cs)
    assert torch.equal(util.codes(sr), rs.flatten()) and torch.equal(util.codes(sc), cs.flatten())


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_dual_special_blocks(d, cabi, in_dtype):
    """zero blocks, NaN and infinity in either direction, the largest and smallest magnitudes: the
    one-read kernel, the two-pass fallback and the oracle agree"""
    x = util.student_t((256, 512), 3, in_dtype)
    x[0:32, 5] = 0
    x[40, 64:96] = 0
    x[7, 40] = float("nan")
    x[130, 300] = float("inf")
    x[200, 17] = float("-inf")
    big = torch.finfo(in_dtype).max
    x[64:96, 100:132] = big
    x[100, 400] = torch.finfo(in_dtype).tiny
    x[96:128, 256:288] = torch.finfo(in_dtype).tiny / 4  # subnormal blocks
    g = x.cuda()
    for out_dtype in (E4, E5):
        cabi.set_tuning("mx.dual", 1)
        one = d.mx_fp8_quantize_dual(g, out_dtype)
        cabi.set_tuning("mx.dual", 0)
        two = d.mx_fp8_quantize_dual(g, out_dtype)
        cabi.set_tuning("mx.dual", 1)
        rd, rs = co.mx_quantize(x, axis=1, transpose=False, out_dtype=out_dtype)
        cd, cs = co.mx_quantize(x, axis=0, transpose=True, out_dtype=out_dtype)
        for got in (one, two):
            assert torch.equal(util.codes(got[0]), rd) and torch.equal(util.codes(got[1]), rs.flatten())
            assert torch.equal(util.codes(got[2]), cd) and torch.equal(util.codes(got[3]), cs.flatten())


def test_dual_feeds_the_gemm(d):
    """x [M, K] quantized once gives the A operand of x @ w^T (row blocks) and, transposed, the A operand of
    x^T @ g (column blocks): both products against the dequantized fp64 matmul"""
    from oracle import eager

    M, K, N = 256, 384, 128
    x, w, g = util.normal((M, K), 1).cuda(), util.normal((N, K), 2).cuda(), util.normal((M, N), 3).cuda()
    xr, xrs, xt, xts = d.mx_fp8_quantize_dual(x, E4, True)
    wd, ws = d.mx_fp8_quantize_blocked(w)
    y = d.mx_fp8_bf16(xr, wd.t(), xrs, ws)  # [M, N]
    gt, gts = d.mx_fp8_quantize_blocked(g, axis=0)  # g^T [N, M] with blocks along M
    dw = d.mx_fp8_bf16(xt, gt.t(), xts, gts)  # x^T g: [K, N]
    deq = lambda t, ax, tr: co.mx_dequant(*co.mx_quantize(t.cpu(), axis=ax, transpose=tr)).double()  # noqa: E731
    ref_y = deq(x, 1, False) @ deq(w, 1, False).T
    ref_dw = deq(x, 0, True) @ deq(g, 0, True).T
    assert eager.compute_error(ref_y, y.cpu().double()).item() > 50
    assert eager.compute_error(ref_dw, dw.cpu().double()).item() > 50


def test_dual_errors_and_compile(d):
    x = util.normal((64, 48), 5).cuda()
    with pytest.raises(RuntimeError):
        d.mx_fp8_quantize_dual(x)  # 48 % 32 != 0
    with pytest.raises(RuntimeError):
        d.mx_fp8_quantize_dual(util.normal((48, 64), 5).cuda())
    with pytest.raises(RuntimeError):
        d.mx_fp8_quantize_dual(x.t())
    x = util.normal((128, 256), 6).cuda()
    eager_out = d.mx_fp8_quantize_dual(x, E4, True)
    compiled = torch.compile(lambda t: d.mx_fp8_quantize_dual(t, E4, True), backend="aot_eager", fullgraph=True)(x)
    for a, b in zip(eager_out, compiled):
        assert a.shape == b.shape and torch.equal(util.codes(a), util.codes(b))


def test_dual_config4_full_size(d):
    x = util.student_t((8192, 8192), 1004)
    g = x.cuda()
    dr, sr, dc, sc = d.mx_fp8_quantize_dual(g)
    rd, rs = d.mx_fp8_quantize(g)
    cd, cs = d.mx_fp8_quantize(g, 32, 0, True)
    assert torch.equal(util.codes(dr), util.codes(rd)) and torch.equal(util.codes(sr), util.codes(rs))
    assert torch.equal(util.codes(dc), util.codes(cd)) and torch.equal(util.codes(sc), util.codes(cs))
    ord_, ors = co.mx_quantize(x[:512])
    assert torch.equal(util.codes(dr)[:512], ord_) and torch.equal(util.codes(sr)[: 512 * 256], ors.flatten())


@pytest.mark.parametrize("shape", [(128, 512), (384, 1536), (2048, 4096)], ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_row_cast_blocked_scales_four_row_pass(d, cabi, shape, in_dtype):
    """rows % 128 == 0 and cols % 512 == 0 take the pass that covers 4 rows x 512 elements; same
    bytes as the flat pass and as the oracle's to_blocked"""
    x = _wide_range(shape, 21, in_dtype)
    x[5, 33] = float("nan")
    g = x.cuda()
    for out_dtype in (E4, E5):
        rd, rs = co.mx_quantize(x, out_dtype=out_dtype)
        for band4 in (1, 0):
            cabi.set_tuning("mx.row_band4", band4)
            data, scale = d.mx_fp8_quantize_blocked(g, 1, out_dtype)
            assert torch.equal(util.codes(data), rd) and torch.equal(util.codes(scale), co.to_blocked(rs))


@pytest.mark.parametrize("out_dtype", [E4, E5])
def test_mx_casts_every_bf16_pattern(d, out_dtype):
    """all 65536 bf16 bit patterns, once with 32 neighbouring patterns per block (every block
    magnitude from subnormal to infinity, NaN blocks) and once shuffled, through the row, column,
    transposed-column and one-read kernels"""
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    perm = torch.randperm(65536, generator=util.gen(4))
    for x in (pats.reshape(2048, 32), pats.reshape(32, 2048).t().contiguous(), pats[perm].reshape(256, 256)):
        g = x.cuda()
        rd, rs = co.mx_quantize(x, axis=1, transpose=False, out_dtype=out_dtype)
        data, scale = d.mx_fp8_quantize(g, 32, 1, False, out_dtype)
        assert torch.equal(util.codes(data), rd) and torch.equal(util.codes(scale), rs.flatten())
        if x.shape[0] % 32 == 0:
            cd, cs = co.mx_quantize(x, axis=0, transpose=True, out_dtype=out_dtype)
            data, scale = d.mx_fp8_quantize(g, 32, 0, True, out_dtype)
            assert torch.equal(util.codes(data), cd) and torch.equal(util.codes(scale), cs.flatten())
            data, scale = d.mx_fp8_quantize(g, 32, 0, False, out_dtype)
            assert torch.equal(util.codes(data), cd.t()) and torch.equal(util.codes(scale).view(cs.shape[1], cs.shape[0]), cs.t())
            dr, sr, dc, sc = d.mx_fp8_quantize_dual(g, out_dtype)
            assert torch.equal(util.codes(dr), rd) and torch.equal(util.codes(sr), rs.flatten())
            assert torch.equal(util.codes(dc), cd) and torch.equal(util.codes(sc), cs.flatten())


@pytest.mark.parametrize("shape", [(32, 8), (64, 36), (128, 100), (160, 264), (992, 1312), (2048, 4096)], ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_transposed_column_cast_both_kernels(d, cabi, shape, in_dtype):
    """the transposed column cast runs as the one-read kernel without its row half when a lane's 8 (fp32: 4)
    columns are whole, otherwise (36 and 100 columns of 16-bit data) as the 4-columns-per-lane kernel; with
    the switch off always as the latter.  Both against the oracle, plain and blocked scales."""
    x = _wide_range(shape, 33, in_dtype)
    if shape[0] >= 64:
        x[40, 3] = float("nan")
        x[32:64, 5] = 0
    g = x.cuda()
    for out_dtype in (E4, E5):
        cd, cs = co.mx_quantize(x, axis=0, transpose=True, out_dtype=out_dtype)
        for via_dual in (1, 0):
            cabi.set_tuning("mx.colt_via_dual", via_dual)
            data, scale = d.mx_fp8_quantize(g, 32, 0, True, out_dtype)
            assert torch.equal(util.codes(data), cd) and torch.equal(util.codes(scale), cs.flatten())
            data, scale = d.mx_fp8_quantize_blocked(g, 0, out_dtype)
            assert torch.equal(util.codes(data), cd) and torch.equal(util.codes(scale), co.to_blocked(cs))
