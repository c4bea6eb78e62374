"""GPU parity of mx_fp4_bf16 (e2m1 operands, E8M0 block-32 scales) against the CPU oracle, on the
reference's size list (test/test_mx.py:42-59 with format "fp4"), with operands from the oracle's MXFP4
cast, and of mx_fp4_quantize (the device cast that makes such operands; the reference takes them from
torchao's MXTensor) bit for bit against the same oracle."""
import pytest
import torch

from oracle import c_oracle as co
from oracle import eager
from tests import util

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def d(gpu_device):
    import driss_torch_amd

    return driss_torch_amd


@pytest.fixture(scope="module")
def cabi(gpu_device):
    from driss_torch_amd import cabi as c

    return c


def _operands(M, K, N, seed, dist="rand"):
    mk = util.uniform if dist == "rand" else util.normal
    a, sa = co.mx_fp4_quantize(mk((M, K), seed, torch.float32))
    b, sb = co.mx_fp4_quantize(mk((N, K), seed + 1, torch.float32) * 3)
    return a, sa, b, sb


def _run(d, a, sa, b, sb):
    return d.mx_fp4_bf16(a.cuda(), b.cuda().t(), d.to_blocked(sa.cuda()), d.to_blocked(sb.cuda()))


def _check(d, M, K, N, seed, dist):
    a, sa, b, sb = _operands(M, K, N, seed, dist)
    out = _run(d, a, sa, b, sb)
    assert out.shape == (M, N) and out.dtype == torch.bfloat16
    da, db = eager.mx_fp4_dequant(a, sa), eager.mx_fp4_dequant(b, sb)
    ref = da @ db.T
    got = out.cpu().double()
    # Tolerance as for the e4m3 GEMM: products of e2m1 values are exact in fp32, the accumulation
    # is fp32 and the store rounds to bf16 (relative 2^-9), so every entry lies within
    # 2^-8 * sum_k |a||b| of the exact product; SQNR against the exact product > 50 dB (the
    # reference asks 80 dB against a bf16 matmul of the same operands, test/test_mx.py:64).
    bound = da.abs() @ db.abs().T
    err = (got - ref).abs()
    assert (err <= bound * 2**-8 + 1e-30).all(), f"max rel {(err / bound).max().item():.3e}"
    assert eager.compute_error(ref, got).item() > 50
    return out


@pytest.mark.parametrize("size", [(128, 128, 128), (256, 256, 256), (384, 384, 384), (512, 512, 512), (768, 768, 768),
                                  (1024, 1024, 1024), (128, 256, 384), (256, 384, 512), (129, 256, 384), (133, 512, 528)],
                         ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}")
@pytest.mark.parametrize("dist", ["rand", "randn"])
def test_mx_fp4_gemm_reference_sizes(d, size, dist):
    M, K, N = size
    _check(d, M, K, N, 900 + M + N, dist)


@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("size", [(128, 128, 128), (512, 256, 640), (133, 640, 528), (300, 1152, 264), (64, 2048, 8)])
def test_mx_fp4_gemm_both_tile_shapes(d, cabi, variant, size):
    """K = 128, 640, 1152 end in a half-filled 256-element step; K = 256, 2048 do not"""
    cabi.set_tuning("gemm.variant", variant)
    try:
        _check(d, *size, 950, "randn")
    finally:
        cabi.set_tuning("gemm.variant", 0)


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("K", [32, 64, 96, 160, 224, 288, 352, 480, 1312])
def test_mx_fp4_gemm_k_of_any_whole_number_of_blocks(d, cabi, variant, K):
    """K a multiple of 32 but not of 128: the last 256-element step holds 1..7 blocks (its second
    128-element half missing, partly or wholly filled); the K-blocks of the scale padding count as
    zero and the loads stay inside the rows (the output is checked against the exact product)"""
    cabi.set_tuning("gemm.variant", variant)
    try:
        _check(d, 133, K, 264, 970 + K, "randn")
    finally:
        cabi.set_tuning("gemm.variant", 0)


@pytest.mark.parametrize("size", [(1, 640, 8), (16, 2048, 256), (17, 96, 2056), (33, 1312, 264), (48, 480, 136), (64, 8192, 512),
                                  (5, 32, 24), (24, 4128, 4104), (8, 480, 264), (28, 416, 264), (40, 2048, 64), (52, 160, 520),
                                  (56, 2080, 72)], ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}")
def test_mx_fp4_gemm_few_rows_kernel(d, cabi, size):
    """the kernel for problems of at most 64 rows, forced for every N (the last size takes it by default
    too): every count of 16-row tiles, ragged M and N, K with a partly filled last 128-element step"""
    cabi.set_tuning("gemm.variant", 9)
    try:
        out = _check(d, *size, 2300 + size[0], "randn")
    finally:
        cabi.set_tuning("gemm.variant", 0)
    if size[2] >= 4096:
        assert torch.equal(_check(d, *size, 2300 + size[0], "randn"), out)


@pytest.mark.parametrize("splits", [0, 2, 3, 4, 16])
@pytest.mark.parametrize("size", [(16, 2048, 256), (133, 1408, 264), (40, 16512, 136), (24, 8288, 136)], ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}")
def test_mx_fp4_gemm_split_k(d, cabi, splits, size):
    """K shared between workgroups, including a K whose last 256-element step is half filled
    (1408 = 5.5 steps, 16512 = 64.5, which the library splits by itself): the half step belongs to the last split only."""
    cabi.set_tuning("gemm.split_k", splits)
    try:
        out = _check(d, *size, 1300 + size[0], "randn")
        for _ in range(3):
            assert torch.equal(_check(d, *size, 1300 + size[0], "randn"), out)
    finally:
        cabi.set_tuning("gemm.split_k", 0)


def test_mx_fp4_gemm_leftover_tiles_as_quadrants(d, cabi):
    """272 tiles of 256 x 256: one round on the big kernel, 16 tiles as 128 x 128 quadrants or as 256 x 128 halves; the same
    bits as the big kernel alone (with a half-filled last K-step: 384 = 1.5 steps)"""
    size = (4352, 384, 4096)
    outs = []
    for tail in (2, 0, 3):
        cabi.set_tuning("gemm.tail_quads", tail)
        try:
            outs.append(_check(d, *size, 1500, "randn"))
        finally:
            cabi.set_tuning("gemm.tail_quads", 1)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[2], outs[1])


def test_mx_fp4_gemm_bit_exact_when_sums_fit_fp32(d):
    """sparse operands and a narrow scale range: every product and every partial sum is a multiple
    of 2^-6 below 2^12, exact in fp32 in any order, so the result must equal the C oracle's float64
    reference rounded once to bf16, bit for bit, for full and half-filled last steps"""
    g = util.gen(91)
    for (M, K, N) in ((160, 384, 136), (130, 512, 264)):
        a = torch.randint(0, 16, (M, K), generator=g, dtype=torch.uint8) * (torch.rand(M, K, generator=g) < 0.03)
        b = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8) * (torch.rand(N, K, generator=g) < 0.5)
        ap = (a[:, 0::2] | (a[:, 1::2] << 4)).to(torch.uint8)
        bp = (b[:, 0::2] | (b[:, 1::2] << 4)).to(torch.uint8)
        sa = torch.randint(125, 130, (M, K // 32), generator=g, dtype=torch.uint8)
        sb = torch.randint(125, 130, (N, K // 32), generator=g, dtype=torch.uint8)
        out = _run(d, ap, sa, bp, sb)
        ref = co.mx_fp4_gemm_ref(ap, bp, co.to_blocked(sa), co.to_blocked(sb))
        assert torch.equal(out.cpu(), ref.bfloat16())


@pytest.mark.parametrize("tiles", [1, 2])
def test_mx_fp4_gemm_few_rows_kernel_bit_exact_when_sums_fit_fp32(d, cabi, tiles):
    """the kernel for few rows on the operands of the test above (exact in fp32 in any order): bit for bit
    the C oracle's reference, for one and two 16-column tiles per wave, every count of 16-row tiles and a K
    with a partly filled last 128-element step"""
    g = util.gen(92)
    cabi.set_tuning("gemm.variant", 9)
    cabi.set_tuning("gemm.few_rows_tiles", tiles)
    try:
        for (M, K, N) in ((16, 384, 136), (33, 480, 264), (64, 1312, 48), (50, 512, 40)):
            a = torch.randint(0, 16, (M, K), generator=g, dtype=torch.uint8) * (torch.rand(M, K, generator=g) < 0.03)
            b = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8) * (torch.rand(N, K, generator=g) < 0.5)
            ap = (a[:, 0::2] | (a[:, 1::2] << 4)).to(torch.uint8)
            bp = (b[:, 0::2] | (b[:, 1::2] << 4)).to(torch.uint8)
            sa = torch.randint(125, 130, (M, K // 32), generator=g, dtype=torch.uint8)
            sb = torch.randint(125, 130, (N, K // 32), generator=g, dtype=torch.uint8)
            out = _run(d, ap, sa, bp, sb)
            ref = co.mx_fp4_gemm_ref(ap, bp, co.to_blocked(sa), co.to_blocked(sb))
            assert torch.equal(out.cpu(), ref.bfloat16()), (M, K, N)
    finally:
        cabi.set_tuning("gemm.variant", 0)
        cabi.set_tuning("gemm.few_rows_tiles", 0)


def test_mx_fp4_gemm_scales_per_row_and_kblock(d):
    M, K, N = 256, 640, 256
    a, sa, b, sb = _operands(M, K, N, 93, "randn")
    base = _run(d, a, sa, b, sb).float()
    sa2 = sa.clone()
    sa2[77, :] += 3
    out = _run(d, a, sa2, b, sb).float()
    assert torch.equal(out[77], base[77] * 8)
    assert torch.equal(out[:77], base[:77]) and torch.equal(out[78:], base[78:])
    for kb in (2, 5, 17, 19):  # K-blocks in the first and second half of a step, and in the half-filled last step
        b2 = torch.zeros_like(b)
        b2[:, kb * 16:(kb + 1) * 16] = b[:, kb * 16:(kb + 1) * 16]
        out = _run(d, a, sa, b2, sb).cpu().double()
        da = eager.mx_fp4_dequant(a, sa)[:, kb * 32:(kb + 1) * 32]
        db = eager.mx_fp4_dequant(b, sb)[:, kb * 32:(kb + 1) * 32]
        ref, bound = da @ db.T, da.abs() @ db.abs().T
        assert ((out - ref).abs() <= bound * 2**-8).all()


def test_mx_fp4_gemm_strided_a_and_float4_storage(d):
    M, K, N = 192, 512, 136
    a, sa, b, sb = _operands(M, K, N, 95, "randn")
    wide = torch.zeros((M, K // 2 + 64), dtype=torch.uint8, device="cuda")
    wide[:, :K // 2] = a.cuda()
    av = wide[:, :K // 2]  # row stride K/2 + 64 bytes
    want = _run(d, a, sa, b, sb)
    got = d.mx_fp4_bf16(av, b.cuda().t(), d.to_blocked(sa.cuda()), d.to_blocked(sb.cuda()))
    assert torch.equal(got, want)
    if hasattr(torch, "float4_e2m1fn_x2"):
        got = d.mx_fp4_bf16(a.cuda().view(torch.float4_e2m1fn_x2), b.cuda().view(torch.float4_e2m1fn_x2).t(),
                            d.to_blocked(sa.cuda()), d.to_blocked(sb.cuda()))
        assert torch.equal(got, want)


def test_mx_fp4_gemm_argument_errors(d):
    a, sa, b, sb = _operands(128, 256, 128, 97)
    A, B, SA, SB = a.cuda(), b.cuda(), d.to_blocked(sa.cuda()), d.to_blocked(sb.cuda())
    with pytest.raises(RuntimeError):
        d.mx_fp4_bf16(A, B, SA, SB)  # b not K-contiguous
    with pytest.raises(RuntimeError):
        d.mx_fp4_bf16(A, B.t(), SA[:-1], SB)  # scale length for K = 2 * a.size(1)
    with pytest.raises(RuntimeError):
        d.mx_fp4_bf16(A[:, :88], B[:, :88].t(), SA, SB)  # K = 176 is not a whole number of MX blocks
    with pytest.raises(RuntimeError):
        d.mx_fp4_bf16(A.view(torch.float8_e4m3fn), B.t(), SA, SB)


def test_mx_fp4_gemm_compile(d):
    a, sa, b, sb = _operands(256, 512, 384, 98)
    args = (a.cuda(), b.cuda().t(), d.to_blocked(sa.cuda()), d.to_blocked(sb.cuda()))
    torch._dynamo.reset()
    fn = torch.compile(d.mx_fp4_bf16, fullgraph=True, backend="aot_eager")
    assert torch.equal(fn(*args), d.mx_fp4_bf16(*args))


def test_mx_fp4_gemm_full_size(d):
    """8192^3; checked on sampled rows against the float64 dequantized product"""
    M = N = K = 8192
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8, device="cuda")
    b = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8, device="cuda")
    sa = torch.randint(120, 134, (M, K // 32), generator=g, dtype=torch.uint8, device="cuda")
    sb = torch.randint(120, 134, (N, K // 32), generator=g, dtype=torch.uint8, device="cuda")
    out = d.mx_fp4_bf16(a, b.t(), d.to_blocked(sa), d.to_blocked(sb))
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 4095, 4096, 8000, 8191])
    da = eager.mx_fp4_dequant(a[rows.cuda()].cpu(), sa[rows.cuda()].cpu())
    cols = torch.arange(0, N, 61)
    db = eager.mx_fp4_dequant(b[cols.cuda()].cpu(), sb[cols.cuda()].cpu())
    ref, bound = da @ db.T, da.abs() @ db.abs().T
    got = out[rows.cuda()][:, cols.cuda()].cpu().double()
    assert ((got - ref).abs() <= bound * 2**-8).all()


# --------------------------------------------------------------------------- MXFP4 cast
def _check_fp4_cast(d, x):
    data, scale = d.mx_fp4_quantize(x.cuda())
    rd, rs = co.mx_fp4_quantize(x)
    M, N = x.shape
    assert data.dtype == torch.uint8 and data.shape == (M, N // 2) and scale.dtype == torch.float8_e8m0fnu
    assert torch.equal(util.codes(scale).view(M, N // 32), rs)
    assert torch.equal(data.cpu(), rd)
    bdata, bscale = d.mx_fp4_quantize(x.cuda(), True)
    assert torch.equal(bdata.cpu(), rd)
    assert torch.equal(util.codes(bscale), co.to_blocked(rs))
    return data, scale


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(128, 32), (1, 64), (77, 96), (256, 512), (384, 1024), (130, 544), (2048, 4096)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_mx_fp4_cast_against_oracle(d, in_dtype, shape):
    g = util.gen(shape[0] + shape[1])
    x = torch.randn(shape, generator=g) * torch.exp(2.0 * torch.randn(shape, generator=g))
    if in_dtype == torch.float16:
        x = x.clamp(-6.0e4, 6.0e4)
    _check_fp4_cast(d, x.to(in_dtype))


def _check_fp4_cast_cols(d, x):
    """blocks down the columns, payload transposed: the row-wise cast of x^T"""
    M, N = x.shape
    rd, rs = co.mx_fp4_quantize(x.t().contiguous())
    for blocked in (False, True):
        data, scale = d.mx_fp4_quantize(x.cuda(), blocked, 0)
        assert data.shape == (N, M // 2) and torch.equal(data.cpu(), rd)
        assert torch.equal(util.codes(scale), (co.to_blocked(rs) if blocked else rs).flatten())


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(32, 128), (64, 4), (96, 76), (256, 512), (1024, 384), (160, 1028), (4096, 2048), (4128, 4104)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_mx_fp4_cast_down_the_columns(d, in_dtype, shape):
    g = util.gen(shape[0] * 3 + shape[1])
    x = torch.randn(shape, generator=g) * torch.exp(2.0 * torch.randn(shape, generator=g))
    if in_dtype == torch.float16:
        x = x.clamp(-6.0e4, 6.0e4)
    _check_fp4_cast_cols(d, x.to(in_dtype))


def test_mx_fp4_cast_down_the_columns_both_kernels(d, cabi):
    """large 16-bit inputs take the one-read kernel without its row-wise half on a grid of walking
    workgroups, everything else the kernel with 32-row lanes: the same bytes (8192 x 8192 and a ragged shape)"""
    for shape in ((8192, 8192), (4128, 4360)):
        x = util.normal(shape, 51, torch.bfloat16).cuda()
        got = {}
        for via in (1, 0):
            cabi.set_tuning("mx.colt_via_dual", via)
            try:
                got[via] = d.mx_fp4_quantize(x, True, 0)
            finally:
                cabi.set_tuning("mx.colt_via_dual", 1)
        assert torch.equal(got[0][0], got[1][0]) and torch.equal(util.codes(got[0][1]), util.codes(got[1][1]))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_mx_fp4_cast_special_blocks(d, in_dtype):
    x = util.normal((128, 512), 41, in_dtype)
    tiny = torch.finfo(in_dtype).tiny
    x[0, :32] = 0.0
    x[1, 32:64] = tiny / 4               # subnormal maximum
    x[2, 5] = float("inf")
    x[3, 40] = float("-inf")
    x[4, 70] = float("nan")
    x[5, 100] = float("nan")
    x[5, 101] = float("inf")
    x[6, :32] = torch.finfo(in_dtype).max
    x[7, :32] = tiny
    x[8, :32] = (torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4)).to(in_dtype)   # the grid's ties
    x[9, :32] = -x[8, :32]
    _check_fp4_cast(d, x)
    _check_fp4_cast_cols(d, x.t().contiguous())


def test_mx_fp4_cast_every_bf16_pattern(d):
    """all 65536 bf16 patterns as block members, under block maxima that put them below, inside and
    above the e2m1 range (NaN patterns only in the NaN rows)"""
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = pats.clone()
    finite[torch.isnan(pats) | torch.isinf(pats)] = 1.0
    rows = []
    for top in (2.0 ** -120, 2.0 ** -20, 0.5, 1.0, 6.0, 448.0, 2.0 ** 60, 3.0e38):
        body = finite.float().view(2048, 32).clone()
        body[:, 0] = top                      # the block maximum, unless a pattern is larger
        rows.append(body.view(64, 1024))
    rows.append(pats.float().view(64, 1024))  # with NaN and infinity patterns in place
    x = torch.cat(rows).to(torch.bfloat16)
    _check_fp4_cast(d, x)
    _check_fp4_cast_cols(d, x.t().contiguous())


def test_mx_fp4_cast_feeds_the_gemm(d):
    """cast -> blocked scales -> mx_fp4_bf16 against the float64 product of the dequantized operands
    and, loosely, against the product of the inputs (e2m1 keeps 1-2 significant bits)"""
    M, K, N = 256, 1024, 384
    a, b = util.normal((M, K), 42), util.normal((N, K), 43)
    ad, sa = d.mx_fp4_quantize(a.cuda(), True)
    bd, sb = d.mx_fp4_quantize(b.cuda(), True)
    out = d.mx_fp4_bf16(ad, bd.t(), sa, sb)
    _, sa_plain = d.mx_fp4_quantize(a.cuda())
    _, sb_plain = d.mx_fp4_quantize(b.cuda())
    da = eager.mx_fp4_dequant(ad.cpu(), util.codes(sa_plain).view(M, K // 32))
    db = eager.mx_fp4_dequant(bd.cpu(), util.codes(sb_plain).view(N, K // 32))
    ref = da @ db.T
    bound = da.abs() @ db.abs().T
    assert ((out.cpu().double() - ref).abs() <= bound * 2**-8).all()
    assert eager.compute_error(a.double() @ b.double().T, out.cpu().double()).item() > 15  # fp4 operands: ~18 dB


def test_mx_fp4_cast_errors_and_compile(d, cabi):
    x = util.normal((64, 128), 44).cuda()
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize(x[:, :48])                  # not contiguous
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize(x[:, :48].contiguous())     # 48 % 32
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize(x.double())
    e_data, e_scale = d.mx_fp4_quantize(x[:0])
    assert e_data.shape == (0, 64) and e_scale.numel() == 0
    L = cabi.lib()
    data = torch.empty(64 * 64 + 8, dtype=torch.uint8, device="cuda")
    scale = torch.empty(64 * 4, dtype=torch.uint8, device="cuda")
    assert L.dt_mx_fp4_quantize(x.data_ptr(), cabi.BF16, 64, 128, 1, 0, data.data_ptr() + 2, scale.data_ptr(), None) == 4
    assert L.dt_mx_fp4_quantize(x.data_ptr(), cabi.BF16, 64, 128, 1, 2, data.data_ptr(), scale.data_ptr(), None) == 6
    assert L.dt_mx_fp4_quantize(x.data_ptr(), cabi.BF16, 64, 128, 3, 0, data.data_ptr(), scale.data_ptr(), None) == 6
    assert L.dt_mx_fp4_quantize(x.data_ptr(), 7, 64, 128, 1, 0, data.data_ptr(), scale.data_ptr(), None) == 1
    assert L.dt_mx_fp4_quantize(x.data_ptr(), cabi.BF16, 48, 128, 0, 0, data.data_ptr(), scale.data_ptr(), None) == 2  # 48 rows down the columns
    assert L.dt_mx_fp4_quantize(x.data_ptr(), cabi.BF16, 64, 128, 0, 0, data.data_ptr() + 4, scale.data_ptr(), None) == 4
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize(x[:48].contiguous(), False, 0)
    fn = torch.compile(lambda t: d.mx_fp4_quantize(t, True), fullgraph=True, backend="aot_eager")
    got, want = fn(x), d.mx_fp4_quantize(x, True)
    assert torch.equal(got[0], want[0]) and torch.equal(util.codes(got[1]), util.codes(want[1]))


# ------------------------------------------------- both MXFP4 operands from one read of x
def _check_fp4_dual(d, x):
    """mx_fp4_quantize_dual against the C oracle's cast of x (rows) and of x^T (columns, transposed)"""
    M, N = x.shape
    rd, rs = co.mx_fp4_quantize(x)
    cd, cs = co.mx_fp4_quantize(x.t().contiguous())
    for blocked in (False, True):
        dr, sr, dc, sc = d.mx_fp4_quantize_dual(x.cuda(), blocked)
        assert dr.dtype == torch.uint8 and dr.shape == (M, N // 2) and dc.shape == (N, M // 2)
        assert sr.dtype == torch.float8_e8m0fnu and sc.dtype == torch.float8_e8m0fnu
        assert torch.equal(dr.cpu(), rd) and torch.equal(dc.cpu(), cd)
        assert torch.equal(util.codes(sr), (co.to_blocked(rs) if blocked else rs).flatten())
        assert torch.equal(util.codes(sc), (co.to_blocked(cs) if blocked else cs).flatten())


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape", [(32, 32), (128, 256), (96, 160), (160, 96), (512, 1056), (1056, 512), (2048, 4096), (4128, 288)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_mx_fp4_dual_against_oracle(d, in_dtype, shape):
    """whole and ragged tiles (128 rows x 256 or 128 columns), wide-range data"""
    g = util.gen(shape[0] * 5 + shape[1])
    x = torch.randn(shape, generator=g) * torch.exp(2.0 * torch.randn(shape, generator=g))
    if in_dtype == torch.float16:
        x = x.clamp(-6.0e4, 6.0e4)
    _check_fp4_dual(d, x.to(in_dtype))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_mx_fp4_dual_special_blocks(d, in_dtype):
    x = util.normal((128, 512), 45, in_dtype)
    tiny = torch.finfo(in_dtype).tiny
    x[0, :32] = 0.0
    x[:32, 7] = 0.0
    x[1, 32:64] = tiny / 4
    x[2, 5] = float("inf")
    x[3, 40] = float("-inf")
    x[4, 70] = float("nan")
    x[5, 100] = float("nan")
    x[5, 101] = float("inf")
    x[6, :32] = torch.finfo(in_dtype).max
    x[64:96, 300] = torch.finfo(in_dtype).max
    x[7, :32] = tiny
    x[8, :32] = (torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4)).to(in_dtype)
    x[96:128, 9] = -x[8, :32]
    _check_fp4_dual(d, x)


def test_mx_fp4_dual_matches_the_single_casts_at_full_size(d):
    """8192 x 8192 bf16: the one-read kernel against the two single casts, both scale layouts"""
    x = util.normal((8192, 8192), 46, torch.bfloat16).cuda()
    for blocked in (False, True):
        dr, sr, dc, sc = d.mx_fp4_quantize_dual(x, blocked)
        wr, wsr = d.mx_fp4_quantize(x, blocked, 1)
        wc, wsc = d.mx_fp4_quantize(x, blocked, 0)
        assert torch.equal(dr, wr) and torch.equal(dc, wc)
        assert torch.equal(util.codes(sr), util.codes(wsr)) and torch.equal(util.codes(sc), util.codes(wsc))


def test_mx_fp4_dual_feeds_the_gemm_both_ways(d):
    """x [M, K] cast once: its row operand in x @ w^T and its transposed operand in x^T @ g"""
    M, K, N = 256, 512, 384
    x, w, g = util.normal((M, K), 47), util.normal((N, K), 48), util.normal((N, M), 49)
    xr, xrs, xt, xts = d.mx_fp4_quantize_dual(x.cuda(), True)
    wd, ws = d.mx_fp4_quantize(w.cuda(), True)
    gd, gs = d.mx_fp4_quantize(g.cuda(), True)
    fwd = d.mx_fp4_bf16(xr, wd.t(), xrs, ws)                    # [M, N] = x w^T
    wgrad = d.mx_fp4_bf16(xt, gd.t(), xts, gs)                  # [K, N] = x^T g^T
    assert eager.compute_error(x.double() @ w.double().T, fwd.cpu().double()).item() > 15
    assert eager.compute_error(x.double().T @ g.double().T, wgrad.cpu().double()).item() > 15


def test_mx_fp4_dual_errors_fallback_and_compile(d, cabi):
    x = util.normal((128, 256), 50).cuda()
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize_dual(x[:, :48].contiguous())   # 48 % 32
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize_dual(x[:48].contiguous())
    with pytest.raises(RuntimeError):
        d.mx_fp4_quantize_dual(x.t())                    # not contiguous
    e = d.mx_fp4_quantize_dual(x[:0])
    assert e[0].shape == (0, 128) and e[2].shape == (256, 0)
    want = d.mx_fp4_quantize_dual(x, True)
    cabi.set_tuning("mx.dual", 0)                        # the two single casts behind the same entry point
    try:
        two = d.mx_fp4_quantize_dual(x, True)
    finally:
        cabi.set_tuning("mx.dual", 1)
    for a, b in zip(want, two):
        assert torch.equal(util.codes(a), util.codes(b))
    L = cabi.lib()
    buf = torch.empty(4 * 128 * 256, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert L.dt_mx_fp4_quantize_dual(x.data_ptr(), cabi.BF16, 128, 48, 0, p, p, p, p, None) == 2
    assert L.dt_mx_fp4_quantize_dual(x.data_ptr(), cabi.BF16, 128, 256, 2, p, p, p, p, None) == 6
    assert L.dt_mx_fp4_quantize_dual(x.data_ptr(), 9, 128, 256, 0, p, p, p, p, None) == 1
    assert L.dt_mx_fp4_quantize_dual(x.data_ptr(), cabi.BF16, 128, 256, 0, p, p, None, p, None) == 3
    assert L.dt_mx_fp4_quantize_dual(None, cabi.BF16, 0, 256, 0, None, None, None, None, None) == 0
    fn = torch.compile(lambda t: d.mx_fp4_quantize_dual(t, True), fullgraph=True, backend="aot_eager")
    got = fn(x)
    for a, b in zip(got, want):
        assert torch.equal(util.codes(a), util.codes(b))
