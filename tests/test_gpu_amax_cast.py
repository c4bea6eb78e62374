"""GPU parity: amax, saturated_cast, dynamic_scaled_quant (per tensor, pair, rowwise) against
the CPU oracle, bit for bit, on the reference's own test grids (test/test_amax.py:10-12,
test/test_sat_cast.py:27-30, test/test_dynamic_quant.py:28-31) and on the benchmark configs."""
import pytest
import torch

from oracle import c_oracle as co
from oracle import eager
from tests import util

pytestmark = pytest.mark.gpu

FP8 = [torch.float8_e4m3fn, torch.float8_e5m2]
COLS = [7, 17, 127, 512, 3212, 4097]


@pytest.fixture(scope="module")
def d(gpu_device):
    import driss_torch_amd

    return driss_torch_amd


@pytest.fixture(scope="module")
def cabi(gpu_device):
    from driss_torch_amd import cabi as c

    return c


# ------------------------------------------------------------------------------- amax
@pytest.mark.parametrize("num_rows", [4, 64, 512, 4096])
@pytest.mark.parametrize("num_cols", COLS)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_amax_reference_grid(d, num_rows, num_cols, in_dtype):
    a = util.normal((num_rows, num_cols), 100 + num_rows + num_cols, in_dtype)
    got = d.amax(a.cuda())
    assert got.shape == (1,) and got.dtype == torch.float32
    assert torch.equal(got.cpu(), co.amax(a))
    assert torch.equal(got.cpu(), eager.eager_amax(a))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_amax_edges(d, cabi, in_dtype):
    # odd numel (the reference refuses it), single element, NaN, inf, negative extreme, misaligned view
    for shape in [(3, 7), (1, 1), (1, 9)]:
        a = util.normal(shape, 5, in_dtype)
        assert torch.equal(d.amax(a.cuda()).cpu(), co.amax(a))
    a = util.normal((64, 130), 6, in_dtype)
    a[17, 3] = -1e30
    assert d.amax(a.cuda()).item() == co.amax(a).item()
    a[5, 5] = float("inf")
    assert d.amax(a.cuda()).item() == float("inf")
    a[40, 100] = float("nan")
    assert torch.isnan(d.amax(a.cuda()))
    base = util.normal((1, 4099), 7, in_dtype).cuda()
    for off in (1, 2, 3, 5):
        v = base[:, off:]  # element-aligned but not 16-byte aligned
        got = cabi.amax(v)
        assert torch.equal(got.cpu(), co.amax(v.cpu().contiguous()))
    # the workspace re-arms itself: many calls in a row stay correct
    xs = [util.normal((257, 33), 50 + i, in_dtype) for i in range(6)]
    outs = [d.amax(x.cuda()) for x in xs]
    for x, o in zip(xs, outs):
        assert torch.equal(o.cpu(), co.amax(x))


def test_amax_argument_errors(d):
    with pytest.raises(RuntimeError):
        d.amax(torch.zeros(4, 4, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError):
        d.amax(torch.zeros(4, 4, 4, device="cuda"))
    with pytest.raises(RuntimeError):
        d.amax(torch.zeros(0, 4, device="cuda"))


def test_amax_full_size_config(d):
    a = util.normal_with_outliers((8192, 8192), 1002)
    got = d.amax(a.cuda())
    assert torch.equal(got.cpu(), co.amax(a))
    assert (a.float().abs() == got.item()).any()


# ---------------------------------------------------------------------- saturated_cast
@pytest.mark.parametrize("num_rows", [3, 64, 512, 4096])
@pytest.mark.parametrize("num_cols", COLS)
@pytest.mark.parametrize("fp8_dtype", FP8)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_saturated_cast_reference_grid(d, num_rows, num_cols, in_dtype, fp8_dtype):
    a = util.uniform((num_rows, num_cols), 200 + num_rows + num_cols, in_dtype)
    scale = eager.tensor_to_scale(a, fp8_dtype)  # 0-dim fp32, as torchao's tensor_to_scale returns
    ag, sg = a.cuda(), scale.cuda()
    # 0-dim device scale: eager keeps the product (and the scale) in bf16 -> mode 2
    got = d.saturated_cast(ag, sg, fp8_dtype)
    assert got.dtype == fp8_dtype and got.shape == a.shape
    assert torch.equal(util.codes(got), co.saturated_cast(a, scale.item(), fp8_dtype, co.ROUND_V2))
    # the same computation by eager PyTorch on the device (test/test_sat_cast.py:37-42)
    assert torch.equal(util.codes(got), util.codes(eager.eager_scaled_quant(ag, sg, fp8_dtype)))
    # rank-1 scale: eager promotes to fp32 -> mode 3
    got1 = d.saturated_cast(ag, sg.reshape(1), fp8_dtype)
    assert torch.equal(util.codes(got1), co.saturated_cast(a, scale.item(), fp8_dtype, co.ROUND_V3))
    assert torch.equal(util.codes(got1), util.codes(eager.eager_scaled_quant(ag, sg.reshape(1), fp8_dtype)))


@pytest.mark.parametrize("fp8_dtype", FP8)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", [1, 2, 3])
def test_saturated_cast_modes_signed_and_special(d, in_dtype, fp8_dtype, mode):
    a = util.normal((515, 259), 31 + mode, in_dtype, std=3.0)
    a[0, :8] = torch.tensor([float("inf"), -float("inf"), float("nan"), 0.0, -0.0, 1e-30, -1e-30, 1e30]).to(in_dtype)
    a[1, 0] = -float("nan")
    scale = eager.tensor_to_scale(a[2:], fp8_dtype)
    got = d.saturated_cast_mode(a.cuda(), scale.cuda(), fp8_dtype, mode)
    assert torch.equal(util.codes(got), co.saturated_cast(a, scale.item(), fp8_dtype, mode))
    # saturation: a scale 8x too large clamps instead of overflowing
    big = (scale * 8).cuda()
    got = d.saturated_cast_mode(a.cuda(), big, fp8_dtype, mode)
    assert torch.equal(util.codes(got), co.saturated_cast(a, (scale * 8).item(), fp8_dtype, mode))


@pytest.mark.parametrize("fp8_dtype", FP8)
def test_saturated_cast_every_bf16_pattern(d, fp8_dtype):
    """all 65536 bf16 bit patterns (NaNs of both signs, infinities, subnormals) under every rounding
    mode and scales that put the products below, inside and beyond the fp8 range"""
    a = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).reshape(256, 256)
    ag = a.cuda()
    for scale in (1.0, 0.37, 448.0 / 3.0, 57344.0, 1e-3, 2.0**-20, 3.0e38):
        sg = torch.tensor([scale], device="cuda")
        for mode in (1, 2, 3):
            got = d.saturated_cast_mode(ag, sg, fp8_dtype, mode)
            assert torch.equal(util.codes(got), co.saturated_cast(a, scale, fp8_dtype, mode)), (scale, mode)


@pytest.mark.parametrize("fp8_dtype", FP8)
def test_saturated_cast_fp32_bit_pattern_sweep(d, fp8_dtype):
    """2^20 fp32 patterns: every exponent with random mantissas, plus the neighbourhood of every fp8
    rounding boundary (midpoints between representable values, +- 1 ulp)"""
    g = util.gen(9)
    bits = torch.randint(0, 2**31 - 1, (1 << 20,), generator=g, dtype=torch.int64)
    bits = bits | (torch.randint(0, 2, (1 << 20,), generator=g, dtype=torch.int64) << 31)
    x = bits.to(torch.uint32).view(torch.float32)
    codes = torch.arange(256, dtype=torch.uint8).view(fp8_dtype).float()
    vals = codes[torch.isfinite(codes)].unique()
    mids = ((vals[:-1].double() + vals[1:].double()) / 2).float()
    near = torch.cat([mids, torch.nextafter(mids, torch.tensor(float("inf"))), torch.nextafter(mids, torch.tensor(-float("inf"))), vals])
    x = torch.cat([x, near, near * 0.5, near * 3.0])
    x = x[: x.numel() // 4 * 4].reshape(-1, 4).contiguous()
    for scale in (1.0, 2.0, 1.0 / 3.0):
        got = d.saturated_cast_mode(x.cuda(), torch.tensor([scale], device="cuda"), fp8_dtype, 3)
        assert torch.equal(util.codes(got), co.saturated_cast(x, scale, fp8_dtype, co.ROUND_V3)), scale


def test_saturated_cast_reference_edge_vector(d):
    """test/test_sat_cast.py:66-83: 0.3223 * 57344 -> e5m2 is 20480 with single rounding; the
    rank-1 scale of that test selects it, a 0-dim scale reproduces eager's 16384."""
    a = torch.tensor([[0.3223], [0.3223]], dtype=torch.bfloat16, device="cuda")
    s1 = torch.tensor([57344.0], device="cuda")
    assert d.saturated_cast(a, s1, torch.float8_e5m2).float().unique().item() == 20480.0
    assert d.saturated_cast(a, s1.reshape(()), torch.float8_e5m2).float().unique().item() == 16384.0
    assert torch.equal(util.codes(d.saturated_cast(a, s1, torch.float8_e5m2)),
                       util.codes(eager.eager_scaled_quant(a, s1, torch.float8_e5m2)))


def test_saturated_cast_layouts_and_errors(d):
    a = util.normal((96, 40), 77)
    scale = eager.tensor_to_scale(a, torch.float8_e4m3fn)
    ag, sg = a.cuda(), scale.cuda()
    ref = co.saturated_cast(a, scale.item(), torch.float8_e4m3fn, co.ROUND_V2)
    # column-major input: output keeps the strides (src/saturated_cast.cu:243-249)
    at = ag.t().contiguous().t()
    got = d.saturated_cast(at, sg, torch.float8_e4m3fn)
    assert got.stride() == at.stride() and torch.equal(util.codes(got.contiguous()), ref)
    # a strided view is made contiguous first
    wide = torch.zeros(96, 80, dtype=torch.bfloat16, device="cuda")
    wide[:, ::2] = ag
    got = d.saturated_cast(wide[:, ::2], sg, torch.float8_e4m3fn)
    assert torch.equal(util.codes(got), ref)
    # empty input -> empty output
    assert d.saturated_cast(ag[:0], sg, torch.float8_e4m3fn).shape == (0, 40)
    with pytest.raises(RuntimeError):
        d.saturated_cast(ag, sg, torch.bfloat16)
    with pytest.raises(RuntimeError):
        d.saturated_cast(ag.half(), sg, torch.float8_e5m2)
    with pytest.raises(RuntimeError):
        d.saturated_cast(ag, sg.double(), torch.float8_e5m2)
    with pytest.raises(RuntimeError):
        d.saturated_cast(ag, torch.ones(2, device="cuda"), torch.float8_e5m2)
    with pytest.raises(RuntimeError):
        d.saturated_cast(ag[0], sg, torch.float8_e5m2)


def test_saturated_cast_unaligned_pointers(cabi):
    base = util.normal((1, 5000), 78).cuda()
    scale = torch.tensor(37.5, device="cuda")
    outbuf = torch.empty(6000, dtype=torch.float8_e4m3fn, device="cuda")
    for xo, oo in ((1, 0), (0, 3), (3, 5), (8, 8)):
        x = base[0, xo:xo + 4001]
        out = outbuf[oo:oo + 4001]
        cabi.saturated_cast(x, scale, torch.float8_e4m3fn, cabi.ROUND_F32, out=out)
        assert torch.equal(util.codes(out), co.saturated_cast(x.cpu().contiguous(), 37.5, torch.float8_e4m3fn, co.ROUND_V3))


@pytest.mark.parametrize("fp8_dtype", FP8)
def test_saturated_cast_compile(d, fp8_dtype):
    """test/test_sat_cast.py:45-62 with a backend that needs no code generator"""
    torch._dynamo.reset()
    a = util.uniform((64, 512), 90).cuda()
    scale = eager.tensor_to_scale(a, fp8_dtype)
    fn = torch.compile(d.saturated_cast, fullgraph=True, backend="aot_eager")
    assert torch.equal(util.codes(fn(a, scale, fp8_dtype)), util.codes(d.saturated_cast(a, scale, fp8_dtype)))


def test_saturated_cast_config1_all_modes(d):
    a = util.normal((4096, 4096), 1001)
    scale = eager.tensor_to_scale(a, torch.float8_e4m3fn)
    for mode in (1, 2, 3):
        got = d.saturated_cast_mode(a.cuda(), scale.cuda(), torch.float8_e4m3fn, mode)
        assert torch.equal(util.codes(got), co.saturated_cast(a, scale.item(), torch.float8_e4m3fn, mode))
    # mode 1 is literally eager on the CPU with the 0-dim scale
    got = d.saturated_cast_mode(a.cuda(), scale.cuda(), torch.float8_e4m3fn, 1)
    assert torch.equal(util.codes(got), util.codes(eager.eager_scaled_quant(a, scale, torch.float8_e4m3fn)))


# ---------------------------------------------------------------- dynamic_scaled_quant
@pytest.mark.parametrize("num_rows", [3, 64, 512, 4096])
@pytest.mark.parametrize("num_cols", COLS)
@pytest.mark.parametrize("fp8_dtype", FP8)
def test_dynamic_quant_reference_grid_fp32(d, num_rows, num_cols, fp8_dtype):
    a = util.uniform((num_rows, num_cols), 300 + num_rows + num_cols, torch.float32)
    got = d.dynamic_scaled_quant(a.cuda(), fp8_dtype)
    ref, ramax, rscale = co.dynamic_scaled_quant(a, fp8_dtype, co.ROUND_V3)
    assert torch.equal(util.codes(got), ref)
    eq, _, _ = eager.dynamic_scaled_quant(a, fp8_dtype)
    assert torch.equal(util.codes(got), util.codes(eq))


@pytest.mark.parametrize("fp8_dtype", FP8)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_dynamic_quant_outputs_and_modes(d, in_dtype, fp8_dtype):
    a = util.normal_with_outliers((1000, 517), 41, in_dtype)
    ag = a.cuda()
    for mode in (1, 2, 3):
        out, amax, scale = d.dynamic_scaled_quant_ex(ag, fp8_dtype, mode)
        ref, ramax, rscale = co.dynamic_scaled_quant(a, fp8_dtype, mode)
        assert torch.equal(util.codes(out), ref)
        assert amax.item() == ramax.item() and scale.item() == rscale.item()
    # default mode == eager on the device with tensor_to_scale's 0-dim scale
    out = d.dynamic_scaled_quant(ag, fp8_dtype)
    eq = eager.eager_scaled_quant(ag, eager.tensor_to_scale(ag, fp8_dtype), fp8_dtype)
    assert torch.equal(util.codes(out), util.codes(eq))


def test_dynamic_quant_zero_and_nan_tensor(d):
    z = torch.zeros(64, 64, device="cuda")
    out, amax, scale = d.dynamic_scaled_quant_ex(z, torch.float8_e4m3fn, 0)
    assert amax.item() == 0.0 and scale.item() == co.amax_to_scale(0.0, torch.float8_e4m3fn)
    assert (util.codes(out) == 0).all()
    z[3, 3] = float("nan")
    out, amax, scale = d.dynamic_scaled_quant_ex(z, torch.float8_e4m3fn, 0)
    assert torch.isnan(amax) and torch.isnan(scale)
    ref, _, _ = co.dynamic_scaled_quant(z.cpu(), torch.float8_e4m3fn, co.ROUND_V3)
    assert torch.equal(util.codes(out), ref)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_dynamic_quant_pair(d, in_dtype):
    a = util.normal_with_outliers((777, 1029), 43, in_dtype)
    o4, o5, amax, scales = d.dynamic_scaled_quant_pair(a.cuda(), 0)
    r4, ramax, rs4 = co.dynamic_scaled_quant(a, torch.float8_e4m3fn, co.ROUND_V2)
    r5, _, rs5 = co.dynamic_scaled_quant(a, torch.float8_e5m2, co.ROUND_V2)
    assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(o5), r5)
    assert amax.item() == ramax.item() and scales.cpu().tolist() == [rs4.item(), rs5.item()]


def test_dynamic_quant_config2_full_size(d):
    a = util.normal_with_outliers((8192, 8192), 1002)
    o4, o5, amax, scales = d.dynamic_scaled_quant_pair(a.cuda(), 0)
    r4, ramax, rs4 = co.dynamic_scaled_quant(a, torch.float8_e4m3fn, co.ROUND_V2)
    r5, _, rs5 = co.dynamic_scaled_quant(a, torch.float8_e5m2, co.ROUND_V2)
    assert amax.item() == ramax.item() and scales.cpu().tolist() == [rs4.item(), rs5.item()]
    assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(o5), r5)
    single = d.dynamic_scaled_quant(a.cuda(), torch.float8_e4m3fn)
    assert torch.equal(util.codes(single), r4)


@pytest.mark.parametrize("fp8_dtype", FP8)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(3, 7), (64, 8), (33, 512), (100, 4096), (5, 4097), (9, 8200), (4, 20000), (2, 131072)])
def test_rowwise_shapes(d, in_dtype, fp8_dtype, shape):
    a = util.rows_log_uniform_sigma(shape, 51 + shape[1], in_dtype)
    if shape[0] > 2:
        a[1] = 0  # an all-zero row: amax 0 -> scale fmax/1e-12, payload zeros
    out, amax, scale = d.dynamic_scaled_quant_rowwise(a.cuda(), fp8_dtype)
    ref, ramax, rscale = co.dynamic_scaled_quant_rowwise(a, fp8_dtype)
    assert amax.shape == (shape[0], 1) and scale.shape == (shape[0], 1)
    assert torch.equal(amax.cpu(), ramax)
    assert torch.equal(scale.cpu().view(torch.int32), rscale.view(torch.int32))
    assert torch.equal(util.codes(out), ref)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("extra", [0, 3])
@pytest.mark.parametrize("vecs", [1, 40, 257, 300, 512, 513, 1024, 1030, 2048, 2500, 4096, 4100, 8192, 8193, 9000, 16384, 16385])
def test_rowwise_long_rows(d, in_dtype, vecs, extra):
    """rows of 257 ... 16384 sixteen-byte vectors get a workgroup each and stay in its registers (1 to 64
    vectors per lane, ragged last pass); longer ones are read twice.  Row maxima in the first and in the
    last vector of a row, an all-zero row, NaN in one row"""
    # extra: a few elements past the last whole vector, which also leaves every row but the first misaligned
    # (such rows take the same kernel with element-aligned vector accesses)
    cols = vecs * (8 if in_dtype == torch.bfloat16 else 4) + extra
    a = util.rows_log_uniform_sigma((6, cols), 52 + vecs, in_dtype)
    a[1] = 0
    a[2, 0] = 3.0e4
    a[3, cols - 1] = -3.0e4
    a[4, cols // 2] = float("nan")
    # the tensor itself one element off a 16-byte boundary as well
    buf = torch.empty(a.numel() + 1, dtype=in_dtype, device="cuda")
    buf[1:] = a.cuda().flatten()
    shifted = buf[1:].view(a.shape)
    for fp8_dtype in FP8:
        ref, ramax, rscale = co.dynamic_scaled_quant_rowwise(a, fp8_dtype)
        for src in (a.cuda(), shifted):
            out, amax, scale = d.dynamic_scaled_quant_rowwise(src, fp8_dtype)
            assert torch.equal(amax.cpu().view(torch.int32), ramax.view(torch.int32))
            assert torch.equal(scale.cpu().view(torch.int32), rscale.view(torch.int32))
            assert torch.equal(util.codes(out), ref)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_rowwise_config3_full_size(d, in_dtype):
    a = util.rows_log_uniform_sigma((16384, 4096), 1003, in_dtype)
    ag = a.cuda()
    out, amax, scale = d.dynamic_scaled_quant_rowwise(ag, torch.float8_e4m3fn)
    ref, ramax, rscale = co.dynamic_scaled_quant_rowwise(a, torch.float8_e4m3fn)
    assert torch.equal(amax.cpu(), ramax) and torch.equal(scale.cpu().view(torch.int32), rscale.view(torch.int32))
    assert torch.equal(util.codes(out), ref)
    # and the eager formulation on the device
    eq, eamax, escale = eager.dynamic_scaled_quant_rowwise(ag, torch.float8_e4m3fn)
    assert torch.equal(util.codes(out), util.codes(eq)) and torch.equal(scale, escale)
