"""GPU parity past the 32-bit marks: tensors of more than 2^32 elements (per-tensor and row-wise
ops, the MX casts) and GEMM operands / outputs of more than 4 GiB.

The inputs repeat a small seeded block, so the oracle runs on the block and every repetition on
the device is compared with it; single elements planted beyond element 2^32 break the period
where an index that wrapped would otherwise land on equal data.
"""
import pytest
import torch

from oracle import c_oracle as co
from oracle import eager
from tests import util

pytestmark = pytest.mark.gpu

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
TWO32 = 1 << 32


@pytest.fixture(scope="module")
def d(gpu_device):
    import driss_torch_amd

    free, _ = torch.cuda.mem_get_info()
    if free < 48 << 30:
        pytest.skip("needs 48 GiB of free device memory")
    return driss_torch_amd


def _periodic(base, reps):
    """1-D device tensor: ``base`` repeated ``reps`` times"""
    x = torch.empty(reps * base.numel(), dtype=base.dtype, device="cuda")
    x.view(reps, base.numel()).copy_(base.cuda().view(1, -1))
    return x


def _all_rows_equal(got_u8, expected_row_u8):
    return bool((got_u8.view(-1, expected_row_u8.numel()) == expected_row_u8.cuda().view(1, -1)).all())


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_per_tensor_ops_past_2_32_elements(d, in_dtype):
    period = (1 << 22) + 64
    reps = TWO32 // period + 3
    base = util.normal((period,), 2001, in_dtype)
    x = _periodic(base, reps)
    n = x.numel()
    assert n > TWO32
    x2 = x.view(reps, period)
    assert d.amax(x2).item() == co.amax(base).item()
    planted = TWO32 + 12345
    x[planted] = 77.0
    assert d.amax(x2).item() == 77.0
    x[n - 1] = -99.0
    assert d.amax(x2).item() == 99.0

    for fp8 in (E4, E5):
        out, amax, scale = d.dynamic_scaled_quant_ex(x2, fp8, 3)
        assert amax.item() == 99.0 and scale.item() == co.amax_to_scale(99.0, fp8)
        s = scale.item()
        codes = out.view(torch.uint8).view(-1)
        special = torch.tensor([[77.0, -99.0]], dtype=in_dtype)
        want = co.saturated_cast(special, s, fp8, 3).view(-1)
        assert codes[planted].item() == want[0].item() and codes[n - 1].item() == want[1].item()
        ref = co.saturated_cast(base.view(1, -1), s, fp8, 3).view(-1)
        # every whole period except the two that hold a planted value
        keep = torch.ones(reps, dtype=torch.bool)
        keep[planted // period] = False
        keep[reps - 1] = False
        rows = codes.view(reps, period)[keep.cuda()]
        assert _all_rows_equal(rows, ref)
        # and those two, away from the planted element
        for r, col in ((planted // period, planted % period), (reps - 1, period - 1)):
            row = codes.view(reps, period)[r].cpu()
            mask = torch.ones(period, dtype=torch.bool)
            mask[col] = False
            assert torch.equal(row[mask], ref[mask])
        got = d.saturated_cast_mode(x2, scale.reshape(1), fp8, 3).view(torch.uint8).view(-1)
        assert torch.equal(got, codes)
        del out, got, codes, rows
    e4, e5, amax, scales = d.dynamic_scaled_quant_pair(x2, 3)
    assert amax.item() == 99.0
    assert torch.equal(e4.view(torch.uint8), d.dynamic_scaled_quant_ex(x2, E4, 3)[0].view(torch.uint8))
    assert torch.equal(e5.view(torch.uint8), d.dynamic_scaled_quant_ex(x2, E5, 3)[0].view(torch.uint8))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_rowwise_past_2_32_elements(d, in_dtype):
    cols, base_rows = 4104, 1024
    reps = TWO32 // (cols * base_rows) + 2
    base = util.rows_log_uniform_sigma((base_rows, cols), 2002, in_dtype)
    x = _periodic(base.view(-1), reps).view(reps * base_rows, cols)
    assert x.numel() > TWO32
    last = x.shape[0] - 1
    x[last, cols - 1] = 3.0e5
    out, amax, scale = d.dynamic_scaled_quant_rowwise(x, E4)
    ref, ramax, rscale = co.dynamic_scaled_quant_rowwise(base, E4)
    codes = out.view(torch.uint8)
    assert _all_rows_equal(codes[:-base_rows].reshape(-1), ref.view(-1))
    assert torch.equal(codes[-base_rows:-1].cpu(), ref[:-1])
    assert _all_rows_equal(amax[:-1].view(torch.int32).view(-1)[: (reps - 1) * base_rows], ramax.view(torch.int32).view(-1))
    assert _all_rows_equal(scale[:-1].view(torch.int32).view(-1)[: (reps - 1) * base_rows], rscale.view(torch.int32).view(-1))
    lref, lamax, lscale = co.dynamic_scaled_quant_rowwise(x[last:].cpu(), E4)
    assert torch.equal(codes[last:].cpu(), lref) and amax[last].item() == lamax.item() and scale[last].item() == lscale.item()


def _tile2d(base, rep_r, rep_c):
    r, c = base.shape
    x = torch.empty((rep_r * r, rep_c * c), dtype=base.dtype, device="cuda")
    x.view(rep_r, r, rep_c, c).copy_(base.cuda().view(1, r, 1, c))
    return x


def _tiles_equal(got_u8, exp_u8, rep_r, rep_c):
    r, c = exp_u8.shape
    return bool((got_u8.view(rep_r, r, rep_c, c) == exp_u8.cuda().view(1, r, 1, c)).all())


def test_mx_casts_past_2_32_elements(d):
    # 65664 x 65792 = 4.32e9 elements; rows a multiple of 128 and columns of 512, so the tiled kernels run
    base_r, base_c, rep_r, rep_c = 864, 512, 76, 128 + 1
    base = util.student_t((base_r, base_c), 2003)
    x = _tile2d(base, rep_r, rep_c)
    R, C = x.shape
    assert R * C > TWO32 and R % 128 == 0 and C % 512 == 0
    rd, rs = co.mx_quantize(base, 1, False)
    cd, cs = co.mx_quantize(base, 0, True)   # [base_c, base_r], [base_c, base_r / 32]
    cd_in_place, cs_in_place = co.mx_quantize(base, 0, False)

    data, scale = d.mx_fp8_quantize(x)
    assert _tiles_equal(data.view(torch.uint8), rd, rep_r, rep_c)
    assert _tiles_equal(scale.view(torch.uint8).view(R, C // 32), rs, rep_r, rep_c)
    full_rs = scale.view(torch.uint8).view(R, C // 32).cpu()
    data_b, scale_b = d.mx_fp8_quantize_blocked(x)
    assert torch.equal(data_b.view(torch.uint8), data.view(torch.uint8))
    assert torch.equal(scale_b.view(torch.uint8).cpu(), co.to_blocked(full_rs))
    del data_b, scale_b

    data_c, scale_c = d.mx_fp8_quantize(x, axis=0)
    assert _tiles_equal(data_c.view(torch.uint8), cd_in_place, rep_r, rep_c)
    assert _tiles_equal(scale_c.view(torch.uint8).view(R // 32, C), cs_in_place, rep_r, rep_c)
    del data_c, scale_c

    data_t, scale_t = d.mx_fp8_quantize(x, axis=0, transpose=True)
    assert _tiles_equal(data_t.view(torch.uint8), cd, rep_c, rep_r)
    assert _tiles_equal(scale_t.view(torch.uint8).view(C, R // 32), cs, rep_c, rep_r)
    full_cs = scale_t.view(torch.uint8).view(C, R // 32).cpu()

    for blocked in (False, True):
        o = d.mx_fp8_quantize_dual(x, E4, blocked)
        assert torch.equal(o[0].view(torch.uint8), data.view(torch.uint8))
        assert torch.equal(o[2].view(torch.uint8), data_t.view(torch.uint8))
        if blocked:
            assert torch.equal(o[1].view(torch.uint8).cpu(), co.to_blocked(full_rs))
            assert torch.equal(o[3].view(torch.uint8).cpu(), co.to_blocked(full_cs))
        else:
            assert torch.equal(o[1].view(torch.uint8), scale.view(torch.uint8))
            assert torch.equal(o[3].view(torch.uint8), scale_t.view(torch.uint8))
        del o

    # the MXFP4 cast of the same tensor (packed pairs: column period base_c / 2)
    fd, fs = co.mx_fp4_quantize(base)
    d4, s4 = d.mx_fp4_quantize(x)
    assert _tiles_equal(d4, fd, rep_r, rep_c)
    assert _tiles_equal(s4.view(torch.uint8).view(R, C // 32), fs, rep_r, rep_c)
    d4b, s4b = d.mx_fp4_quantize(x, True)
    assert torch.equal(d4b, d4)
    assert torch.equal(s4b.view(torch.uint8).cpu(), co.to_blocked(s4.view(torch.uint8).view(R, C // 32).cpu()))
    del d4, s4, d4b, s4b

    # a block past element 2^32 that differs from its period, in both directions
    r0, c0 = R - 32, C - 32
    x[r0 + 5, c0 + 7] = 1.0e4
    patch = x[r0:, c0:].cpu()
    data, scale = d.mx_fp8_quantize(x)
    pd, ps = co.mx_quantize(patch, 1, False)
    assert torch.equal(data.view(torch.uint8)[r0:, c0:].cpu(), pd)
    assert torch.equal(scale.view(torch.uint8).view(R, C // 32)[r0:, -1:].cpu(), ps)
    o = d.mx_fp8_quantize_dual(x, E4, False)
    pd, ps = co.mx_quantize(patch, 0, True)
    assert torch.equal(o[0].view(torch.uint8), data.view(torch.uint8))
    assert torch.equal(o[2].view(torch.uint8)[c0:, r0:].cpu(), pd)
    assert torch.equal(o[3].view(torch.uint8).view(C, R // 32)[c0:, -1:].cpu(), ps)


def _random_mx_operand(rows, K, seed):
    """device uint8 e4m3 codes [rows, K] without NaN, plain scale bytes [rows, K/32] in 120..134"""
    g = torch.Generator(device="cuda").manual_seed(seed)
    codes = torch.randint(0, 0x7F, (rows, K), dtype=torch.uint8, device="cuda", generator=g)
    codes |= torch.randint(0, 2, (rows, K), dtype=torch.uint8, device="cuda", generator=g) << 7
    scale = torch.randint(120, 135, (rows, K // 32), dtype=torch.uint8, device="cuda", generator=g)
    return codes, scale


def _check_rows(out, rows, a_codes, a_scale, b_codes, b_scale):
    idx = torch.tensor(rows)
    da = eager.mx_dequant(a_codes[idx.cuda()].cpu().view(E4), a_scale[idx.cuda()].cpu())
    db = eager.mx_dequant(b_codes.cpu().view(E4), b_scale.cpu())
    ref = da.double() @ db.double().T
    bound = da.abs().double() @ db.abs().double().T
    got = out[idx.cuda()].cpu().double()
    # bf16 store (2^-9 relative to the entry) plus fp32 accumulation, measured against sum |a||b|
    assert ((got - ref).abs() <= bound * 2**-8).all()
    assert eager.compute_error(ref, got).item() > 50


def test_mx_gemm_operand_larger_than_4_gib(d):
    M, K, N = 66048, 65664, 256
    assert M * K > TWO32
    a, sa = _random_mx_operand(M, K, 2004)
    b, sb = _random_mx_operand(N, K, 2005)
    sa_b = co.to_blocked(sa.cpu()).cuda().view(torch.float8_e8m0fnu)
    sb_b = co.to_blocked(sb.cpu()).cuda().view(torch.float8_e8m0fnu)
    wrap = TWO32 // K  # the row whose bytes straddle offset 2^32
    rows = [0, 255, 256, wrap - 1, wrap, wrap + 1, wrap + 300, M - 257, M - 1]
    out = d.mx_fp8_bf16(a.view(E4), b.view(E4).t(), sa_b, sb_b)
    _check_rows(out, rows, a, sa, b, sb)
    # and as the K-contiguous second operand
    out_t = d.mx_fp8_bf16(b.view(E4), a.view(E4).t(), sb_b, sa_b)
    assert torch.equal(out_t, out.t())


def test_mx_gemm_output_larger_than_4_gib(d):
    M = N = 46592
    K = 128
    assert M * N * 2 > TWO32
    a, sa = _random_mx_operand(M, K, 2006)
    b, sb = _random_mx_operand(N, K, 2007)
    sa_b = co.to_blocked(sa.cpu()).cuda().view(torch.float8_e8m0fnu)
    sb_b = co.to_blocked(sb.cpu()).cuda().view(torch.float8_e8m0fnu)
    out = d.mx_fp8_bf16(a.view(E4), b.view(E4).t(), sa_b, sb_b)
    _check_rows(out, [0, 1, 23000, 23048, 46080, M - 2, M - 1], a, sa, b, sb)
