"""Pins the MX part of the oracle: exponent formula against exact ceil(log2) arithmetic,
C oracle against the eager restatement, the blocked layout against its view/permute
definition, the GEMM reference against float64 matmul and brute force."""
import ctypes as C
import json
import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import eager
from tests import util

GOLD = Path(__file__).parent / "golden"


def _student_t(shape, seed, df=3.0):
    g = torch.Generator().manual_seed(seed)
    n = torch.randn(shape, generator=g)
    chi = sum(torch.randn(shape, generator=g) ** 2 for _ in range(int(df)))
    return n / torch.sqrt(chi / df)


def test_mx_exponent_matches_exact_ceil_log2():
    lib = co.lib()
    g = torch.Generator().manual_seed(1)
    vals = torch.cat([torch.rand(5000, generator=g) * 1000, torch.linspace(-30, 30, 61).exp2(), torch.tensor([16.125, 0.999, 448.0])]).float()
    for v in vals.tolist():
        # exact: frexp gives v = m * 2^e with m in [0.5, 1): ceil(log2 v) = e-1 if m == 0.5 else e
        m, e = math.frexp(v)
        exact = e - 1 if m == 0.5 else e
        assert lib.dto_mx_ceil_log2(C.c_float(v)) == exact
    assert lib.dto_mx_ceil_log2(C.c_float(0.0)) == -128  # src/mx_cast.cu:59
    assert lib.dto_mx_ceil_log2(C.c_float(1e-40)) == -126  # subnormal, src/mx_cast.cu:59
    ev = eager.mx_ceil_exponent(vals)
    assert ev.tolist() == [lib.dto_mx_ceil_log2(C.c_float(v)) for v in vals.tolist()]


def test_mx_golden_scale_bytes():
    kat = json.loads((GOLD / "mx_kat.json").read_text())
    for row in kat["scale_byte"]:
        v = np.array([int(row["max_abs_bits"], 16)], dtype=np.uint32).view(np.float32)[0]
        x = torch.zeros(1, 32, dtype=torch.float32)
        x[0, 7] = -float(v)
        x[0, 8] = float(v) / 3
        data, scale = co.mx_quantize(x)
        assert int(scale[0, 0]) == row["e4m3_scale_byte"], row
        # dequantized max element is within one e4m3 ulp (2^-3 relative) of the input
        deq = co.mx_dequant(data, scale)
        if v > 0:
            assert abs(deq[0, 7].item() + v) <= v * 2**-3


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_mx_c_oracle_vs_eager(in_dtype, out_dtype):
    a = _student_t((64, 256), 21).to(in_dtype)
    a[3, 32:64] = 0  # all-zero block -> byte 0, zero payload
    a[5, 70] = 3e4 if in_dtype != torch.float16 else 6e4
    data, scale = co.mx_quantize(a, out_dtype=out_dtype)
    rs, rd = eager.to_mx(a, out_dtype)
    assert torch.equal(scale, rs)
    assert torch.equal(data, rd.view(torch.uint8))
    assert scale[3, 1] == 0 and (data[3, 32:64] == 0).all()


def test_mx_block_properties():
    """per block: the scaled max lies in (2^7, 2^8], so after rounding to e4m3 the payload max
    magnitude lies in [2^7, 2^8]; dequantization error <= 2^-4 * blockmax (e4m3 has 3 mantissa bits, scaled
    max <= 256 -> quantum 32 at the top binade) -- catches an off-by-one in the exponent."""
    a = _student_t((128, 512), 22).to(torch.bfloat16)
    data, scale = co.mx_quantize(a)
    deq = co.mx_dequant(data, scale)
    x = a.float().reshape(128, 16, 32)
    bm = x.abs().amax(-1)
    pm = data.view(torch.float8_e4m3fn).float().reshape(128, 16, 32).abs().amax(-1)
    assert ((pm >= 128) & (pm <= 256)).all()
    err = (deq.reshape(128, 16, 32) - x).abs().amax(-1)
    assert (err <= bm * 2**-4).all()


@pytest.mark.parametrize("transpose", [False, True])
def test_mx_axis0_is_axis1_of_transpose(transpose):
    a = _student_t((96, 64), 23).to(torch.bfloat16)
    d0, s0 = co.mx_quantize(a, axis=0, transpose=transpose)
    dT, sT = co.mx_quantize(a.T.contiguous(), axis=1)
    if transpose:
        assert torch.equal(d0, dT) and torch.equal(s0, sT)
    else:
        assert torch.equal(d0, dT.T) and torch.equal(s0, sT.T)
    d1t, s1t = co.mx_quantize(a, axis=1, transpose=True)
    d1, s1 = co.mx_quantize(a, axis=1)
    assert torch.equal(d1t, d1.T) and torch.equal(s1t, s1.T)


@pytest.mark.parametrize("shape", [(128, 4), (256, 8), (129, 5), (133, 16), (1, 1), (640, 64)])
def test_to_blocked_matches_view_permute_definition(shape):
    g = torch.Generator().manual_seed(31)
    s = torch.randint(1, 255, shape, generator=g, dtype=torch.int32).to(torch.uint8)
    ref = eager.to_blocked(s)
    got = co.to_blocked(s)
    assert torch.equal(ref, got)
    R, Cc = shape
    # length = 128*ceil(R/128)*4*ceil(C/4); equals the operator's check when C % 4 == 0
    assert got.numel() == 128 * ((R + 127) // 128) * 4 * ((Cc + 3) // 4)
    lib = co.lib()
    for r, c in [(0, 0), (R - 1, Cc - 1), (R // 2, Cc // 2)]:
        assert int(got[lib.dto_blocked_offset(r, c, Cc)]) == int(s[r, c])


def _mx_operands(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    b = torch.randn(N, K, generator=g).to(torch.bfloat16)
    ad, asc = co.mx_quantize(a)
    bd, bsc = co.mx_quantize(b)
    return ad, asc, bd, bsc


@pytest.mark.parametrize("size", [(32, 16, 64), (129, 40, 128), (64, 64, 256)])
def test_mx_gemm_reference(size):
    M, N, K = size
    ad, asc, bd, bsc = _mx_operands(M, N, K, 41)
    got = co.mx_gemm_ref(ad, bd, co.to_blocked(asc), co.to_blocked(bsc))
    ref64 = (co.mx_dequant(ad, asc).double() @ co.mx_dequant(bd, bsc).double().T)
    torch.testing.assert_close(got.double(), ref64, rtol=1e-6, atol=1e-6)
    ref_eager = eager.mx_gemm_ref(ad.view(torch.float8_e4m3fn), asc, bd.view(torch.float8_e4m3fn), bsc)
    assert eager.compute_error(ref64, ref_eager) > 120
    # brute force one entry with python floats
    m, n = M // 2, N // 3
    da, db = co.mx_dequant(ad, asc), co.mx_dequant(bd, bsc)
    acc = sum(float(da[m, k]) * float(db[n, k]) for k in range(K))
    assert abs(acc - float(got[m, n])) <= 1e-5 * max(1.0, abs(acc))


def test_mx_gemm_scale_linearity():
    """bumping one operand's scale bytes by +1 doubles the matching contribution: a property
    that fails if scales are applied to the wrong rows / k-blocks."""
    M, N, K = 32, 32, 128
    ad, asc, bd, bsc = _mx_operands(M, N, K, 43)
    base = co.mx_gemm_ref(ad, bd, co.to_blocked(asc), co.to_blocked(bsc))
    asc2 = asc.clone()
    asc2[7, :] += 1
    out = co.mx_gemm_ref(ad, bd, co.to_blocked(asc2), co.to_blocked(bsc))
    torch.testing.assert_close(out[7], base[7] * 2)
    assert torch.equal(out[:7], base[:7]) and torch.equal(out[8:], base[8:])


# ----------------------------------------------------------------------------- MXFP4 (e2m1)
def test_e2m1_decode_matches_the_ocp_table_and_closed_form():
    """OCP Microscaling Formats v1.0, FP4 E2M1: magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6; bit 3 is the sign"""
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for code in range(16):
        s, e, m = code >> 3, (code >> 1) & 3, code & 1
        closed = (m * 0.5) if e == 0 else (1 + m / 2) * 2.0 ** (e - 1)
        closed = -closed if s else closed
        got = co.e2m1_to_f32(code)
        assert got == closed == (-table[code & 7] if s else table[code & 7])
        assert math.copysign(1.0, got) == (-1.0 if s else 1.0)
    assert eager.E2M1_VALUES == table


def test_e2m1_encode_is_nearest_even_and_saturates():
    grid = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    g = util.gen(31)
    xs = (torch.rand(4000, generator=g) * 8 - 1).tolist() + [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 7.0, 1e9]
    for x in xs:
        for sign in (1.0, -1.0):
            code = co.f32_to_e2m1(sign * x)
            a = abs(x)
            d = [abs(a - v) for v in grid]
            best = min(d)
            cands = [i for i, v in enumerate(d) if v == best]
            want = cands[0] if len(cands) == 1 else [i for i in cands if i % 2 == 0][0]
            assert code & 7 == want, (x, code)
            assert (code >> 3) == (1 if math.copysign(1.0, sign * x) < 0 else 0)
    for code in range(16):  # every code is a fixed point
        assert co.f32_to_e2m1(co.e2m1_to_f32(code)) == code


def test_fp4_unpack_low_nibble_first_c_vs_eager():
    g = util.gen(32)
    packed = torch.randint(0, 256, (37, 48), generator=g, dtype=torch.uint8)
    a, b = co.fp4_unpack(packed), eager.fp4_unpack(packed)
    assert torch.equal(a, b)
    assert a[3, 10] == co.e2m1_to_f32(int(packed[3, 5]) & 15) and a[3, 11] == co.e2m1_to_f32(int(packed[3, 5]) >> 4)


def test_fp4_operand_generator_properties():
    x = util.normal((64, 256), 33, torch.float32)
    x[5, 32:64] = 0.0
    data, scale = co.mx_fp4_quantize(x)
    assert data.shape == (64, 128) and scale.shape == (64, 8)
    deq = eager.mx_fp4_dequant(data, scale).float()
    blk = x.view(64, 8, 32)
    amax = blk.abs().amax(-1)
    # shared exponent floor(log2(amax)) - 2: the block maximum lands in [4, 8) before rounding
    e = scale.double() - 127
    nz = amax > 0
    scaled_max = amax.double() / torch.exp2(e)
    assert ((scaled_max[nz] >= 4) & (scaled_max[nz] < 8)).all()
    assert (scale[5, 1] == 0) and (deq[5, 32:64] == 0).all()
    # error: half a grid step (the widest is 2, between 4 and 6) of the block scale, saturation at 6
    err = (deq.view(64, 8, 32) - blk).abs().double()
    assert (err <= torch.exp2(e).unsqueeze(-1) * 2.0 + 1e-30).all()
    # idempotent on its own output
    d2, s2 = co.mx_fp4_quantize(deq)
    assert torch.equal(eager.mx_fp4_dequant(d2, s2).float(), deq)


def test_fp4_quantize_c_vs_eager_and_special_blocks():
    """the C restatement against the torch one on wide-range data in fp32 and bf16, and the documented
    special blocks: zero and subnormal maxima (byte 0), infinity (byte 253, payload saturates), NaN
    (byte 255, every nibble 7), the largest and smallest normal maxima, exact ties"""
    g = util.gen(36)
    x = torch.randn(96, 256, generator=g) * torch.exp(3.0 * torch.randn(96, 256, generator=g))
    x[0, :32] = 0.0
    x[1, :32] = 1e-41                      # subnormal block
    x[2, 5] = float("inf")
    x[3, 40] = float("-inf")
    x[4, 70] = float("nan")
    x[5, :32] = torch.finfo(torch.float32).max
    x[6, :32] = torch.finfo(torch.float32).tiny * 3
    x[7, :32] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4) * 1.0   # ties of the grid at scale 1 (max 6 -> byte 127)
    x[7, 31] = -5.0
    for t in (x, x.to(torch.bfloat16)):
        dc, sc = co.mx_fp4_quantize(t)
        de, se = eager.mx_fp4_quantize(t)
        assert torch.equal(sc, se) and torch.equal(dc, de)
    d, s = co.mx_fp4_quantize(x)
    assert s[0, 0] == 0 and (d[0, :16] == 0).all()
    assert s[1, 0] == 0 and (d[1, :16] == 0).all()
    assert s[2, 0] == 253 and (d[2, 2] & 15) == 0 and (d[2, 2] >> 4) == 7      # element 5 = +inf -> 6
    assert s[3, 1] == 253 and (d[3, 20] & 15) == 15                            # element 40 = -inf -> -6
    assert s[4, 2] == 255 and (d[4, 32:48] == 0x77).all()
    assert s[5, 0] == 252 and (d[5, :16] == 0x77).all()                        # max = 1.99.. * 2^127 -> 7.99.. -> saturates at 6
    assert s[6, 0] == 0
    assert s[7, 0] == 127
    # 0.25 -> 0 (tie to even code 0), 0.75 -> 1.0 (code 2), 1.25 -> 1.0, 1.75 -> 2.0 (code 4), 2.5 -> 2.0, 3.5 -> 4.0 (code 6), 5 -> 4.0, 6 -> 6
    assert [int(d[7, 0]) & 15, int(d[7, 0]) >> 4, int(d[7, 1]) & 15, int(d[7, 1]) >> 4] == [0, 2, 2, 4]
    assert [int(d[7, 2]) & 15, int(d[7, 2]) >> 4, int(d[7, 3]) & 15, int(d[7, 3]) >> 4] == [4, 6, 6, 7]
    assert int(d[7, 15]) >> 4 == 8 | 6                                          # -5 -> -4


def test_fp4_gemm_ref_against_float64_matmul_and_brute_force():
    M, N, K = 70, 52, 384
    a, sa = co.mx_fp4_quantize(util.normal((M, K), 34, torch.float32))
    b, sb = co.mx_fp4_quantize(util.normal((N, K), 35, torch.float32) * 7)
    ref = co.mx_fp4_gemm_ref(a, b, co.to_blocked(sa), co.to_blocked(sb))
    want = eager.mx_fp4_dequant(a, sa) @ eager.mx_fp4_dequant(b, sb).T
    assert torch.equal(ref, want.float())
    m, n = 13, 41
    acc = 0.0
    for k in range(K):
        av = co.e2m1_to_f32((int(a[m, k // 2]) >> (4 * (k & 1))) & 15) * 2.0 ** (int(sa[m, k // 32]) - 127)
        bv = co.e2m1_to_f32((int(b[n, k // 2]) >> (4 * (k & 1))) & 15) * 2.0 ** (int(sb[n, k // 32]) - 127)
        acc += av * bv
    assert abs(ref[m, n].item() - acc) <= 1e-6 * abs(acc)
