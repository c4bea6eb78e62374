"""Pins the C oracle's number-format routines against torch's CPU conversions (library
routines) exhaustively, against the committed known-answer vectors, and the eager
restatement against the C oracle (two independent implementations)."""
import ctypes as C
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import eager

GOLD = Path(__file__).parent / "golden"


def _all_bf16():
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16)


def _f32_sweep(n=1 << 20, seed=0):
    g = torch.Generator().manual_seed(seed)
    bits = torch.randint(-(2**31), 2**31 - 1, (n,), generator=g, dtype=torch.int64).to(torch.int32)
    rnd = bits.view(torch.float32)
    # dense around the fp8 ranges, ties and subnormal boundaries
    e = torch.linspace(-20, 18, 4001).exp2()
    dense = torch.cat([e, -e, e * 1.5, e * 1.25, e * 1.0625, e * 1.125, e * (1 + 2**-20)])
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 448.0, 464.0, 465.0, 480.0,
                            57344.0, 61439.9, 61440.0, 65536.0, 2**-9, 2**-10, 1.5 * 2**-10, 2**-16, 2**-17, 1.5 * 2**-17])
    return torch.cat([rnd, dense, special, -special])


def _vec(fn, x_f32):
    lib = co.lib()
    f = getattr(lib, fn)
    arr = x_f32.numpy()
    return torch.tensor([f(C.c_float(float(v))) for v in arr], dtype=torch.uint8)


def _c_cast_codes(x, out_dtype):
    # scale 1.0 in V3 mode, then compare only where |x| <= fmax (unsaturated == plain convert)
    return co.saturated_cast(x, 1.0, out_dtype, co.ROUND_V3)


@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_fp8_convert_all_bf16_patterns(out_dtype):
    x = _all_bf16()
    fmax = torch.finfo(out_dtype).max
    ref = torch.clamp(x.float(), -fmax, fmax).to(out_dtype).view(torch.uint8)
    got = _c_cast_codes(x, out_dtype)
    nan = torch.isnan(x.float())
    assert torch.equal(got[~nan], ref[~nan])
    # NaN keeps its sign and becomes the canonical fp8 NaN (0x7F / 0xFF), as torch's convert does
    ref_nan = x.float().to(out_dtype).view(torch.uint8)
    assert torch.equal(got[nan], ref_nan[nan])


@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_fp8_convert_fp32_sweep_unsaturated(out_dtype):
    """the raw (non-saturating) convert: beyond max e4m3fn gives NaN, e5m2 gives inf"""
    x = _f32_sweep()
    ref = x.to(out_dtype).view(torch.uint8)
    lib = co.lib()
    fn = lib.dto_f32_to_e4m3fn if out_dtype == torch.float8_e4m3fn else lib.dto_f32_to_e5m2
    sub = x[:: max(1, x.numel() // 200000)]  # python loop: keep it to ~200k calls
    sub = torch.cat([sub, x[-40000:]])
    ref = sub.to(out_dtype).view(torch.uint8)
    got = torch.tensor([fn(C.c_float(v)) for v in sub.tolist()], dtype=torch.uint8)
    assert torch.equal(got, ref)


@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_fp8_convert_fp32_sweep_saturated(out_dtype):
    x = _f32_sweep()
    fmax = torch.finfo(out_dtype).max
    nan = torch.isnan(x)
    ref = torch.clamp(x, -fmax, fmax).to(out_dtype).view(torch.uint8)
    got = _c_cast_codes(x, out_dtype)
    assert torch.equal(got[~nan], ref[~nan])


def test_bf16_round_matches_torch():
    x = _f32_sweep()
    lib = co.lib()
    sub = x[:: max(1, x.numel() // 100000)]
    ref = sub.to(torch.bfloat16).view(torch.int16).to(torch.int32) & 0xFFFF
    got = torch.tensor([lib.dto_f32_to_bf16(C.c_float(v)) for v in sub.tolist()], dtype=torch.int32)
    nan = torch.isnan(sub)
    assert torch.equal(got[~nan], ref[~nan])
    assert all(((g & 0x7F80) == 0x7F80 and (g & 0x7F)) for g in got[nan].tolist())


def test_fp8_decode_all_codes():
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    lib = co.lib()
    for dt, fn in ((torch.float8_e4m3fn, lib.dto_e4m3fn_to_f32), (torch.float8_e5m2, lib.dto_e5m2_to_f32)):
        ref = codes.view(dt).float()
        got = torch.tensor([fn(int(c)) for c in codes.tolist()], dtype=torch.float32)
        assert torch.equal(torch.isnan(ref), torch.isnan(got))
        ok = ~torch.isnan(ref)
        assert torch.equal(ref[ok].view(torch.int32), got[ok].view(torch.int32))


def test_e8m0_decode_matches_torch():
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    ref = codes.view(torch.float8_e8m0fnu).float()
    lib = co.lib()
    got = torch.tensor([lib.dto_e8m0_to_f32(int(c)) for c in codes.tolist()], dtype=torch.float32)
    assert torch.isnan(got[255]) and torch.isnan(ref[255])
    assert torch.equal(ref[:255].view(torch.int32), got[:255].view(torch.int32))


def test_golden_known_answers():
    kat = json.loads((GOLD / "fp8_kat.json").read_text())
    lib = co.lib()
    for row in kat["convert"]:
        v = np.array([int(row["f32_bits"], 16)], dtype=np.uint32).view(np.float32)[0]
        assert lib.dto_f32_to_e4m3fn(C.c_float(v)) == row["e4m3fn"], row
        assert lib.dto_f32_to_e5m2(C.c_float(v)) == row["e5m2"], row
    for row in kat["scaled_quant_bf16"]:
        x = torch.tensor([int(row["x_bf16_bits"], 16)], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        for mode in (1, 2, 3):
            od = torch.float8_e5m2 if row["out"] == "e5m2" else torch.float8_e4m3fn
            got = co.saturated_cast(x, row["scale"], od, mode)
            assert int(got[0]) == row[f"v{mode}"], (row, mode)
    for row in kat["amax_to_scale"]:
        od = torch.float8_e5m2 if row["out"] == "e5m2" else torch.float8_e4m3fn
        a = np.array([int(row["amax_bits"], 16)], dtype=np.uint32).view(np.float32)[0]
        s = np.float32(co.amax_to_scale(a, od))
        assert hex(int(np.array([s]).view(np.uint32)[0])) == row["scale_bits"], row


def test_reference_edge_case_vector():
    """test/test_sat_cast.py:66-83: 0.3223(bf16) * 57344 -> e5m2.  The closest code is 20480
    (single rounding); rounding the product to bf16 first gives 16384."""
    x = torch.tensor([0.3223], dtype=torch.bfloat16)
    v3 = co.saturated_cast(x, 57344.0, torch.float8_e5m2, co.ROUND_V3).view(torch.float8_e5m2).float()
    v2 = co.saturated_cast(x, 57344.0, torch.float8_e5m2, co.ROUND_V2).view(torch.float8_e5m2).float()
    assert v3.item() == 20480.0
    assert v2.item() == 16384.0
    # and the eager formulation reproduces both through type promotion
    a = torch.tensor([[0.3223], [0.3223]], dtype=torch.bfloat16)
    assert eager.eager_scaled_quant(a, torch.tensor([57344.0]), torch.float8_e5m2).float()[0, 0] == 20480.0
    assert eager.eager_scaled_quant(a, torch.tensor(57344.0), torch.float8_e5m2).float()[0, 0] == 16384.0


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("mode", [1, 2, 3])
def test_c_oracle_vs_eager_modes(in_dtype, out_dtype, mode):
    g = torch.Generator().manual_seed(7 + mode)
    a = (torch.randn(257, 131, generator=g) * 3).to(in_dtype)
    a[0, 0], a[0, 1], a[0, 2], a[0, 3] = float("inf"), -float("inf"), 0.0, -0.0
    scale = eager.tensor_to_scale(a[1:], out_dtype)
    ref = eager.scaled_quant_mode(a, scale, out_dtype, mode).view(torch.uint8)
    got = co.saturated_cast(a, scale.item(), out_dtype, mode)
    assert torch.equal(got, ref)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_eager_promotion_is_v1_and_v3_on_cpu(in_dtype, out_dtype):
    """the literal eager_scaled_quant: 0-dim CPU scale -> V1, rank-1 scale -> V3"""
    g = torch.Generator().manual_seed(11)
    a = torch.randn(128, 96, generator=g).to(in_dtype)
    s0 = eager.tensor_to_scale(a, out_dtype)
    assert s0.dim() == 0 and s0.dtype == torch.float32
    v1 = eager.eager_scaled_quant(a, s0, out_dtype).view(torch.uint8)
    v3 = eager.eager_scaled_quant(a, s0.reshape(1), out_dtype).view(torch.uint8)
    assert torch.equal(v1, co.saturated_cast(a, s0.item(), out_dtype, co.ROUND_V1))
    assert torch.equal(v3, co.saturated_cast(a, s0.item(), out_dtype, co.ROUND_V3))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_amax_brute_force_and_invariants(in_dtype):
    g = torch.Generator().manual_seed(3)
    a = torch.randn(64, 127, generator=g).to(in_dtype)
    got = co.amax(a)
    assert torch.equal(got, eager.eager_amax(a))
    assert got.item() == max(abs(v) for v in a.float().flatten().tolist())  # brute force
    assert (a.float().abs() == got.item()).any()  # amax is one of the |x_i|
    perm = torch.randperm(a.numel(), generator=g)
    assert torch.equal(co.amax(a.flatten()[perm].reshape(a.shape)), got)  # permutation invariant
    b = a.clone()
    b[5, 5] = float("nan")
    assert torch.isnan(co.amax(b)) and torch.isnan(eager.eager_amax(b))


def test_scale_formula_closed_form():
    """f32(fmax / max(f64(amax), 1e-12)); for amax >= 1e-12 it equals the IEEE fp32 quotient."""
    g = torch.Generator().manual_seed(5)
    amaxes = torch.cat([torch.rand(2000, generator=g) * 100, torch.logspace(-20, 30, 500), torch.tensor([0.0, 1e-12, 1e-13])]).float()
    for od in (torch.float8_e4m3fn, torch.float8_e5m2):
        fmax = torch.finfo(od).max
        ref = eager.amax_to_scale(amaxes, od)
        got = torch.tensor([co.amax_to_scale(v, od) for v in amaxes.tolist()], dtype=torch.float32)
        assert torch.equal(ref.view(torch.int32), got.view(torch.int32))
        big = amaxes >= 1e-12
        q32 = torch.tensor(fmax, dtype=torch.float32) / amaxes[big]
        assert torch.equal(q32.view(torch.int32), got[big].view(torch.int32))
    assert co.amax_to_scale(0.0, torch.float8_e4m3fn) == np.float32(448.0 / 1e-12)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_dynamic_and_rowwise_vs_eager(in_dtype, out_dtype):
    g = torch.Generator().manual_seed(13)
    sig = 10 ** (torch.rand(96, 1, generator=g) * 6 - 3)
    a = (torch.randn(96, 160, generator=g) * sig).to(in_dtype)
    # per tensor: literal eager on CPU has a 0-dim scale -> V1
    q, am, sc = co.dynamic_scaled_quant(a, out_dtype, co.ROUND_V1)
    rq, ram, rsc = eager.dynamic_scaled_quant(a, out_dtype)
    assert torch.equal(q, rq.view(torch.uint8)) and torch.equal(am, ram) and sc.item() == rsc.item()
    # rowwise: [rows,1] scale -> fp32 promotion
    q, am, sc = co.dynamic_scaled_quant_rowwise(a, out_dtype)
    rq, ram, rsc = eager.dynamic_scaled_quant_rowwise(a, out_dtype)
    assert torch.equal(q, rq.view(torch.uint8))
    assert torch.equal(am, ram) and torch.equal(sc.view(torch.int32), rsc.view(torch.int32))
