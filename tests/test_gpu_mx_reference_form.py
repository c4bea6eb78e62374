"""The reference's own acceptance test of the block-scaled GEMMs, in its own form
(test/test_mx.py:9-67): `rand` bf16 operands -> MX cast -> op, compared with the bf16 matmul of the
operands dequantized to bf16 (`a_mx.to_dtype(bf16) @ b_mx.to_dtype(bf16).T`), SQNR > 80 dB, on its
eleven shapes including 8192^3, for e4m3 and e2m1 operands.  Everything runs on the device.

What stands in for the absent third-party helpers: the casts of this library for
`MXTensor.to_mx` (the comparison does not depend on how the operands were quantized, both sides
take the same payload and scales), `to_blocked` of this library for transformer_nuggets', and
`compute_error` = 20 log10(|x| / |x - y|) restated below (torchao.float8.float8_utils)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [(128, 128, 128), (256, 256, 256), (384, 384, 384), (512, 512, 512), (768, 768, 768), (1024, 1024, 1024),
         (8192, 8192, 8192), (128, 256, 384), (256, 384, 512), (129, 256, 384), (133, 512, 528)]
E2M1_VALUES = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


@pytest.fixture(scope="module")
def d(gpu_device):
    import driss_torch

    return driss_torch


def compute_error(x, y):
    ps = torch.norm(x.float())
    pn = torch.norm(x.float() - y.float())
    return (20 * torch.log10(ps / pn)).item()


def _scale_bf16(scale, rows, k):
    """E8M0 bytes [rows * k/32] -> bf16 [rows, k], one power of two per 32 elements (exact in bf16)"""
    e = scale.view(torch.uint8).view(rows, k // 32).to(torch.int32) - 127
    return torch.ldexp(torch.ones((), device=scale.device), e).to(torch.bfloat16).repeat_interleave(32, dim=1)


def _dequant_bf16(fmt, data, scale, rows, k):
    """what MXTensor.to_dtype(torch.bfloat16) gives: payload times block scale, in bf16 (exact: a payload
    has at most 4 significant bits)"""
    if fmt == "fp8":
        vals = data.to(torch.bfloat16)
    else:
        lut = torch.tensor(E2M1_VALUES + [-v for v in E2M1_VALUES], dtype=torch.bfloat16, device=data.device)
        b = data.view(torch.uint8)
        nib = torch.stack((b & 0xF, b >> 4), dim=-1).reshape(rows, k)  # even element in the low nibble
        vals = lut[nib.long()]
    return vals * _scale_bf16(scale, rows, k)


def run_matrix_test(d, M, K, N, fmt):
    a = torch.rand((M, K), dtype=torch.bfloat16, device="cuda")
    b = torch.rand((N, K), dtype=torch.bfloat16, device="cuda")
    if fmt == "fp8":
        a_data, a_scale = d.mx_fp8_quantize(a)
        b_data, b_scale = d.mx_fp8_quantize(b)
        mx_func = d.mx_fp8_bf16
    else:
        a_data, a_scale = d.mx_fp4_quantize(a)
        b_data, b_scale = d.mx_fp4_quantize(b)
        mx_func = d.mx_fp4_bf16
    assert b_data.is_contiguous()
    a_scale_block = d.to_blocked(a_scale.view(M, K // 32))
    b_scale_block = d.to_blocked(b_scale.view(N, K // 32))
    out_hp = _dequant_bf16(fmt, a_data, a_scale, M, K) @ _dequant_bf16(fmt, b_data, b_scale, N, K).transpose(-1, -2)
    out = mx_func(a_data, b_data.transpose(-1, -2), a_scale_block, b_scale_block)
    assert out.shape == out_hp.shape and out.dtype == torch.bfloat16
    return compute_error(out_hp, out), out_hp, out


@pytest.mark.parametrize("size", SIZES, ids=lambda s: f"{s[0]}x{s[1]}x{s[2]}")
@pytest.mark.parametrize("fmt", ["fp8", "fp4"])
def test_matrix_multiplication(d, size, fmt):
    M, K, N = size
    torch.manual_seed(M * 31 + K * 7 + N)
    sqnr, out_hp, out = run_matrix_test(d, M, K, N, fmt)
    differ = (out_hp != out).float().mean().item()
    assert sqnr > 80, f"{fmt} SQNR {sqnr} below threshold for dims {M}x{K}x{N} ({differ:.2e} of the entries differ)"
