"""dt_dynamic_scaled_quant_noalloc, the entry point that allocates nothing (its reduction scratch is a
device array inside the library): through the C ABI, bit for bit against dt_dynamic_scaled_quant on
the same input, two calls in a row with the second on a smaller input, then the oracle and the limits."""
import pytest
import torch

from oracle import c_oracle as co
from tests import util

pytestmark = pytest.mark.gpu

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _noalloc(cabi, x, out_dtype, mode):
    L = cabi.lib()
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    amax = torch.empty(1, dtype=torch.float32, device=x.device)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    st = L.dt_dynamic_scaled_quant_noalloc(x.data_ptr(), cabi.IN_DTYPE[x.dtype], x.numel(), cabi.OUT_DTYPE[out_dtype], mode,
                                           out.data_ptr(), amax.data_ptr(), scale.data_ptr(),
                                           torch.cuda.current_stream().cuda_stream)
    assert st == 0, L.dt_status_string(st)
    return out, amax, scale


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("out_dtype", [E4, E5])
def test_noalloc_matches_the_workspace_entry_point_twice_in_a_row(gpu_device, in_dtype, out_dtype):
    from driss_torch_amd import cabi

    mode = cabi.ROUND_BF16_SCALE_PRODUCT
    big = util.normal_with_outliers((2048, 4099), 11, in_dtype).cuda()
    small = (util.normal((37, 1001), 12, in_dtype) * 0.01).cuda()  # a smaller amax: nothing of the first call may linger
    for x in (big, small):
        want, want_amax, want_scale = cabi.dynamic_scaled_quant(x, out_dtype, mode)
        got, amax, scale = _noalloc(cabi, x, out_dtype, mode)
        torch.cuda.synchronize()
        assert torch.equal(util.codes(got), util.codes(want))
        assert amax.item() == want_amax.item() and scale.item() == want_scale.item()
        ref, ramax, rscale = co.dynamic_scaled_quant(x.cpu(), out_dtype, co.ROUND_V2)
        assert torch.equal(util.codes(got), ref) and amax.item() == ramax.item() and scale.item() == rscale.item()


def test_noalloc_limits_and_no_device_allocation(gpu_device):
    from driss_torch_amd import cabi

    L = cabi.lib()
    x = util.normal((512, 512), 13).cuda()
    _noalloc(cabi, x, E4, 2)  # the first call on the device looks the scratch up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        _noalloc(cabi, x, E4, 2)
    torch.cuda.synchronize()
    out = torch.empty(8, dtype=torch.uint8, device="cuda")
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before - (2 << 20)  # nothing but torch's own small block for `out`
    fake = x.data_ptr()
    too_many = (1 << 34) + 2
    assert L.dt_dynamic_scaled_quant_noalloc(fake, cabi.BF16, too_many, cabi.E4M3FN, 2, out.data_ptr(), None, None, None) == 10
    assert b"no-allocation" in L.dt_status_string(10)
    assert L.dt_dynamic_scaled_quant_noalloc(fake, cabi.BF16, 0, cabi.E4M3FN, 2, out.data_ptr(), None, None, None) == 8
    assert L.dt_dynamic_scaled_quant_noalloc(None, cabi.BF16, 16, cabi.E4M3FN, 2, out.data_ptr(), None, None, None) == 3
    assert L.dt_dynamic_scaled_quant_noalloc(fake, cabi.F16, 16, cabi.E4M3FN, 2, out.data_ptr(), None, None, None) == 1
