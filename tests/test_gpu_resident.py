"""GPU parity of the single-kernel ("resident") per-tensor dynamic quantization: the tensor is held
in registers and LDS between the amax reduction and the cast.  Bit for bit against the CPU oracle
and against the two-kernel path, on ragged sizes, at and past the capacity of the chip, with NaN and
infinity in the data, from two streams, and with the barrier's wait forced to give up."""
import pytest
import torch

from oracle import c_oracle as co
from tests import util

pytestmark = pytest.mark.gpu

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
MODE = {1: "ROUND_V1", 2: "ROUND_V2", 3: "ROUND_V3"}


@pytest.fixture()
def cabi(gpu_device):
    from driss_torch_amd import cabi as c

    keep = {k: c.get_tuning(k) for k in ("dynamic.resident", "dynamic.resident_min_kib", "dynamic.resident_gap_lo_kib",
                                         "dynamic.resident_gap_hi_kib", "dynamic.resident_spin_limit")}
    c.set_tuning("dynamic.resident_min_kib", 0)  # every size takes the resident kernel
    c.set_tuning("dynamic.resident_gap_hi_kib", 0)
    yield c
    for k, v in keep.items():
        c.set_tuning(k, v)


def _timeout_flag(cabi):
    ws = cabi.workspace(torch.device("cuda"))
    torch.cuda.synchronize()
    return int(ws[196:200].cpu().view(torch.int32).item())


def _both_paths(cabi, x, fn):
    cabi.set_tuning("dynamic.resident", 1)
    a = fn(x)
    cabi.set_tuning("dynamic.resident", 0)
    b = fn(x)
    cabi.set_tuning("dynamic.resident", 1)
    return a, b


@pytest.mark.parametrize("shape", [(1, 8), (3, 7), (64, 17), (512, 127), (1000, 1003), (4096, 4097), (1, 1 << 20)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fp8_dtype", [E4, E5])
def test_resident_single_output(cabi, shape, in_dtype, fp8_dtype):
    x = util.normal_with_outliers(shape, 31 + shape[1], in_dtype)
    modes = (1, 2, 3) if in_dtype == torch.bfloat16 else (3,)
    for mode in modes:
        (out, amax, scale), (out2, amax2, scale2) = _both_paths(cabi, x.cuda(), lambda t: cabi.dynamic_scaled_quant(t, fp8_dtype, mode))
        ref, ramax, rscale = co.dynamic_scaled_quant(x, fp8_dtype, getattr(co, MODE[mode]))
        assert torch.equal(util.codes(out), ref) and torch.equal(util.codes(out2), ref)
        assert amax.item() == ramax.item() == amax2.item() and scale.item() == rscale.item() == scale2.item()
    assert _timeout_flag(cabi) == 0


@pytest.mark.parametrize("shape", [(5, 3), (257, 1023), (2048, 2048), (3000, 1111)], ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_resident_pair(cabi, shape, in_dtype):
    x = util.normal_with_outliers(shape, 77, in_dtype)
    modes = (1, 2, 3) if in_dtype == torch.bfloat16 else (3,)
    for mode in modes:
        (o4, o5, amax, scales), (p4, p5, amax2, scales2) = _both_paths(cabi, x.cuda(), lambda t: cabi.dynamic_scaled_quant_pair(t, mode))
        r4, ramax, rs4 = co.dynamic_scaled_quant(x, E4, getattr(co, MODE[mode]))
        r5, _, rs5 = co.dynamic_scaled_quant(x, E5, getattr(co, MODE[mode]))
        assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(o5), r5)
        assert torch.equal(util.codes(p4), r4) and torch.equal(util.codes(p5), r5)
        assert amax.item() == ramax.item() and scales.tolist() == [rs4.item(), rs5.item()] == scales2.tolist()
        # the identity the shared product relies on
        assert scales[1].item() == 128.0 * scales[0].item()


@pytest.mark.parametrize("amax", [1e-30, 3e-13, 1e-12, 7.3e-5, 0.1, 1.0, 3.14159, 448.0, 57344.0, 6.5e4, 1e20, 3.3e38])
def test_e5m2_scale_is_128_times_e4m3_scale(amax):
    """the pair kernel derives the e5m2 operand from the e4m3 one: fmax ratio 57344 / 448 = 2^7"""
    assert co.amax_to_scale(amax, E5) == 128.0 * co.amax_to_scale(amax, E4)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_resident_special_values(cabi, in_dtype):
    """an infinity makes the scale 0 and inf * 0 a NaN; a NaN makes everything NaN: both take the
    kernel's re-read path and must equal the two-kernel result and the oracle"""
    for special in (float("inf"), float("-inf"), float("nan")):
        x = util.normal((300, 257), 5, in_dtype)
        x[17, 3] = special
        # (a NaN times a NaN scale keeps the sign of whichever operand the multiplier picks: use one sign)
        x[299, 256] = special if special != special else -special
        (o4, o5, amax, _), (p4, p5, amax2, _) = _both_paths(cabi, x.cuda(), lambda t: cabi.dynamic_scaled_quant_pair(t, 2 if in_dtype == torch.bfloat16 else 3))
        r4, ramax, _ = co.dynamic_scaled_quant(x, E4, co.ROUND_V2 if in_dtype == torch.bfloat16 else co.ROUND_V3)
        assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(p4), r4)
        assert torch.equal(util.codes(o5), util.codes(p5))
        assert (amax.item() == ramax.item()) or (amax.item() != amax.item() and ramax.item() != ramax.item())
    x = torch.zeros((64, 64), dtype=in_dtype)
    o4, o5, amax, scales = cabi.dynamic_scaled_quant_pair(x.cuda(), 3)
    assert amax.item() == 0.0 and not util.codes(o4).any() and not util.codes(o5).any()
    assert _timeout_flag(cabi) == 0


def test_resident_capacity_boundary(cabi):
    """8192 x 8192 bf16 (and 8192 x 4096 fp32) is exactly what 256 CUs hold; with one more row the
    kernel keeps what fits and reads the rest twice"""
    cabi.set_tuning("dynamic.resident", 1)
    for shape, dtype in (((8192, 8192), torch.bfloat16), ((8192, 4096), torch.float32), ((8193, 8192), torch.bfloat16)):
        x = util.normal_with_outliers(shape, 1002, dtype)
        o4, o5, amax, scales = cabi.dynamic_scaled_quant_pair(x.cuda(), 2 if dtype == torch.bfloat16 else 3)
        mode = co.ROUND_V2 if dtype == torch.bfloat16 else co.ROUND_V3
        r4, ramax, rs4 = co.dynamic_scaled_quant(x, E4, mode)
        r5, _, rs5 = co.dynamic_scaled_quant(x, E5, mode)
        assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(o5), r5)
        assert amax.item() == ramax.item() and scales.tolist() == [rs4.item(), rs5.item()]
    assert _timeout_flag(cabi) == 0


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_resident_with_overflow_against_oracle(cabi, in_dtype):
    """a tensor somewhat larger than the chip holds, ragged, with the maximum in the part that is not
    kept (the slots past the 128th of a lane's share) and in the kept part: oracle, every rounding mode"""
    cabi.set_tuning("dynamic.resident", 1)
    cols = 8200 if in_dtype == torch.bfloat16 else 4100
    x = util.normal_with_outliers((9001, cols), 1003, in_dtype)
    modes = (1, 2, 3) if in_dtype == torch.bfloat16 else (3,)
    for where in ((9000, cols - 3), (17, 5)):
        x[where] = 16384.0
        g = x.cuda()
        for mode in modes:
            out, amax, scale = cabi.dynamic_scaled_quant(g, E5, mode)
            ref, ramax, rscale = co.dynamic_scaled_quant(x, E5, getattr(co, MODE[mode]))
            assert amax.item() == ramax.item() == 16384.0 and scale.item() == rscale.item()
            assert torch.equal(util.codes(out), ref)
        o4, o5, amax, scales = cabi.dynamic_scaled_quant_pair(g, modes[-1])
        r4, _, rs4 = co.dynamic_scaled_quant(x, E4, getattr(co, MODE[modes[-1]]))
        assert torch.equal(util.codes(o4), r4) and scales[0].item() == rs4.item()
        x[where] = 0.5
    assert _timeout_flag(cabi) == 0


def test_resident_with_overflow_sizes_and_special_values(cabi):
    """from one vector past the capacity to four times the capacity (and just beyond, where the two
    kernels take over): the same bits as the two-kernel path, also with an infinity or a NaN in the
    part that is read twice"""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    cap = cus * 256 * 128 * 8  # bf16 elements the chip holds
    base = util.normal_with_outliers((1, 1 << 20), 1004, torch.bfloat16).cuda()
    for numel in (cap + 8, cap + 8 * 256 * cus + 3, 2 * cap - 5, 4 * cap, 4 * cap + 8):
        x = base.repeat(1, numel // base.numel() + 1)[:, :numel].contiguous()
        x[0, numel - 7] = 768.0
        for special in (None, float("inf"), float("nan")):
            if special is not None:
                x[0, numel - 100] = special
            cabi.set_tuning("dynamic.resident_overflow", 1)
            a = cabi.dynamic_scaled_quant_pair(x, 2)
            cabi.set_tuning("dynamic.resident_overflow", 0)
            b = cabi.dynamic_scaled_quant_pair(x, 2)
            cabi.set_tuning("dynamic.resident_overflow", 1)
            assert torch.equal(util.codes(a[0]), util.codes(b[0])) and torch.equal(util.codes(a[1]), util.codes(b[1]))
            assert torch.equal(a[2].view(torch.int32), b[2].view(torch.int32)) and torch.equal(a[3].view(torch.int32), b[3].view(torch.int32))
            if special is None:
                assert a[2].item() == 768.0
        del x
    assert _timeout_flag(cabi) == 0


def test_resident_back_to_back_and_two_streams(cabi):
    """the workspace re-arms itself between launches of different sizes, and launches from two
    streams are chained by the host instead of sharing the chip"""
    cabi.set_tuning("dynamic.resident", 1)
    xs = [util.normal_with_outliers(s, 9 + i) for i, s in enumerate([(2048, 2048), (100, 37), (4096, 1024), (64, 64)])]
    refs = [co.dynamic_scaled_quant(x, E4, co.ROUND_V2)[0] for x in xs]
    gx = [x.cuda() for x in xs]
    outs = [cabi.dynamic_scaled_quant(g, E4, 2)[0] for g in gx for _ in range(2)]
    for i, o in enumerate(outs):
        assert torch.equal(util.codes(o), refs[i // 2])
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    results = []
    for rep in range(6):
        st = streams[rep % 2]
        with torch.cuda.stream(st):
            results.append((rep % len(xs), cabi.dynamic_scaled_quant(gx[rep % len(xs)], E4, 2)[0]))
    torch.cuda.synchronize()
    for i, o in results:
        assert torch.equal(util.codes(o), refs[i])
    for st in streams:
        with torch.cuda.stream(st):
            ws = cabi.workspace(torch.device("cuda"))
            torch.cuda.synchronize()
            assert int(ws[196:200].cpu().view(torch.int32).item()) == 0


def test_resident_not_taken_on_a_stream_restricted_to_some_cus(cabi):
    """a stream created with a CU mask of half the chip could never hold one workgroup per CU at
    once: the library sees the mask and takes the two kernels there (right results, no give-up flag;
    the spin limit is lowered so that a launch of the resident kernel would show up at once)"""
    import ctypes

    hip = ctypes.CDLL("libamdhip64.so")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    words = (cus + 31) // 32
    mask = (ctypes.c_uint32 * words)(*([0xFFFFFFFF] * (words // 2) + [0] * (words - words // 2)))
    handle = ctypes.c_void_p()
    assert hip.hipExtStreamCreateWithCUMask(ctypes.byref(handle), ctypes.c_uint32(words), mask) == 0
    stream = torch.cuda.ExternalStream(handle.value)
    cabi.set_tuning("dynamic.resident", 1)
    cabi.set_tuning("dynamic.resident_spin_limit", 64)
    x = util.normal_with_outliers((4096, 4096), 77)
    xg = x.cuda()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        o4, o5, amax, scales = cabi.dynamic_scaled_quant_pair(xg, 2)
        flag_ws = cabi.workspace(torch.device("cuda"))
        small = cabi.dynamic_scaled_quant(xg[:8], E4, 2)  # a grid of few workgroups fits the masked CUs: resident
    stream.synchronize()
    r4, ramax, _ = co.dynamic_scaled_quant(x, E4, co.ROUND_V2)
    r5, _, _ = co.dynamic_scaled_quant(x, E5, co.ROUND_V2)
    assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(o5), r5) and amax.item() == ramax.item()
    assert torch.equal(util.codes(small[0]), co.dynamic_scaled_quant(x[:8], E4, co.ROUND_V2)[0])
    assert int(flag_ws[196:200].cpu().view(torch.int32).item()) == 0
    cabi.set_tuning("dynamic.resident_spin_limit", 1 << 19)


def test_one_kernel_path_needs_the_opt_in(gpu_device):
    """without the opt-in (dt_set_exclusive_gpu / DRISS_TORCH_RESIDENT) the torch op and the C ABI never
    launch the kernel that waits for the whole chip, whatever the tensor's size: they run the reduction and
    the cast, with the same bits; with it a tensor of 32 MiB and more takes the one kernel"""
    import driss_torch_amd as d
    from driss_torch_amd import cabi as c

    L = c.lib()
    keep = L.dt_get_exclusive_gpu()
    x = util.normal_with_outliers((4096, 4096), 5)  # 32 MiB of bf16: the smallest size of the one-kernel path
    xg = x.cuda()
    ref, ramax, _ = co.dynamic_scaled_quant(x, E4, co.ROUND_V2)
    try:
        d.set_exclusive_gpu(False)
        n0 = L.dt_dynamic_quant_resident_launches()
        out = d.dynamic_scaled_quant(xg, E4)
        o4, o5, amax, _ = d.dynamic_scaled_quant_pair(xg)
        out_c, amax_c, _ = c.dynamic_scaled_quant(xg, E4, 2)
        torch.cuda.synchronize()
        assert L.dt_dynamic_quant_resident_launches() == n0
        assert torch.equal(util.codes(out), ref) and torch.equal(util.codes(o4), ref) and torch.equal(util.codes(out_c), ref)
        assert amax.item() == ramax.item() == amax_c.item()
        d.set_exclusive_gpu(True)
        out = d.dynamic_scaled_quant(xg, E4)
        torch.cuda.synchronize()
        assert L.dt_dynamic_quant_resident_launches() == n0 + 1
        assert torch.equal(util.codes(out), ref)
    finally:
        L.dt_set_exclusive_gpu(keep)


def test_resident_wait_gives_up_loudly(cabi):
    """with a spin limit of one poll most workgroups stop waiting before the last one has arrived:
    every wave still runs to the end, the sticky flag is set and those workgroups write NaN -- and
    the caller is told: the next call on the device returns DT_ERR_RESIDENT_GAVE_UP (a RuntimeError
    through the torch op) and launches nothing, the one-kernel path is off from then on, and the
    workspace is still good for the two kernels and, once switched on again, for the one."""
    import driss_torch_amd as d

    L = cabi.lib()
    assert L.dt_dynamic_quant_gave_up() == 0
    cabi.set_tuning("dynamic.resident", 1)
    cabi.set_tuning("dynamic.resident_spin_limit", 1)
    x = util.normal((8192, 2048), 3).cuda()
    ref, ramax, _ = co.dynamic_scaled_quant(x.cpu(), E4, co.ROUND_V2)
    try:
        out, amax, scale = cabi.dynamic_scaled_quant(x, E4, 2)
        torch.cuda.synchronize()
        assert _timeout_flag(cabi) == 1
        codes = util.codes(out)
        assert ((codes & 0x7F) == 0x7F).any()
        # amax and scale are NaN too, whichever workgroup was the last to leave
        assert amax.isnan().all() and scale.isnan().all()
        cabi.set_tuning("dynamic.resident_spin_limit", 1 << 19)
        # the following call, through the torch op: an error, nothing launched, the path switched off
        with pytest.raises(RuntimeError, match="gave up"):
            d.dynamic_scaled_quant(x, E4)
        assert cabi.get_tuning("dynamic.resident") == 0
        assert L.dt_dynamic_quant_gave_up() == 0  # reported once
        # calls after that take the two kernels, on the same workspace, and are right
        out, amax, scale = cabi.dynamic_scaled_quant(x, E4, 2)
        assert torch.equal(util.codes(out), ref) and amax.item() == ramax.item()
        assert torch.equal(util.codes(d.dynamic_scaled_quant(x, E4)), ref)
        # and so is the one kernel once it is switched on again: the barrier's words were re-armed by the
        # last workgroup to leave, give-up or not (only the sticky flag stays until dt_workspace_init)
        cabi.set_tuning("dynamic.resident", 1)
        out, amax, scale = cabi.dynamic_scaled_quant(x, E4, 2)
        assert torch.equal(util.codes(out), ref) and amax.item() == ramax.item()
        assert _timeout_flag(cabi) == 1
        # the same through the C ABI: give up again, ask without a quantization call
        cabi.set_tuning("dynamic.resident_spin_limit", 1)
        cabi.dynamic_scaled_quant(x, E4, 2)
        torch.cuda.synchronize()
        cabi.set_tuning("dynamic.resident_spin_limit", 1 << 19)
        assert L.dt_dynamic_quant_gave_up() == 1 and L.dt_dynamic_quant_gave_up() == 0
        cabi.dynamic_scaled_quant(x, E4, 2)
        torch.cuda.synchronize()
        cabi.set_tuning("dynamic.resident_spin_limit", 1)
        cabi.dynamic_scaled_quant(x, E4, 2)
        torch.cuda.synchronize()
        cabi.set_tuning("dynamic.resident_spin_limit", 1 << 19)
        with pytest.raises(cabi.DtError) as err:
            cabi.dynamic_scaled_quant_pair(x, 2)
        assert err.value.status == 9
    finally:
        cabi.set_tuning("dynamic.resident_spin_limit", 1 << 19)
        cabi.set_tuning("dynamic.resident", 1)
        L.dt_dynamic_quant_gave_up()
        ws = cabi.workspace(torch.device("cuda"))
        assert L.dt_workspace_init(ws.data_ptr(), ws.numel(), None) == 0
        torch.cuda.synchronize()
    out, amax, scale = cabi.dynamic_scaled_quant(x, E4, 2)
    assert torch.equal(util.codes(out), ref) and amax.item() == ramax.item()
    assert _timeout_flag(cabi) == 0


@pytest.mark.parametrize("slots,delta", [(1, 3), (15, -8), (16, 0), (16, 13), (17, -3), (33, 5), (92, 0), (92, 8), (93, -1), (108, 7), (109, 1)],
                         ids=lambda v: str(v))
def test_resident_batch_boundaries(cabi, slots, delta):
    """sizes around the 16-vector batches a workgroup may skip, around the register / LDS split (92
    vectors per lane) and with a ragged tail: a lane holds `slots` vectors, give or take a few elements"""
    cabi.set_tuning("dynamic.resident", 1)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    numel = slots * cus * 256 * 8 + delta
    x = util.normal_with_outliers((1, numel), 40 + slots, torch.bfloat16)
    x[0, -1] = 4096.0  # the maximum sits in the last (possibly partial) vector
    o4, o5, amax, scales = cabi.dynamic_scaled_quant_pair(x.cuda(), 2)
    r4, ramax, rs4 = co.dynamic_scaled_quant(x, E4, co.ROUND_V2)
    r5, _, rs5 = co.dynamic_scaled_quant(x, E5, co.ROUND_V2)
    assert amax.item() == ramax.item() == 4096.0 and scales.tolist() == [rs4.item(), rs5.item()]
    assert torch.equal(util.codes(o4), r4) and torch.equal(util.codes(o5), r5)
    assert _timeout_flag(cabi) == 0
