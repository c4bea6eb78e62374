"""torch.compile coverage of every op of the path: each wrapper traced with fullgraph=True (so the
fake implementations must produce the right shapes, dtypes and strides) and run through a backend
that needs no code generator, compared bit for bit with the direct call.  Follows
test/test_sat_cast.py:45-62, which does this for saturated_cast only."""
import pytest
import torch

from oracle import eager
from tests import util

pytestmark = pytest.mark.gpu

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


@pytest.fixture(scope="module")
def d(gpu_device):
    import driss_torch_amd

    return driss_torch_amd


def _compiled(fn):
    torch._dynamo.reset()
    return torch.compile(fn, fullgraph=True, backend="aot_eager")


def _same(a, b):
    if isinstance(a, (tuple, list)):
        assert len(a) == len(b)
        for x, y in zip(a, b):
            _same(x, y)
        return
    assert a.dtype == b.dtype and a.shape == b.shape and a.stride() == b.stride()
    if a.dtype in (E4, E5, torch.float8_e8m0fnu):
        assert torch.equal(util.codes(a), util.codes(b))
    else:
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_amax_compile(d, dtype):
    x = util.normal((256, 1024), 7001, dtype).cuda()
    _same(_compiled(d.amax)(x), d.amax(x))


@pytest.mark.parametrize("fp8_dtype", [E4, E5])
def test_dynamic_scaled_quant_compile(d, fp8_dtype):
    x = util.normal((512, 1024), 7002).cuda()
    _same(_compiled(d.dynamic_scaled_quant)(x, fp8_dtype), d.dynamic_scaled_quant(x, fp8_dtype))
    _same(_compiled(d.dynamic_scaled_quant_ex)(x, fp8_dtype), d.dynamic_scaled_quant_ex(x, fp8_dtype))
    _same(_compiled(d.dynamic_scaled_quant_rowwise)(x, fp8_dtype), d.dynamic_scaled_quant_rowwise(x, fp8_dtype))


def test_dynamic_scaled_quant_pair_compile(d):
    x = util.normal((512, 1024), 7003).cuda()
    _same(_compiled(d.dynamic_scaled_quant_pair)(x), d.dynamic_scaled_quant_pair(x))


@pytest.mark.parametrize("axis,transpose", [(1, False), (0, False), (0, True), (1, True)])
def test_mx_fp8_quantize_compile(d, axis, transpose):
    x = util.normal((256, 512), 7004).cuda()

    def fn(t):
        return d.mx_fp8_quantize(t, 32, axis, transpose, E4)

    _same(_compiled(fn)(x), fn(x))


def test_mx_quantize_blocked_and_gemm_compile(d):
    a = util.normal((256, 512), 7005).cuda()
    b = util.normal((384, 512), 7006).cuda()

    def fn(a, b):
        ad, sa = d.mx_fp8_quantize_blocked(a)
        bd, sb = d.mx_fp8_quantize_blocked(b)
        return d.mx_fp8_bf16(ad, bd.t(), sa, sb)

    got, want = _compiled(fn)(a, b), fn(a, b)
    assert got.shape == (256, 384) and got.dtype == torch.bfloat16
    _same(got, want)


def test_to_blocked_compile(d):
    s = torch.randint(0, 255, (256, 12), dtype=torch.uint8, device="cuda")
    _same(_compiled(d.to_blocked)(s), d.to_blocked(s))


@pytest.mark.parametrize("fp8_dtype", [E4, E5])
def test_saturated_cast_compile_default_backend(d, fp8_dtype):
    """test/test_sat_cast.py:45-62 as written there: torch.compile with its default backend"""
    torch._dynamo.reset()
    a = util.uniform((64, 512), 95).cuda()
    scale = eager.tensor_to_scale(a, fp8_dtype)
    fn = torch.compile(d.saturated_cast, fullgraph=True)
    _same(fn(a, scale, fp8_dtype), d.saturated_cast(a, scale, fp8_dtype))


def test_quantize_gemm_step_compile_default_backend(d):
    """a compiled function that mixes the ops with ordinary tensor code (generated kernels before and
    after the custom calls): per-tensor quantization, both MX casts, the GEMM"""
    torch._dynamo.reset()

    def step(a, w):
        q, amax, scale = d.dynamic_scaled_quant_ex(a * 0.5, E4, 0)
        qa, sa = d.mx_fp8_quantize_blocked(a + 1.0)
        qw, sw = d.mx_fp8_quantize_blocked(w)
        y = d.mx_fp8_bf16(qa, qw.t(), sa, sw)
        return y * 2.0 + amax.to(torch.bfloat16), q, scale

    a, w = util.normal((256, 512), 96).cuda(), util.normal((384, 512), 97).cuda()
    _same(torch.compile(step, fullgraph=True)(a, w), step(a, w))


def test_ops_replay_from_a_captured_graph(d):
    """every op recorded once into a HIP graph and replayed with new input contents, with eager
    calls and synchronisations between the replays; each replay equals the eager results bit for bit
    (per-tensor dynamic quantization takes its two-kernel path under capture)"""
    M, K, N = 512, 1024, 256
    sx = util.normal_with_outliers((M, K), 100).cuda()
    sw = util.normal((N, K), 101).cuda()
    scale = torch.tensor([3.7], device="cuda")

    def run(x, w):
        a, sa = d.mx_fp8_quantize_blocked(x)
        b, sb = d.mx_fp8_quantize_blocked(w)
        # the same bytes as one tile with 64 K-steps: the GEMM shares K between workgroups (ticket counters
        # that every replay must find at zero)
        a2, sa2 = d.mx_fp8_quantize_blocked(x.view(64, 8192))
        b2, sb2 = d.mx_fp8_quantize_blocked(w.view(32, 8192))
        return (d.mx_fp8_bf16(a2, b2.t(), sa2, sb2), d.amax(x), d.saturated_cast(x, scale, E4), d.dynamic_scaled_quant(x, E5),
                d.dynamic_scaled_quant_pair(x), d.dynamic_scaled_quant_rowwise(x, E4), d.mx_fp8_quantize(x),
                d.mx_fp8_quantize(x, 32, 0, True), d.mx_fp8_quantize_dual(x, E4, True), d.mx_fp8_bf16(a, b.t(), sa, sb),
                d.mx_fp4_quantize(x, True), d.mx_fp4_quantize_dual(x, True))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(sx, sw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run(sx, sw)
    for seed in (102, 103, 104):
        x = util.normal_with_outliers((M, K), seed).cuda()
        w = util.normal((N, K), seed + 10).cuda()
        sx.copy_(x)
        sw.copy_(w)
        graph.replay()
        torch.cuda.synchronize()
        _same(captured, run(x, w))
        torch.cuda.synchronize()
