"""The binding's inference fusions after the reference's tests/test_inference_fusion.py:30-270:
RMS normalisation over every value with changed inputs, strided views and empty shapes; SiLU with
storage rounding and exceptional values; exact constant rows and argument validation; the gated
MLP stage by stage; SwiGLU with clipping, routing weights, exceptional values, empty views and
graph replay. Yardsticks are CPU FP64 arithmetic with explicit storage rounding and, where the
reference demands it, torch's own FP32 result bit for bit.
"""

import pytest
import torch
import torch.nn.functional as F

from camblas_amd import _native

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def module():
    binding = _native.tensor_module()
    assert binding is not None
    return binding


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(13,), (3, 31), (2, 3, 8192), (0, 8192), (2, 0)])
def test_rms_full_outputs_and_changed_values(module, device, dtype, shape):
    torch.manual_seed(30)
    x = torch.randn(shape, device=device, dtype=dtype)
    weight = torch.randn(shape[-1], device=device, dtype=dtype)
    for changed in (False, True):
        if changed:
            x.mul_(-0.5)
            weight.add_(0.25)
        actual = module.rms_norm(x, weight, 1e-6)
        host = x.cpu().double()
        normalised = (host * (host.square().mean(-1, keepdim=True) + 1e-6).rsqrt()).to(dtype)
        expected = (normalised.double() * weight.cpu().double()).to(dtype)
        torch.testing.assert_close(actual.cpu(), expected,
                                   rtol=0.015625 if dtype == torch.bfloat16 else 4e-6,
                                   atol=0.0078125 if dtype == torch.bfloat16 else 2e-6)
    if x.numel():
        storage = torch.empty((*shape[:-1], shape[-1] * 2), device=device, dtype=dtype)
        storage[..., ::2] = x
        torch.testing.assert_close(module.rms_norm(storage[..., ::2], weight, 1e-6).cpu(), actual.cpu(),
                                   rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_storage_rounding_and_exceptional_values(module, device, dtype):
    gate = torch.linspace(-20, 20, 4097, device=device, dtype=dtype)
    up = torch.randn_like(gate)
    for changed in (False, True):
        if changed:
            gate.add_(0.5)
            up.mul_(-2)
        host = gate.cpu().double()
        activated = (host / (1 + (-host).exp())).to(dtype)
        expected = (activated.double() * up.cpu().double()).to(dtype)
        torch.testing.assert_close(module.silu_multiply(gate, up).cpu(), expected,
                                   rtol=0.0078125 if dtype == torch.bfloat16 else 4e-6,
                                   atol=0.0078125 if dtype == torch.bfloat16 else 2e-6)
    gate = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -1000.0], device=device, dtype=dtype)
    up = torch.tensor([1, 1, 1, float("inf"), 1], device=device, dtype=dtype)
    wanted = torch.tensor([float("nan"), float("inf"), float("nan"), float("nan"), -0.0], dtype=dtype)
    torch.testing.assert_close(module.silu_multiply(gate, up).cpu(), wanted, rtol=0, atol=0, equal_nan=True)
    torch.testing.assert_close(module.silu_multiply(gate.flip(0), up.flip(0)).cpu(), wanted.flip(0),
                               rtol=0, atol=0, equal_nan=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rms_analytic_exceptional_and_validation(module, device, dtype):
    x = torch.full((3, 8192), 4.0, device=device, dtype=dtype)
    weight = torch.arange(8192, device=device).remainder(16).to(dtype)
    torch.testing.assert_close(module.rms_norm(x, weight, 0), weight.expand_as(x), rtol=0, atol=0)
    x[0, 4] = float("nan")
    x[1, 0] = float("inf")
    x[2].zero_()
    got = module.rms_norm(x, weight, 0).cpu()
    # a NaN or an infinity makes the mean of squares NaN or infinite: the NaN row is NaN throughout,
    # the infinite row is inf * 0 = NaN at the infinity and 0 elsewhere (times the weight), and the
    # zero row is 0 * rsqrt(0) = 0 * inf = NaN
    host = x.cpu().float()
    expected = weight.cpu() * (host * host.square().mean(-1, keepdim=True).rsqrt()).to(dtype)
    torch.testing.assert_close(got, expected, rtol=0, atol=0, equal_nan=True)
    for bad in (-1, float("nan")):
        with pytest.raises(ValueError):
            module.rms_norm(x, weight, bad)
    with pytest.raises(ValueError):
        module.rms_norm(x, weight[:4])
    with pytest.raises(ValueError):
        module.rms_norm(x.clone().requires_grad_(), weight)
    with pytest.raises(ValueError):
        module.rms_norm(torch.ones((2, 13), device=device, dtype=torch.float64),
                        torch.ones(13, device=device, dtype=torch.float64))
    with pytest.raises(ValueError):
        module.silu_multiply(torch.ones(13, device=device), torch.ones(7, device=device))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_mlp_stage_by_stage(module, device, dtype):
    torch.manual_seed(31)
    x = torch.randn((2, 3, 17), device=device, dtype=dtype) / 4
    weights = [torch.randn(shape, device=device, dtype=dtype) / 4 for shape in ((31, 17), (31, 17), (13, 31))]
    for changed in (False, True):
        if changed:
            x.add_(0.125)
            for w in weights:
                w.mul_(-0.5)
        gate = (x.cpu().double() @ weights[0].cpu().double().T).to(dtype)
        up = (x.cpu().double() @ weights[1].cpu().double().T).to(dtype)
        g = gate.double()
        activated = (g / (1 + (-g).exp())).to(dtype)
        hidden = (activated.double() * up.double()).to(dtype)
        expected = (hidden.double() @ weights[2].cpu().double().T).to(dtype)
        torch.testing.assert_close(module.gated_mlp(x, *weights).cpu(), expected,
                                   rtol=0.02 if dtype == torch.bfloat16 else 1e-5,
                                   atol=0.002 if dtype == torch.bfloat16 else 2e-6)
    with pytest.raises(ValueError):
        module.gated_mlp(x, weights[0], weights[1][:5], weights[2])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_swiglu_clipping_routing_and_changed_operands(module, device, dtype):
    torch.manual_seed(20261004)
    gate = torch.randn((3, 17, 2304), device=device, dtype=dtype) * 8
    up = torch.randn_like(gate) * 8
    routing = torch.randn((3, 17, 1), device=device, dtype=torch.float32)
    for changed in ("original", "gate", "up", "routing"):
        if changed == "gate":
            gate.mul_(-0.5).add_(0.25)
        elif changed == "up":
            up.mul_(3)
        elif changed == "routing":
            routing.add_(0.25)
        for limit in (0, 10):
            for weights in (None, routing):
                host_g, host_u = gate.cpu().double(), up.cpu().double()
                if limit:
                    host_g, host_u = host_g.clamp(max=limit), host_u.clamp(-limit, limit)
                independent = host_g / (1 + (-host_g).exp()) * host_u
                if weights is not None:
                    independent = weights.cpu().double() * independent
                actual = module.swiglu(gate, up, routing=weights, limit=limit)
                torch.testing.assert_close(actual.cpu().double(), independent,
                                           rtol=0.008 if dtype == torch.bfloat16 else 4e-6,
                                           atol=0.0001 if dtype == torch.bfloat16 else 2e-6)
    with pytest.raises(ValueError):
        module.swiglu(gate, up, routing=routing.to(dtype=torch.float64))
    with pytest.raises(ValueError):
        module.swiglu(gate, up, routing=routing[..., 0, 0])
    for limit in (-1, float("nan"), float("inf")):
        with pytest.raises(ValueError):
            module.swiglu(gate, up, limit=limit)


def test_swiglu_exceptional_values_empty_views_and_graphs(module, device):
    gate = torch.tensor([[float("nan"), float("inf"), -float("inf"), 0, -1000, 1000]], device=device,
                        dtype=torch.bfloat16)
    up = torch.tensor([[1, 1, 1, float("inf"), 1, 1]], device=device, dtype=gate.dtype)
    routing = torch.ones(1, device=device, dtype=torch.float32)
    for limit in (0, 10):
        g, u = gate.float().cpu(), up.float().cpu()
        if limit:
            g, u = g.clamp(max=limit), u.clamp(-limit, limit)
        expected = (g / (1 + (-g).exp()) * u).to(gate.dtype)
        torch.testing.assert_close(module.swiglu(gate, up, routing=routing, limit=limit).cpu(), expected,
                                   rtol=0, atol=0, equal_nan=True)
        assert module.swiglu(gate[:0], up[:0], routing=routing[:0]).shape == (0, 6)
    gate = torch.randn((3, 34), device=device, dtype=torch.bfloat16)[:, ::2]
    up = torch.randn_like(gate)
    routing = torch.randn(3, device=device, dtype=torch.float32)
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(stream):
        module.swiglu(gate, up, routing=routing, limit=10)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            output = module.swiglu(gate, up, routing=routing, limit=10)
        for _ in range(3):
            gate.add_(1)
            up.mul_(-0.5)
            routing.add_(0.25)
            graph.replay()
            stream.synchronize()
            g, u = gate.float().cpu().clamp(max=10).double(), up.float().cpu().clamp(-10, 10).double()
            expected = routing.cpu().double()[:, None] * (g / (1 + (-g).exp()) * u)
            torch.testing.assert_close(output.cpu().double(), expected, rtol=0.008, atol=0.0001)
    graph.reset()
