"""torch.nn.functional.linear, torch.mm(out=), torch.addmm and torch.matmul with the backend
override installed, after the reference's tests/test_linear.py:55-170: all leading batch axes and
a broadcast bias, strided views, empty operands, out ownership and version counting, unsupported
dtypes falling back to ATen, first and second derivatives in FP64, and graph replay on a side
stream with changed inputs and weights. Sorts after the other binding tests: the override stays
installed for the rest of the process.
"""

import pytest
import torch
import torch.nn.functional as F

from camblas_amd import _native

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def binding():
    module = _native.tensor_module()
    assert module is not None
    module.install_torch_backend(_native.ALGORITHMS["lt"])
    previous = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    yield module
    torch.backends.cuda.matmul.allow_tf32 = previous


def launches(binding):
    return sum(binding.stats_all(0, False).values())


def assert_product(actual, expected):
    # ref: tests/test_linear.py:30-53
    dtype = actual.dtype
    # the reference's own bars, unchanged
    rtol, atol = {torch.float64: (2e-13, 3e-14), torch.float32: (1e-5, 3e-6),
                  torch.bfloat16: (0.015625, 0.002), torch.float16: (0.002, 0.0005),
                  torch.complex64: (1e-5, 3e-6)}[dtype]
    torch.testing.assert_close(actual.cpu(), expected.to(dtype), rtol=rtol, atol=atol, equal_nan=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
def test_shapes_views_bias_and_empty(binding, device, dtype):
    torch.manual_seed(5)
    for shape in ((13,), (5, 13), (2, 3, 5, 13)):
        x = torch.randn(shape, device=device, dtype=dtype) / 4
        weight = torch.randn((7, 13), device=device, dtype=dtype) / 4
        bias = torch.randn(7, device=device, dtype=dtype) / 4
        for value in (None, bias):
            before = launches(binding)
            actual = F.linear(x, weight, value)
            assert launches(binding) > before, "the product did not go through the library"
            expected = F.linear(x.cpu().double(), weight.cpu().double(),
                                None if value is None else value.cpu().double())
            assert_product(actual, expected)
    x = torch.randn((2, 5, 26), device=device, dtype=dtype)[..., ::2]
    weight = torch.randn((13, 7), device=device, dtype=dtype).T
    assert_product(F.linear(x, weight), F.linear(x.cpu().double(), weight.cpu().double()))
    for shape, width in (((2, 3, 0), 7), ((0, 5, 13), 7), ((2, 3, 13), 0)):
        x = torch.empty(shape, device=device, dtype=dtype)
        weight = torch.empty((width, shape[-1]), device=device, dtype=dtype)
        assert_product(F.linear(x, weight), torch.zeros((*shape[:-1], width), dtype=torch.float64))
    with pytest.raises(RuntimeError):
        F.linear(torch.ones((2, 13), device=device), torch.ones((7, 12), device=device))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16,
                                   torch.complex64])
def test_out_scalars_and_fallbacks(binding, device, dtype):
    torch.manual_seed(6)
    a = torch.randn((5, 7), device=device, dtype=dtype) / 4
    b = torch.randn((7, 3), device=device, dtype=dtype) / 4
    host = torch.complex128 if dtype.is_complex else torch.float64
    product = a.cpu().to(host) @ b.cpu().to(host)
    for out in (torch.empty((5, 3), device=device, dtype=dtype),
                torch.empty((3, 5), device=device, dtype=dtype).T):
        version = out._version
        assert torch.mm(a, b, out=out) is out
        assert out._version == version + 1
        assert_product(out, product)
    bias = torch.randn(3, device=device, dtype=dtype) / 4
    assert_product(torch.addmm(bias, a, b, alpha=0.7, beta=-0.3), 0.7 * product - 0.3 * bias.cpu().to(host))
    assert_product(torch.matmul(a, b), product)
    bias.fill_(float("nan"))
    assert_product(torch.addmm(bias, a, b, beta=0), product)
    # routed for the three storage types the library takes, ATen's own kernels for the others
    before = launches(binding)
    torch.mm(a, b)
    torch.cuda.synchronize()
    assert launches(binding) - before == (1 if dtype in (torch.float32, torch.float64, torch.bfloat16) else 0)


def test_first_and_second_derivatives(binding, device):
    torch.manual_seed(7)
    host = [torch.randn(shape, dtype=torch.float64).requires_grad_() for shape in ((2, 3, 13), (7, 13), (7,))]
    on_device = [value.detach().to(device).requires_grad_() for value in host]
    reference, actual = F.linear(*host), F.linear(*on_device)
    assert_product(actual, reference.detach())
    expected_grad = torch.autograd.grad(reference.square().sum(), host, create_graph=True)
    actual_grad = torch.autograd.grad(actual.square().sum(), on_device, create_graph=True)
    for result, expected in zip(actual_grad, expected_grad):
        torch.testing.assert_close(result.cpu(), expected, rtol=2e-12, atol=3e-13)
    expected_hessian = torch.autograd.grad(expected_grad[0].sum(), host[0])[0]
    actual_hessian = torch.autograd.grad(actual_grad[0].sum(), on_device[0])[0]
    torch.testing.assert_close(actual_hessian.cpu(), expected_hessian, rtol=2e-12, atol=3e-13)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
def test_graph_replay_with_changed_inputs_and_weights(binding, device, dtype):
    torch.manual_seed(8)
    x = torch.randn((5, 32), device=device, dtype=dtype) / 4
    weight = torch.randn((7, 32), device=device, dtype=dtype) / 4
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(stream):
        for _ in range(3):
            F.linear(x, weight)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            output = F.linear(x, weight)
        for _ in range(3):
            x.add_(0.125)
            weight.mul_(-0.5)
            graph.replay()
            stream.synchronize()
            assert_product(output, F.linear(x.cpu().double(), weight.cpu().double()))
    graph.reset()
