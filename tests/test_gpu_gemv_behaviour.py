"""FP32 single-token products through the Python mirror, after the reference's
tests/test_float_gemv.py:47-233: long reductions with alpha/beta on padded weights, column-major
output padding through the C entry, exceptional values and zero scalars, the sizes either side of
the single-vector shortcut's gate, gradients, graph replay, and captured products that stay valid
after a later call has grown the context's scratch (here the BF16 split-K partial sums).
"""

import ctypes as ct

import pytest
import torch

from camblas_amd import _kernels, _native

pytestmark = pytest.mark.gpu


def check(actual, x, weight, alpha=1, beta=0, old=None):
    expected = alpha * (x.cpu().double() @ weight.cpu().double().T)
    if beta:
        expected += beta * old.cpu().double()
    torch.testing.assert_close(actual.cpu(), expected.float(), rtol=2e-4, atol=5e-5, equal_nan=True)


@pytest.mark.parametrize("inner,columns", [(4096, 1024), (8192, 8192), (28672, 1024)])
def test_long_inner_dimensions_scalars_padding_and_changes(device, inner, columns):
    torch.manual_seed(47)
    x = torch.randn((1, inner), device=device) / 8
    backing = torch.randn((columns, inner + 8), device=device) / 8
    weight = backing[:, :inner]
    code, text = _native.plan_describe(0, "T", "N", columns, 1, inner, inner + 8, inner, columns)
    assert code // 1000 == 1, text  # the single-vector kernel
    output = torch.full((1, columns), float("nan"), device=device)
    _kernels.matmul(x, weight.T, out=output)
    check(output, x, weight)
    old = torch.randn_like(output) / 8
    output.copy_(old)
    x.add_(0.015625)
    weight.mul_(-0.5)
    _kernels.matmul(x, weight.T, out=output, alpha=-0.75, beta=0.25)
    check(output, x, weight, -0.75, 0.25, old)


def test_column_major_output_padding(device):
    columns, inner = 1024, 4096
    weight = torch.randn((columns, inner + 8), device=device) / 8
    x = torch.randn((1, inner), device=device) / 8
    output = torch.full((1, columns + 13), float("nan"), device=device)
    native = _native.context(device)
    status = _native.library().camblas_cuda_sgemm(
        native.handle, b"T", b"N", columns, 1, inner, ct.c_float(1.0), ct.c_void_p(weight.data_ptr()),
        inner + 8, ct.c_void_p(x.data_ptr()), inner, ct.c_float(0.0), ct.c_void_p(output.data_ptr()),
        columns + 13)
    assert status == 0
    torch.cuda.synchronize()
    check(output[:, :columns], x, weight[:, :inner])
    assert torch.isnan(output[:, columns:]).all()


def test_exceptional_inputs_and_zero_scalars(device):
    x = torch.ones((1, 4096), device=device)
    weight = torch.ones((1024, 4096), device=device)
    weight[0, 0] = float("inf")
    weight[1, 0] = float("nan")
    output = _kernels.matmul(x, weight.T)
    check(output, x, weight)
    output.fill_(float("nan"))
    _kernels.matmul(x, weight.T, out=output, alpha=0, beta=0)
    assert not output.any()


def test_neighbouring_dimensions_views_and_gradients(device):
    torch.manual_seed(139)
    for inner, columns in ((4095, 1024), (4096, 1023), (4104, 1025)):
        x = (torch.randn((1, inner + 1), device=device) / 8)[:, 1:]
        weight = torch.randn((columns, inner), device=device) / 8
        check(_kernels.matmul(x, weight.T), x, weight)
    x = (torch.randn((1, 4096), device=device) / 8).requires_grad_()
    weight = (torch.randn((1024, 4096), device=device) / 8).requires_grad_()
    _kernels.matmul_autograd(x, weight.T).sum().backward()
    expected_x = weight.detach().cpu().double().sum(0, keepdim=True).float()
    torch.testing.assert_close(x.grad.cpu(), expected_x, rtol=2e-4, atol=5e-5)
    torch.testing.assert_close(weight.grad.cpu(), x.detach().cpu().expand(1024, -1), rtol=0, atol=0)


def test_graph_replay_with_changed_operands(device):
    torch.manual_seed(159)
    x = torch.randn((1, 4096), device=device) / 8
    weight = torch.randn((1024, 4096), device=device) / 8
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(stream):
        for _ in range(3):
            _kernels.matmul(x, weight.T)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            output = _kernels.matmul(x, weight.T)
        for _ in range(3):
            x.add_(0.015625)
            weight.mul_(-0.5)
            graph.replay()
            stream.synchronize()
            check(output, x, weight)
    graph.reset()


def test_captured_products_survive_scratch_growth(device):
    torch.manual_seed(179)
    with torch.no_grad():
        x = torch.randn((256, 16384), device=device) / 128
        weight = torch.randn((1024, 16384), device=device) / 128
        small, right = torch.randn((17, 13), device=device), torch.randn((13, 19), device=device)
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            # a BF16 product whose plan divides K over workgroups: its partial sums live in the
            # context's scratch, and the captured graph keeps that allocation
            early_x = torch.randn((128, 8192), device=device, dtype=torch.bfloat16) / 128
            early_weight = torch.randn((2048, 8192), device=device, dtype=torch.bfloat16) / 128
            assert "split_k" in _native.plan_describe(2, "T", "N", 2048, 128, 8192, 8192, 8192, 2048)[1]
            for _ in range(3):
                _kernels.matmul(early_x, early_weight.T)
            early_graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(early_graph, stream=stream):
                early_output = _kernels.matmul(early_x, early_weight.T)
            # a larger split-K product afterwards makes the context allocate a bigger scratch
            bigger_x = torch.randn((512, 8192), device=device, dtype=torch.bfloat16) / 128
            wide = torch.randn((4096, 8192), device=device, dtype=torch.bfloat16) / 128
            assert "split_k" in _native.plan_describe(2, "T", "N", 4096, 256, 8192, 8192, 8192, 4096)[1]
            _kernels.matmul(bigger_x[:256], wide.T)
            for _ in range(3):
                _kernels.matmul(x, weight.T)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                output = _kernels.matmul(x, weight.T)
            for _ in range(2):
                x.add_(0.001953125)
                weight.mul_(-0.5)
                graph.replay()
                early_x.add_(0.00390625)
                early_weight.mul_(-0.5)
                early_graph.replay()
                with _native.algorithm("classical"):
                    small_output = _kernels.matmul(small, right)
                stream.synchronize()
                torch.testing.assert_close(early_output.cpu().double(),
                                           early_x.cpu().double() @ early_weight.cpu().double().T,
                                           rtol=0.02, atol=0.002)
                torch.testing.assert_close(output.cpu().double(), x.cpu().double() @ weight.cpu().double().T,
                                           rtol=2e-4, atol=2e-4)
                torch.testing.assert_close(small_output.cpu().double(), small.cpu().double() @ right.cpu().double(),
                                           rtol=2e-5, atol=2e-5)
        early_graph.reset()
        graph.reset()
