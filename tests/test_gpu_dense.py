"""Dense FP32 / FP64 helpers of the C ABI: affine, MLP, MLP gradients, single-head attention.

Strategy and tolerances of the reference's tests/test_cuda.py (:38-58 assert_close: rtol 1e-5 /
atol 3e-6 for FP32, 2e-13 / 3e-14 for FP64, NaN equal; :356-435 affine and MLP with changed inputs
and exceptional values; :677-755 attention with unequal lengths, no keys, NaN queries and the
register / loop boundaries of the softmax; :1264-1283 gradient subsets), with torch's CPU FP64
arithmetic as the yardstick.
"""

import ctypes as ct

import pytest
import torch

from camblas_amd import _kernels, _native

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float64]


def close(actual, expected, magnitude=1.0):
    # magnitude: size of the terms behind an output, where sums of large terms nearly cancel
    rtol, atol = (1e-5, 3e-6) if actual.dtype == torch.float32 else (2e-13, 3e-14)
    atol *= magnitude
    torch.testing.assert_close(actual.cpu(), expected.to(actual.dtype).cpu(), rtol=rtol, atol=atol,
                               equal_nan=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_affine_and_mlp_values_and_all_gradients(device, dtype):
    torch.manual_seed(73013)
    shapes = ((11, 17), (17, 23), (23,), (23, 13), (13,))
    host = [torch.randn(shape, dtype=torch.float64) for shape in shapes]
    inputs = [t.to(device=device, dtype=dtype).requires_grad_() for t in host]
    wanted = [t.to(dtype).double().requires_grad_() for t in host]
    x, w1, b1, w2, b2 = wanted
    expected = torch.relu(x @ w1 + b1) @ w2 + b2
    actual = _kernels.mlp(*inputs)
    close(actual, expected)
    weight = torch.randn(expected.shape, dtype=torch.float64)
    (actual * weight.to(device=device, dtype=dtype)).sum().backward()
    (expected * weight.to(dtype).double()).sum().backward()
    for tensor, oracle in zip(inputs, wanted):
        close(tensor.grad, oracle.grad)
    for relu in (False, True):
        x, w1, b1 = (t.detach().clone().requires_grad_() for t in inputs[:3])
        xr, wr, br = (t.detach().double().cpu().requires_grad_() for t in (x, w1, b1))
        expected = xr @ wr + br
        if relu:
            expected = torch.relu(expected)
        actual = _kernels.affine(x, w1, b1, relu=relu)
        close(actual, expected)
        actual.square().sum().backward()
        expected.square().sum().backward()
        for tensor, oracle in ((x, xr), (w1, wr), (b1, br)):
            close(tensor.grad, oracle.grad)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,inner,columns", [(1, 17, 23), (13, 17, 1), (13, 17, 23), (130, 70, 65)])
def test_affine_changed_inputs_and_exceptional_values(device, dtype, rows, inner, columns):
    torch.manual_seed(705537)
    x = torch.randn((rows, inner), dtype=dtype) * 0.1
    weight = torch.randn((inner, columns), dtype=dtype) * 0.1
    bias = torch.randn((columns,), dtype=dtype) * 0.1
    for relu in (False, True, False):
        for changed in (False, True):
            ax = x + (0.03 if changed else 0)
            aw = weight * (0.7 if changed else 1)
            ab = bias + (0.04 if changed else 0)
            expected = ax.double() @ aw.double() + ab.double()
            if relu:
                expected = torch.relu(expected)
            close(_kernels.affine(ax.to(device), aw.to(device), ab.to(device), relu=relu), expected)
    for value in (float("nan"), float("inf"), -float("inf")):
        for operand in range(3):
            tensors = [x.clone(), weight.clone(), bias.clone()]
            tensors[operand].reshape(-1)[0] = value
            expected = tensors[0].double() @ tensors[1].double() + tensors[2].double()
            for relu in (False, True):
                close(_kernels.affine(*(t.to(device) for t in tensors), relu=relu),
                      torch.relu(expected) if relu else expected)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_lengths_no_keys_and_nan(device, dtype):
    torch.manual_seed(20261004)
    q = torch.randn((13, 17), dtype=dtype)
    k = torch.randn((19, 17), dtype=dtype)
    v = torch.randn((19, 23), dtype=dtype)
    for scale in (0.25, -0.5, 0):
        expected = torch.softmax((q.double() @ k.double().T) * scale, dim=-1) @ v.double()
        close(_kernels.attention(q.to(device), k.to(device), v.to(device), scale=scale), expected)
    expected = torch.softmax((q.double() @ k.double().T) / 17 ** 0.5, dim=-1) @ v.double()
    close(_kernels.attention(q.to(device), k.to(device), v.to(device)), expected)
    none = _kernels.attention(q.to(device), torch.empty((0, 17), dtype=dtype, device=device),
                              torch.empty((0, 23), dtype=dtype, device=device))
    assert torch.equal(none, torch.zeros((13, 23), dtype=dtype, device=device))
    q[0, 0] = float("nan")
    expected = torch.softmax((q.double() @ k.double().T) * 0, dim=-1) @ v.double()
    close(_kernels.attention(q.to(device), k.to(device), v.to(device), scale=0), expected)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("keys", [1, 17, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049,
                                  4095, 4096, 4097])
def test_attention_row_width_boundaries(device, dtype, keys):
    torch.manual_seed(717 + keys)
    q = torch.randn((7, 17), dtype=dtype) * 0.1
    k = torch.randn((keys, 17), dtype=dtype) * 0.1
    v = torch.randn((keys, 23), dtype=dtype) * 0.1
    for scale in (0.25, -0.5, 0, 256):
        expected = torch.softmax((q.double() @ k.double().T) * scale, dim=-1) @ v.double()
        close(_kernels.attention(q.to(device), k.to(device), v.to(device), scale=scale), expected)
    q.add_(0.03)
    v.mul_(0.7)
    expected = torch.softmax((q.double() @ k.double().T) * 0.25, dim=-1) @ v.double()
    close(_kernels.attention(q.to(device), k.to(device), v.to(device), scale=0.25), expected)
    if keys in (257, 1025, 4096, 4097):
        q[0, 0] = float("nan")
        expected = torch.softmax((q.double() @ k.double().T) * 0, dim=-1) @ v.double()
        close(_kernels.attention(q.to(device), k.to(device), v.to(device), scale=0), expected)


def test_attention_gradients(device):
    torch.manual_seed(842)
    q = torch.randn((3, 4), device=device, dtype=torch.float64, requires_grad=True)
    k = torch.randn((5, 4), device=device, dtype=torch.float64, requires_grad=True)
    v = torch.randn((5, 2), device=device, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(_kernels.attention, (q, k, v))


@pytest.mark.parametrize("index", range(5))
def test_mlp_single_requested_gradient(device, index):
    torch.manual_seed(413 + index)
    shapes = ((5, 7), (7, 11), (11,), (11, 3), (3,))
    inputs = [torch.randn(s, device=device, dtype=torch.float64).requires_grad_(i == index)
              for i, s in enumerate(shapes)]
    wanted = [t.detach().cpu().clone().requires_grad_(i == index) for i, t in enumerate(inputs)]
    x, w1, b1, w2, b2 = wanted
    expected = torch.relu(x @ w1 + b1) @ w2 + b2
    actual = _kernels.mlp(*inputs)
    actual.sum().backward()
    expected.sum().backward()
    close(inputs[index].grad, wanted[index].grad)
    assert all(t.grad is None for i, t in enumerate(inputs) if i != index)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 127, 128, 129, 700])
def test_mlp_backward_row_chunks_repeat_bitwise(device, dtype, rows):
    # more than 128 rows: the bias gradients are summed in row chunks through context scratch
    torch.manual_seed(rows)
    x = torch.randn((rows, 19), dtype=dtype, device=device)
    w1 = torch.randn((19, 70), dtype=dtype, device=device)
    w2 = torch.randn((70, 9), dtype=dtype, device=device)
    hidden = torch.relu(torch.randn((rows, 70), dtype=dtype, device=device))
    gradient = torch.randn((rows, 9), dtype=dtype, device=device)
    first = _kernels.mlp_backward(x, w1, w2, hidden, gradient)
    again = _kernels.mlp_backward(x, w1, w2, hidden, gradient)
    g, h = gradient.double().cpu(), hidden.double().cpu()
    dh = (g @ w2.double().cpu().T) * (h > 0)
    expected = (dh @ w1.double().cpu().T, x.double().cpu().T @ dh, dh.sum(0), h.T @ g, g.sum(0))
    for got, repeat, want in zip(first, again, expected):
        assert torch.equal(got, repeat)
        rtol, atol = (2e-5, 2e-5) if dtype == torch.float32 else (2e-13, 1e-12)
        torch.testing.assert_close(got.cpu(), want.to(dtype), rtol=rtol, atol=atol)
    only = _kernels.mlp_backward(x, w1, w2, hidden, gradient, (False, False, False, True, True))
    assert only[:3] == (None, None, None) and torch.equal(only[3], first[3]) and torch.equal(only[4], first[4])


def _relative(actual, expected):
    expected = expected.double().cpu()
    return float((actual.double().cpu() - expected).norm() / expected.norm().clamp_min(1e-300))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("queries,keys,depth,values",
                         [(64, 2048, 64, 64), (64, 8192, 64, 1024), (64, 2048, 512, 64)])
def test_attention_whose_products_divide_k_keeps_the_scores_intact(device, dtype, queries, keys, depth, values):
    # The planner divides K of these products over workgroups (planes in the context's arena) while
    # the score matrix lives in the same arena: first call on a context of its own (a new stream
    # gets one, so the arena starts empty and must be sized for both at once), then warmed.
    torch.manual_seed(queries + keys + depth + values)
    q = torch.randn((queries, depth), dtype=dtype) * 0.3
    k = torch.randn((keys, depth), dtype=dtype) * 0.3
    v = torch.randn((keys, values), dtype=dtype)
    expected = torch.softmax((q.double() @ k.double().T) * 0.25, dim=-1) @ v.double()
    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        qd, kd, vd = q.to(device), k.to(device), v.to(device)
        results = [_kernels.attention(qd, kd, vd, scale=0.25) for _ in range(3)]
        stream.synchronize()
    bar = 1e-5 if dtype == torch.float32 else 1e-13
    for result in results:
        assert _relative(result, expected) <= bar
        assert torch.equal(result, results[0])


@pytest.mark.parametrize("dtype", DTYPES)
def test_mlp_backward_whose_products_divide_k_keeps_the_partials_intact(device, dtype):
    # rows=1024, hidden=256, outputs=64: dw2 = h^T grad divides K over workgroups while the bias
    # gradients' row-chunk partials are held in the same arena
    torch.manual_seed(1024)
    rows, inputs, hidden_width, outputs = 1024, 96, 256, 64
    stream = torch.cuda.Stream(device)
    with torch.cuda.stream(stream):
        x = torch.randn((rows, inputs), dtype=dtype, device=device)
        w1 = torch.randn((inputs, hidden_width), dtype=dtype, device=device) * 0.1
        w2 = torch.randn((hidden_width, outputs), dtype=dtype, device=device) * 0.1
        hidden = torch.relu(torch.randn((rows, hidden_width), dtype=dtype, device=device))
        gradient = torch.randn((rows, outputs), dtype=dtype, device=device)
        runs = [_kernels.mlp_backward(x, w1, w2, hidden, gradient) for _ in range(3)]
        stream.synchronize()
    g, h = gradient.double().cpu(), hidden.double().cpu()
    dh = (g @ w2.double().cpu().T) * (h > 0)
    expected = (dh @ w1.double().cpu().T, x.double().cpu().T @ dh, dh.sum(0), h.T @ g, g.sum(0))
    bar = 1e-5 if dtype == torch.float32 else 1e-13
    for run in runs:
        for got, first, want in zip(run, runs[0], expected):
            assert torch.equal(got, first)
            assert _relative(got, want) <= bar


def test_c_abi_validation_counters_and_empty_shapes(device):
    native = _native.context(device)
    library = _native.library()
    handle = native.handle
    buffer = torch.zeros(64, dtype=torch.float32, device=device)
    p = ct.c_void_p(buffer.data_ptr())
    before = _native.stats(device)
    # negative sizes, unknown dtype, missing operands, aliased MLP outputs
    assert library.camblas_cuda_affine(handle, 0, -1, 2, 2, p, p, p, 0, p) != 0
    assert b"affine" in library.camblas_cuda_error(handle)
    assert library.camblas_cuda_affine(handle, 2, 2, 2, 2, p, p, p, 0, p) != 0
    assert library.camblas_cuda_affine(handle, 0, 2, 2, 2, p, p, None, 0, p) != 0
    assert library.camblas_cuda_affine(handle, 0, 2, 2, 2, None, p, p, 0, p) != 0
    assert library.camblas_cuda_mlp(handle, 0, 2, 2, 2, 2, p, p, p, p, p, p, p) != 0
    assert b"alias" in library.camblas_cuda_error(handle)
    assert library.camblas_cuda_attention(handle, 0, 2, -2, 2, 2, ct.c_double(1), p, p, p, p) != 0
    assert library.camblas_cuda_attention(handle, 3, 2, 2, 2, 2, ct.c_double(1), p, p, p, p) != 0
    assert library.camblas_cuda_attention(handle, 0, 2, 2, 2, 2, ct.c_double(1), p, p, None, p) != 0
    assert library.camblas_cuda_mlp_backward(handle, 0, 2, 2, 2, 2, p, p, p, p, None, p, p, p, p, p, p) != 0
    assert library.camblas_cuda_mlp_backward(handle, 0, 2, 2, 2, 2, p, p, p, p, p, None, p, None, None, None, None) != 0
    # empty shapes succeed without touching anything
    assert library.camblas_cuda_affine(handle, 0, 0, 2, 2, None, None, None, 0, None) == 0
    assert library.camblas_cuda_attention(handle, 1, 0, 2, 2, 2, ct.c_double(1), None, None, None, None) == 0
    # inner == 0: the result is the bias (x and weight may be absent)
    bias = torch.tensor([1.0, -2.0, 3.0], device=device)
    out = torch.full((2, 3), 7.0, device=device)
    assert library.camblas_cuda_affine(handle, 0, 2, 0, 3, None, None, ct.c_void_p(bias.data_ptr()), 1,
                                       ct.c_void_p(out.data_ptr())) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, torch.relu(bias).expand(2, 3))
    middle = _native.stats(device)
    assert middle["affine"] == before["affine"] + 1
    x = torch.randn((4, 5), device=device)
    _kernels.mlp(x, torch.randn((5, 6), device=device), torch.randn(6, device=device),
                 torch.randn((6, 3), device=device), torch.randn(3, device=device))
    _kernels.attention(x, x, x)
    _kernels.mlp_backward(x, torch.randn((5, 6), device=device), torch.randn((6, 3), device=device),
                          torch.randn((4, 6), device=device), torch.randn((4, 3), device=device))
    after = _native.stats(device)
    assert after["affine"] == middle["affine"] + 2
    assert after["attention"] == middle["attention"] + 1
    assert after["backward"] == middle["backward"] + 1


@pytest.mark.parametrize("dtype", DTYPES)
def test_captured_attention_survives_scratch_growth(device, dtype):
    # a captured graph keeps using the score storage it was captured with after a larger call has
    # made the context allocate a new one (ref: tests/test_cuda.py:511-538)
    torch.manual_seed(3)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        q = torch.randn((17, 16), device=device, dtype=dtype)
        k = torch.randn((513, 16), device=device, dtype=dtype)
        v = torch.randn((513, 13), device=device, dtype=dtype)
        for _ in range(3):
            _kernels.attention(q, k, v)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        captured = _kernels.attention(q, k, v)
    with torch.cuda.stream(stream):
        larger = [torch.randn(shape, device=device, dtype=dtype) for shape in ((129, 16), (4097, 16), (4097, 13))]
        _kernels.attention(*larger)
        for _ in range(3):
            q.add_(0.1)
            v.mul_(0.9)
            graph.replay()
            stream.synchronize()
            expected = torch.softmax((q.double().cpu() @ k.double().cpu().T) / 4, dim=-1) @ v.double().cpu()
            close(captured, expected)
    stream.synchronize()
    torch.cuda.current_stream().wait_stream(stream)
    graph.reset()


def test_scratch_growth_is_refused_during_capture(device):
    # (ref: src/cuda/backend.cu:399-426) a first large call inside a capture cannot allocate
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        q = torch.randn((8, 16), device=device)
        _kernels.attention(q, q, q)  # creates the context of this stream
        big_q = torch.randn((3000, 16), device=device)
        big_k = torch.randn((3100, 16), device=device)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="scratch"):
        with torch.cuda.graph(graph, stream=stream):
            _kernels.attention(big_q, big_k, big_k)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        out = _kernels.attention(big_q, big_k, big_k)  # fine outside a capture
    stream.synchronize()
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_captured_mlp_training_step_replays_with_changed_inputs(device, dtype):
    # forward and backward captured once, replayed after the inputs change and after a larger call
    # has grown the context's scratch (ref: tests/test_cuda.py:540-583)
    torch.manual_seed(4)
    shapes = ((129, 17), (17, 23), (23,), (23, 13), (13,))
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        inputs = [torch.randn(shape, device=device, dtype=dtype, requires_grad=True) for shape in shapes]
        for _ in range(3):
            for value in inputs:
                value.grad = None
            _kernels.mlp(*inputs).square().mean().backward()
        for value in inputs:
            value.grad = None
        with torch.cuda.graph(graph, stream=stream):
            output = _kernels.mlp(*inputs)
            output.square().mean().backward()
        larger = [torch.randn(shape, device=device, dtype=dtype, requires_grad=True)
                  for shape in ((513, 17), (17, 23), (23,), (23, 13), (13,))]
        _kernels.mlp(*larger).square().mean().backward()
        for _ in range(3):
            with torch.no_grad():
                inputs[0].add_(0.03)
                inputs[1].mul_(0.9)
                inputs[2].sub_(0.01)
            graph.replay()
            stream.synchronize()
            wanted = [value.detach().double().cpu().requires_grad_(True) for value in inputs]
            x, w1, b1, w2, b2 = wanted
            expected = torch.relu(x @ w1 + b1) @ w2 + b2
            expected.square().mean().backward()
            # outputs of size 30 from 23 terms: the absolute tolerance follows that size
            close(output.detach(), expected.detach(), magnitude=10)
            for actual, desired in zip(inputs, wanted):
                close(actual.grad, desired.grad, magnitude=10)
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph.reset()


def test_raw_affine_binding_writes_into_the_given_output(device):
    # the positional entry the reference's Python layer binds beside the autograd form
    # (ref: src/cuda/torch_bindings.cpp:738-775, :1227): x, weight, bias, relu, output, algorithm
    from camblas_amd import _native

    module = _native.tensor_module()
    generator = torch.Generator().manual_seed(12)
    x = torch.randn((9, 33), generator=generator).to(device)
    weight = torch.randn((33, 21), generator=generator).to(device)
    bias = torch.randn((21,), generator=generator).to(device)
    out = torch.full((9, 21), float("nan"), device=device)
    returned = module.affine(x, weight, bias, True, out, -1)
    assert returned.data_ptr() == out.data_ptr()
    close(out, torch.relu(x.double().cpu() @ weight.double().cpu() + bias.double().cpu()))
    fresh = module.affine(x, weight, bias, False, None, -1)
    close(fresh, x.double().cpu() @ weight.double().cpu() + bias.double().cpu())
