"""The compiled ATen binding (_camblas_cuda_torch) on the GPU: explicit products with transpose
views, out/alpha/beta and autograd, the linear wrapper, and the dispatcher override of
torch.mm / mm.out / addmm with its fall-back rules (ref: src/cuda/torch_bindings.cpp:146-271,
src/cuda/torch_backend.cuh:7-88; strategy of tests/test_torch_backend.py and tests/test_linear.py
in the reference: FP64 product of the same operands, tolerance by storage type, dispatch counters).

This file sorts last on purpose: installing the backend cannot be undone inside a process.
Tolerances: relative Frobenius <= 1e-5 (FP32), 1e-12 (FP64), 1e-2 (BF16) against the FP64 product.
"""

import pytest
import torch
import torch.nn.functional as F

from camblas_amd import _native

pytestmark = pytest.mark.gpu
BAR = {torch.float32: 1e-5, torch.float64: 1e-12, torch.bfloat16: 1e-2}


@pytest.fixture(scope="module")
def binding():
    module = _native.tensor_module()
    assert module is not None, "camblas_amd/lib/_camblas_cuda_torch*.so is not built"
    return module


def error(got, want):
    got, want = got.double(), want.double()
    return ((got - want).norm() / want.norm().clamp_min(1e-300)).item()


def randn(shape, dtype, device, seed):
    generator = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(shape, generator=generator, dtype=torch.float64).to(dtype).to(device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("views", ["nn", "tn", "nt", "strided"])
def test_matmul_public_layouts(binding, device, dtype, views):
    m, k, n = 45, 96, 70
    a = randn((m, k), dtype, device, 1)
    b = randn((k, n), dtype, device, 2)
    if views == "tn":
        a = randn((k, m), dtype, device, 1).t()
    elif views == "nt":
        b = randn((n, k), dtype, device, 2).t()
    elif views == "strided":
        a = randn((m, 2 * k), dtype, device, 1)[:, ::2]      # neither stride is 1: copied
        b = randn((k, n + 8), dtype, device, 2)[:, :n]        # padded rows: used in place
    got = binding.matmul_public(a, b)
    assert got.shape == (m, n) and got.dtype == dtype and got.is_contiguous()
    assert error(got, a.double() @ b.double()) <= BAR[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matmul_public_out_alpha_beta(binding, device, dtype):
    a, b = randn((33, 64), dtype, device, 3), randn((64, 40), dtype, device, 4)
    c = randn((33, 40), dtype, device, 5)
    want = 0.5 * (a.double() @ b.double()) - 1.5 * c.double()
    version = c._version
    out = binding.matmul_public(a, b, out=c, alpha=0.5, beta=-1.5)
    assert out.data_ptr() == c.data_ptr() and c._version == version + 1
    assert error(c, want) <= BAR[dtype]
    with pytest.raises(ValueError, match="alias"):
        binding.matmul_public(a, b, out=a.view(-1)[: 33 * 40].view(33, 40))
    with pytest.raises(ValueError, match="beta requires"):
        binding.matmul_public(a, b, beta=1.0)
    with pytest.raises(ValueError, match="same device and dtype"):
        binding.matmul_public(a, b.float() if dtype != torch.float32 else b.double())
    with pytest.raises(ValueError, match="GPU"):
        binding.matmul_public(a.cpu(), b.cpu())


def test_matmul_public_autograd(binding, device):
    a = randn((24, 48), torch.float32, device, 6).requires_grad_()
    b = randn((48, 16), torch.float32, device, 7).requires_grad_()
    g = randn((24, 16), torch.float32, device, 8)
    binding.matmul_public(a, b).backward(g)
    assert error(a.grad, g.double() @ b.detach().double().t()) <= 1e-5
    assert error(b.grad, a.detach().double().t() @ g.double()) <= 1e-5
    with pytest.raises(ValueError, match="Autograd matmul"):
        binding.matmul_public(a, b, alpha=2.0)
    # second derivative goes through the same entry
    a2 = randn((6, 5), torch.float64, device, 9).requires_grad_()
    b2 = randn((5, 4), torch.float64, device, 10).requires_grad_()
    assert torch.autograd.gradcheck(lambda u, v: binding.matmul_public(u, v), (a2, b2))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_dense_helpers_with_gradients(binding, device, dtype):
    # affine / MLP / attention of the binding against CPU FP64 autograd
    # (ref: tests/test_cuda.py:356-378, :485-509, :677-698, :1264-1283)
    tight = dict(rtol=1e-5, atol=3e-6) if dtype == torch.float32 else dict(rtol=2e-13, atol=3e-14)
    shapes = ((11, 17), (17, 23), (23,), (23, 13), (13,))
    inputs = [randn(shape, dtype, device, 40 + i).requires_grad_() for i, shape in enumerate(shapes)]
    wanted = [t.detach().double().cpu().requires_grad_() for t in inputs]
    x, w1, b1, w2, b2 = wanted
    expected = torch.relu(x @ w1 + b1) @ w2 + b2
    actual = binding.mlp_public(*inputs)
    torch.testing.assert_close(actual.cpu(), expected.to(dtype), **tight)
    actual.square().sum().backward()
    expected.square().sum().backward()
    for tensor, oracle in zip(inputs, wanted):
        torch.testing.assert_close(tensor.grad.cpu(), oracle.grad.to(dtype), **tight)
    output, hidden = binding.mlp(*(t.detach() for t in inputs))
    torch.testing.assert_close(hidden.cpu(), torch.relu(x @ w1 + b1).detach().to(dtype), **tight)
    only = binding.mlp_backward(inputs[0].detach(), inputs[1].detach(), inputs[3].detach(), hidden,
                                torch.ones_like(output), [False, False, True, False, True])
    assert only[0] is None and only[1] is None and only[3] is None
    torch.testing.assert_close(only[4].cpu(), torch.full((13,), 11.0, dtype=dtype), **tight)
    for relu in (False, True):
        got = binding.affine_public(inputs[0].detach(), inputs[1].detach(), inputs[2].detach(), relu=relu)
        want = (x @ w1 + b1).detach()
        torch.testing.assert_close(got.cpu(), (torch.relu(want) if relu else want).to(dtype), **tight)
    q, k, v = (randn(shape, dtype, device, 50 + i) for i, shape in enumerate(((13, 17), (19, 17), (19, 23))))
    want = torch.softmax(q.double().cpu() @ k.double().cpu().T / 17 ** 0.5, -1) @ v.double().cpu()
    torch.testing.assert_close(binding.attention_public(q, k, v).cpu(), want.to(dtype), **tight)
    torch.testing.assert_close(binding.attention(q, k, v, 0.25).cpu(),
                               (torch.softmax(q.double().cpu() @ k.double().cpu().T * 0.25, -1)
                                @ v.double().cpu()).to(dtype), **tight)
    if dtype == torch.float64:
        small = [randn(shape, dtype, device, 60 + i).requires_grad_() for i, shape in
                 enumerate(((3, 4), (4, 5), (5,)))]
        assert torch.autograd.gradcheck(lambda a, b, c: binding.affine_public(a, b, c, relu=True), small)
        assert torch.autograd.gradgradcheck(lambda a, b, c: binding.affine_public(a, b, c), small)
        qkv = [randn(shape, dtype, device, 70 + i).requires_grad_() for i, shape in
               enumerate(((3, 4), (5, 4), (5, 2)))]
        assert torch.autograd.gradcheck(lambda a, b, c: binding.attention_public(a, b, c), qkv)
    with pytest.raises(ValueError, match="affine"):
        binding.affine_public(inputs[0], inputs[1].t(), inputs[2])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_public(binding, device, dtype):
    x = randn((3, 5, 256), dtype, device, 11)
    w = randn((72, 256), dtype, device, 12)
    bias = randn((72,), dtype, device, 13)
    got = binding.linear_public(x, w, bias)
    assert got.shape == (3, 5, 72)
    want = x.double() @ w.double().t() + bias.double()
    assert error(got, want) <= 1.5 * BAR[dtype]
    assert error(binding.linear_public(x[0, 0], w), x[0, 0].double() @ w.double().t()) <= BAR[dtype]
    with pytest.raises(ValueError, match="linear requires"):
        binding.linear_public(x, w[:, :100])


def test_fusion_entries(binding, device):
    x = randn((7, 512), torch.bfloat16, device, 14)
    gate_w, up_w = randn((384, 512), torch.bfloat16, device, 15) * 0.05, randn((384, 512), torch.bfloat16, device, 16) * 0.05
    down_w = randn((512, 384), torch.bfloat16, device, 17) * 0.05
    gate, up = x.double() @ gate_w.double().t(), x.double() @ up_w.double().t()
    want = (F.silu(gate) * up) @ down_w.double().t()
    assert error(binding.gated_mlp(x, gate_w, up_w, down_w), want) <= 2e-2
    q, k, v = binding.qkv_linear(x, gate_w, up_w, gate_w)
    assert error(q, gate) <= 1e-2 and error(k, up) <= 1e-2 and torch.equal(q, v)
    weight = randn((512,), torch.bfloat16, device, 18) * 0.1 + 1
    residual = randn((7, 512), torch.bfloat16, device, 19)
    added, normed = binding.add_rms_norm(x, residual, weight, 1e-5)
    assert torch.equal(added, x + residual)
    a64 = added.double()
    want = a64 * torch.rsqrt((a64 * a64).mean(-1, keepdim=True) + 1e-5) * weight.double()
    assert error(normed, want) <= 1e-2
    assert error(binding.rms_norm(added, weight, 1e-5), want) <= 1e-2
    assert error(binding.silu_multiply(x, residual), F.silu(x.double()) * residual.double()) <= 1e-2
    assert error(binding.swiglu(x, residual), F.silu(x.double()) * residual.double()) <= 1e-2
    with pytest.raises(ValueError, match="inference only"):
        binding.silu_multiply(x.clone().requires_grad_(), residual)


def test_block32_fp8_entries(binding, device):
    # the binding's fp8_decode / fp8_linear against the ctypes path (same library entry points) and
    # the reference's argument errors (ref: tests/test_quantized.py:218-240)
    from camblas_amd import _kernels

    assert binding.fp8_decode_supported(device.index or 0) and binding.fp8_decode_supported()
    n, k = 64, 256
    x = (torch.randn(1, k, device=device) * 2).to(torch.float8_e4m3fn)
    w = torch.randn(n, k, device=device).to(torch.float8_e4m3fn)
    sx = torch.rand(1, k // 32, device=device) + 0.5
    sw = torch.rand(n // 32, k // 32, device=device) + 0.5
    assert torch.equal(binding.fp8_decode(x, sx, w, sw), _kernels.fp8_decode(x, sx, w, sw))
    token = torch.randn(1, k, device=device).bfloat16()
    assert torch.equal(binding.fp8_linear(token, w, sw), _kernels.fp8_linear(token, w, sw))
    dequantised = (x.float().view(-1, 32) * sx.view(-1, 1)).view(1, k).double() @ (
        w.float().view(n // 32, 32, k // 32, 32) * sw.view(n // 32, 1, k // 32, 1)).view(n, k).double().t()
    assert error(binding.fp8_decode(x, sx, w, sw), dequantised) <= 1e-2
    for operands in ((x.expand(2, -1).contiguous(), sx.expand(2, -1).contiguous(), w, sw),
                     (x, sx[:, :2], w, sw), (x, sx[:, :1].expand_as(sx), w, sw)):
        with pytest.raises(ValueError):
            binding.fp8_decode(*operands)
    for operands in ((token.expand(2, -1).contiguous(), w, sw), (token, w, sw[:, :2]),
                     (token.clone().requires_grad_(), w, sw)):
        with pytest.raises(ValueError):
            binding.fp8_linear(*operands)


def test_quantized_groups_route_multiply_reduce(binding, device):
    # an expert-parallel slice end to end through the binding (ref: tests/test_quantized.py:324-472
    # strategy: route, grouped product, ordered reduction, each against an independent restatement)
    import numpy as np

    import oracle

    tokens, choices, experts_total, rows, inner, outputs = 12, 2, 6, 8, 128, 64
    generator = torch.Generator(device="cpu").manual_seed(5)
    chosen = torch.stack([torch.randperm(experts_total, generator=generator)[:choices]
                          for _ in range(tokens)]).to(device)                      # int64 [tokens, choices]
    active = torch.tensor([4, 1, 3], dtype=torch.int32, device=device)             # local experts served
    slots, reverse, counts = binding.route_groups(chosen, active, first_expert=0, rows=rows)
    want_counts, want_slots, want_reverse = oracle.route_groups(chosen.cpu().numpy(), active.cpu().numpy(), 0, rows)
    assert np.array_equal(slots.cpu().numpy(), want_slots) and np.array_equal(counts.cpu().numpy(), want_counts)
    assert np.array_equal(reverse.cpu().numpy(), want_reverse)

    hidden = (torch.randn(tokens, inner, generator=generator) * 4).to(torch.float8_e4m3fn).to(device)
    gathered = torch.zeros((3, rows, inner), dtype=torch.float8_e4m3fn, device=device)
    valid = slots >= 0
    gathered.view(torch.uint8)[valid] = hidden.view(torch.uint8)[torch.div(slots[valid], choices, rounding_mode="floor").long()]
    gathered_scale = torch.full((3, rows, inner // 32), 127, dtype=torch.uint8, device=device).view(torch.float8_e8m0fnu)
    weights = [(torch.randn(outputs, inner, generator=generator) * 2).to(torch.float8_e4m3fn).to(device)
               for _ in range(experts_total)]
    scales = [torch.randint(124, 129, (outputs // 32, inner // 32), generator=generator, dtype=torch.uint8)
              .to(device).view(torch.float8_e8m0fnu) for _ in range(experts_total)]
    group = binding.QuantizedGroups(weights, scales)
    products = group.matmul(gathered, gathered_scale, active, torch.clamp(counts, max=rows))
    assert products.shape == (3, rows, outputs) and products.dtype == torch.bfloat16
    for g, expert in enumerate(active.tolist()):
        count = min(int(counts[g]), rows)
        want = oracle.mx_matmul_f64(gathered[g].view(torch.uint8).cpu().numpy(), gathered_scale[g].view(torch.uint8).cpu().numpy(),
                                    weights[expert].view(torch.uint8).cpu().numpy(), scales[expert].view(torch.uint8).cpu().numpy())
        got = products[g].float().cpu().numpy()
        assert (np.abs(got[:count] - want[:count]) <= 0.02 + 0.008 * np.abs(want[:count])).all()
        assert not got[count:].any()
    single = binding.quantized_matmul(gathered[0], gathered_scale[0], weights[4], scales[4])
    assert torch.equal(single[: int(counts[0])], products[0][: int(counts[0])])
    summed = binding.reduce_groups(products, chosen, reverse)
    want_sum = oracle.reduce_groups(products.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1, outputs),
                                    chosen.cpu().numpy(), reverse.cpu().numpy())
    assert np.array_equal(summed.cpu().numpy(), want_sum)
    with pytest.raises(ValueError):
        binding.quantized_matmul(gathered[0], gathered_scale[0], weights[4], scales[4], activation_block=128)
    with pytest.raises(ValueError):
        binding.route_groups(chosen.int(), active, first_expert=0, rows=rows)


def test_backend_override_routes_and_falls_back(binding, device):
    binding.install_torch_backend(_native.ALGORITHMS["lt"])
    binding.install_torch_backend(_native.ALGORITHMS["lt"])  # idempotent

    def dispatched(run):
        before = sum(binding.stats_all(device.index or 0, False).values())
        result = run()
        torch.cuda.synchronize()
        return result, sum(binding.stats_all(device.index or 0, False).values()) - before

    # BF16 and FP32 products, transposed views, F.linear with and without bias
    a, b = randn((64, 256), torch.bfloat16, device, 20), randn((256, 48), torch.bfloat16, device, 21)
    got, count = dispatched(lambda: torch.mm(a, b))
    assert count == 1 and error(got, a.double() @ b.double()) <= 1e-2
    w, bias = randn((48, 256), torch.bfloat16, device, 22), randn((48,), torch.bfloat16, device, 23)
    got, count = dispatched(lambda: F.linear(a.view(4, 16, 256), w, bias))
    assert count == 1 and got.shape == (4, 16, 48)
    assert error(got, a.double().view(4, 16, 256) @ w.double().t() + bias.double()) <= 1e-2
    got, count = dispatched(lambda: a @ w.t())
    assert count == 1 and error(got, a.double() @ w.double().t()) <= 1e-2
    # BF16 addmm for every way a bias broadcasts: rows and full matrices with unit stride along the
    # output features are read by the product itself, the other forms are spread over the output
    # first; either way one product is counted and alpha * a b + beta * bias is rounded once
    product = a.double() @ w.double().t()
    wide = randn((64, 96), torch.bfloat16, device, 27)
    forms = {"row": bias, "row matrix": bias.view(1, 48), "full": wide[:, :48].contiguous(), "pitched": wide[:, 48:],
             "column": wide[:, :1], "scalar": wide[0, 0], "strided": wide.t()[:48, :1].t().expand(64, 48)}
    for name, form in forms.items():
        got, count = dispatched(lambda: torch.addmm(form, a, w.t(), beta=0.5, alpha=2.0))
        assert count == 1, name
        want = 2.0 * product + 0.5 * form.double()
        assert error(got, want) <= 1e-2, name
        assert (got.float() - want.float()).abs().max() <= 2.0**-7 * want.abs().max(), name
    previous = torch.backends.cuda.matmul.allow_tf32
    try:
        torch.backends.cuda.matmul.allow_tf32 = False
        a32, b32 = randn((50, 80), torch.float32, device, 24), randn((80, 30), torch.float32, device, 25)
        got, count = dispatched(lambda: torch.mm(a32, b32))
        assert count == 1 and error(got, a32.double() @ b32.double()) <= 1e-5
        out = torch.empty((50, 30), device=device)
        _, count = dispatched(lambda: torch.mm(a32, b32, out=out))
        assert count == 1 and error(out, a32.double() @ b32.double()) <= 1e-5
        # addmm: beta scales the broadcast bias; beta = 0 never reads it
        row = randn((30,), torch.float32, device, 26)
        got, count = dispatched(lambda: torch.addmm(row, a32, b32, beta=0.5, alpha=2.0))
        assert count == 1 and error(got, 2.0 * (a32.double() @ b32.double()) + 0.5 * row.double()) <= 1e-5
        poisoned = torch.full((50, 30), float("nan"), device=device)
        got, count = dispatched(lambda: torch.addmm(poisoned, a32, b32, beta=0.0))
        assert count == 1 and torch.isfinite(got).all()
        # autograd derives its products from mm, so they are routed as well
        left = a32.clone().requires_grad_()
        _, count = dispatched(lambda: torch.mm(left, b32).sum().backward())
        assert count == 2 and error(left.grad, torch.ones(50, 30, device=device).double() @ b32.double().t()) <= 1e-5
        # fall-backs keep ATen's result and do not touch the library: reduced-precision FP32
        # allowed by the caller, other dtypes, empty operands
        torch.backends.cuda.matmul.allow_tf32 = True
        got, count = dispatched(lambda: torch.mm(a32, b32))
        assert count == 0 and error(got, a32.double() @ b32.double()) <= 1e-2
        torch.backends.cuda.matmul.allow_tf32 = False
        half = a32.half()
        got, count = dispatched(lambda: torch.mm(half, b32.half()))
        assert count == 0 and got.dtype == torch.float16
        got, count = dispatched(lambda: torch.mm(a32[:0], b32))
        assert count == 0 and got.shape == (0, 30)
        got, count = dispatched(lambda: torch.mm(a32[:, :0], b32[:0]))
        assert count == 0 and got.shape == (50, 30) and not got.any()
    finally:
        torch.backends.cuda.matmul.allow_tf32 = previous


def test_stats_and_close(binding, device):
    index = device.index or 0
    a, b = randn((32, 64), torch.bfloat16, device, 30), randn((64, 32), torch.bfloat16, device, 31)
    binding.stats(index, True, 0)
    binding.matmul_public(a, b)
    counts = binding.stats(index, False, 0)
    assert set(counts) == set(_native.COUNTERS) and sum(counts.values()) == 1
    assert sum(binding.stats(index, True, 0).values()) == 1
    assert sum(binding.stats(index, False, 0).values()) == 0
    binding.close()
    torch.cuda.synchronize()
    # contexts are recreated on demand after close
    assert error(binding.matmul_public(a, b), a.double() @ b.double()) <= 1e-2
