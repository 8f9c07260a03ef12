"""E8M0 block-scaled products through the binding with torch's native storage types
(float8_e4m3fn, float4_e2m1fn_x2, float8_e8m0fnu), after the reference's tests/test_quantized.py:
rejected metadata (:268-293), a captured product that reads fresh operands (:295-322, known
answers: 32 inputs of 1.0 times E2M1 1.5 = 48), captured grouped products that keep their weight
storage alive and follow changed selections (:473-508), and the C entry's dimension, null,
alignment, alias and empty-row rules (:510-544).
"""

import ctypes

import pytest
import torch

from camblas_amd import _native

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def binding():
    module = _native.tensor_module()
    assert module is not None
    return module


def operands(device, rows=1, outputs=8, inner=32, packed=True, block=32):
    # ref: tests/test_quantized.py:66-108
    x = (torch.randn(rows, inner, device=device) * 8).to(torch.float8_e4m3fn)
    if packed:
        weight = torch.randint(0, 256, (outputs, inner // 2), dtype=torch.uint8, device=device)
        weight = weight.view(torch.float4_e2m1fn_x2)
    else:
        weight = (torch.randn(outputs, inner, device=device) * 4).to(torch.float8_e4m3fn)
    sx = torch.randint(122, 129, (rows, inner // block), dtype=torch.uint8, device=device)
    sw = torch.randint(121, 128, (outputs if packed else (outputs + 31) // 32, inner // 32),
                       dtype=torch.uint8, device=device)
    return x, sx.view(torch.float8_e8m0fnu), weight, sw.view(torch.float8_e8m0fnu)


def test_invalid_shapes_dtypes_views_and_devices(binding, device):
    x, sx, weight, sw = operands(device)
    invalid = (
        (x.float(), sx, weight, sw),
        (x, sx.float(), weight, sw),
        (x.cpu(), sx, weight, sw),
        (x, sx, weight[:7], sw[:7]),
        (x, sx[:, :0], weight, sw),
        (x, sx, weight, sw[:7]),
        (x, sx, weight, sw.float()),
    )
    for arguments in invalid:
        with pytest.raises(ValueError):
            binding.quantized_matmul(*arguments)
    with pytest.raises(ValueError):
        binding.quantized_matmul(x, sx, weight, sw, activation_block=64)
    x2, sx2, weight2, sw2 = operands(device, 2, 8, 64)
    with pytest.raises(ValueError):
        binding.quantized_matmul(x2.view(torch.uint8).T.view(torch.float8_e4m3fn), sx2, weight2, sw2)
    with pytest.raises(ValueError):
        binding.quantized_matmul(x.float().requires_grad_().to(torch.float8_e4m3fn), sx, weight, sw)


def test_captured_product_reads_fresh_operands(binding, device):
    with torch.inference_mode():
        x, sx, weight, sw = operands(device)
        x.view(torch.uint8).zero_()
        sx.view(torch.uint8).fill_(127)
        sw.view(torch.uint8).fill_(127)
        weight.view(torch.uint8).fill_(0x22)
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream):
            before = binding.quantized_matmul(x, sx, weight, sw)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                output = binding.quantized_matmul(x, sx, weight, sw)
            x.view(torch.uint8).fill_(0x38)
            weight.view(torch.uint8).fill_(0x33)
            for _ in range(3):
                graph.replay()
                stream.synchronize()
                torch.testing.assert_close(output.cpu(), torch.full((1, 8), 48, dtype=torch.bfloat16),
                                           rtol=0, atol=0)
        assert (before == 0).all()
        graph.reset()


def test_captured_grouped_products_keep_weights_and_follow_selections(binding, device):
    with torch.inference_mode():
        x, sx, w0, s0 = operands(device, 2)
        _, _, w1, s1 = operands(device, 2)
        x = x.unsqueeze(0).expand(2, -1, -1).contiguous()
        sx = sx.unsqueeze(0).expand(2, -1, -1).contiguous()
        x.view(torch.uint8).fill_(0x38)
        sx.view(torch.uint8).fill_(127)
        for weight, scale in ((w0, s0), (w1, s1)):
            weight.view(torch.uint8).fill_(0x22)
            scale.view(torch.uint8).fill_(127)
        pool = binding.QuantizedGroups([w0, w1], [s0, s1])
        active = torch.tensor([1, 0], device=device, dtype=torch.int32)
        counts = torch.tensor([2, 1], device=device, dtype=torch.int32)
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream):
            pool.matmul(x, sx, active, counts)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                output = pool.matmul(x, sx, active, counts)
            x.view(torch.uint8).fill_(0x30)
            w0.view(torch.uint8).fill_(0x33)
            counts.copy_(torch.tensor([1, 2], device=device, dtype=torch.int32))
            del w0, w1, s0, s1
            graph.replay()
        stream.synchronize()
        # group 0 reads weight set 1 (nibble 2 = 1.0): 32 * 0.5 * 1.0 = 16 for its one valid row;
        # group 1 reads set 0 (now nibble 3 = 1.5): 32 * 0.5 * 1.5 = 24 for both rows
        expected = torch.tensor([[16, 0], [24, 24]], dtype=torch.bfloat16).unsqueeze(-1).expand(2, 2, 8)
        torch.testing.assert_close(output.cpu(), expected, rtol=0, atol=0)
        graph.reset()


def test_c_entry_dimensions_alignment_aliases_and_empty_rows(device):
    library = _native.library()
    operation = library.camblas_cuda_quantized_matmul
    context = _native.context(device).handle
    x, sx, weight, sw = operands(device)
    output = torch.empty((1, 8), device=device, dtype=torch.bfloat16)
    dimensions = [1, 1, 8, 32, 32]
    pointers = [t.data_ptr() for t in (x, sx, weight, sw, output)]

    def call(sizes, addresses):
        return operation(context, *sizes, *(ctypes.c_void_p(a) if a else None for a in addresses))

    assert call([1, 0, 8, 32, 32], [0] * 5) == 0  # no rows: nothing is touched
    for index, bad in ((0, 2), (1, -1), (1, 65536), (2, 7), (3, 31), (4, 64)):
        invalid = dimensions.copy()
        invalid[index] = bad
        assert call(invalid, pointers) != 0
    for index in range(5):
        invalid = pointers.copy()
        invalid[index] = 0
        assert call(dimensions, invalid) != 0
    for index in (0, 2, 4):
        invalid = pointers.copy()
        invalid[index] += 1
        assert call(dimensions, invalid) != 0
    for pointer in pointers[:4]:
        assert call(dimensions, pointers[:4] + [pointer]) != 0
    assert call(dimensions, pointers) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(1152, 5120), (1792, 5120), (4096, 1280), (5120, 2048), (5120, 576),
                                   (8192, 1280), (25600, 6144)])
@pytest.mark.parametrize("sample", [0, 1])
def test_block32_products_on_the_plugin_shapes(binding, device, shape, sample):
    # ref: tests/test_sglang.py:361-470 without its Triton yardstick: power-of-two block scales,
    # padded / column-major scale storage, the fused BF16 quantiser against the CPU recipe
    # (scale = smallest power of two >= amax/448), selected outputs rebuilt in FP64 and held to
    # the reference's rounding unit max(|value|, 1) / 128
    n, k = shape
    torch.manual_seed(413 + sample)
    a = (torch.randn(1, k, device=device) * 0.75).to(torch.float8_e4m3fn)
    b = (torch.randn(n, k, device=device) * 0.6).to(torch.float8_e4m3fn)
    a_scale = (2.0 ** torch.randint(-3, 2, (1, k // 32), device=device)).float()
    b_scale = (2.0 ** torch.randint(-3, 2, (n // 32, k // 32), device=device)).float()
    if sample == 1:
        storage = torch.empty((k // 32, 4), device=device)
        a_scale = storage[:, 0].view(1, -1)
        a_scale.uniform_(0.001, 0.08)
        b_scale = b_scale.T.contiguous().T

    def rebuilt(actual, a, a_scale):
        indices = torch.arange(0, n, max(1, n // 16), device=device)[:16]
        decoded_a = a.float().cpu().double() * a_scale.cpu().double().repeat_interleave(32, dim=1)
        decoded_b = b.index_select(0, indices).float().cpu().double()
        decoded_b *= b_scale.index_select(0, indices // 32).cpu().double().repeat_interleave(32, dim=1)
        reference = decoded_a @ decoded_b.T
        received = actual.index_select(1, indices).float().cpu()
        assert ((reference - received).abs() <= reference.abs().clamp_min(1.0) / 128).all()

    native = binding.fp8_decode(a, a_scale, b, b_scale)
    assert native.shape == (1, n) and native.dtype == torch.bfloat16
    rebuilt(native, a, a_scale)
    if k <= 8192:
        bf16 = (torch.randn(1, k, device=device) * (80 if sample else 0.75)).to(torch.bfloat16)
        fused = binding.fp8_linear(bf16, b, b_scale)
        values = bf16.float().cpu().view(1, k // 32, 32)
        raw = values.abs().amax(-1).clamp_min(1.0e-10) * (1.0 / 448.0)
        bits = raw.view(torch.int32).long()
        exponent = ((bits >> 23) & 255) - 127 + ((bits & 0x7FFFFF) != 0)
        cpu_scales = torch.ldexp(torch.ones_like(raw), exponent.int())
        cpu_q = (values / cpu_scales.unsqueeze(-1)).reshape(1, k).to(torch.float8_e4m3fn)
        # the fused kernel must equal the two-step path on the CPU-quantised token bit for bit
        two_step = binding.fp8_decode(cpu_q.to(device), cpu_scales.to(device), b, b_scale)
        assert torch.equal(fused.view(torch.int16), two_step.view(torch.int16))
        rebuilt(fused, cpu_q.to(device), cpu_scales.to(device))
