"""The headline configurations at their full sizes, checked through properties that do not need a
full-size CPU product: sampled outputs against the oracle's FP64 accumulation (the sample covers
the first and last rows, tile seams and random positions), exact power-of-two scaling, token
permutation, independence of a token's result from its neighbours, zero and NaN propagation.

Also the decoder-layer decode step at its full size (batch 32, hidden 8192, 64 query / 8 KV heads of
128, FFN 28672, context 2048) against the whole oracle pipeline.

Shapes: BF16 decode x [M in {1, 8, 32}, 8192] . W [28672, 8192]^T; BF16 prefill x [4096, 8192] .
W [10240, 8192]^T with and without beta = 1; FP8 block-scaled A [M in {1, 16, 256, 4096}, 7168] .
W [18432, 7168]^T with 1x128 / 128x128 FP32 scales. Tolerances are the small-size tests': relative
Frobenius error <= 1e-2 against FP64 accumulation, and an element-wise bound of one BF16 rounding
plus 1e-4 of the largest output.
"""

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels
from helpers import bf16_values, from_device_bf16, from_device_fp8, rel_frobenius

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-2


def sample(count, size, seed, seams=()):
    """Sorted sample of indices below `size`: both ends, the seams given, and random ones."""
    rng = np.random.default_rng(seed)
    fixed = [0, 1, size - 2, size - 1] + [s + d for s in seams for d in (-1, 0) if 0 < s + d < size]
    picked = set(int(i) for i in fixed if 0 <= i < size)
    while len(picked) < min(count, size):
        picked.add(int(rng.integers(0, size)))
    return np.array(sorted(picked))


def close_to(got, want64):
    assert rel_frobenius(got, want64) <= TOLERANCE
    wanted = oracle.bf16_to_f32(oracle.f32_to_bf16(want64.astype(np.float32)))
    bound = 2.0 ** -7 * np.abs(wanted) + 1e-4 * np.abs(want64).max()
    assert (np.abs(got - wanted) <= bound).all()


def bf16_normal(shape, std, seed, device):
    generator = torch.Generator(device=device).manual_seed(seed)
    return (torch.randn(shape, generator=generator, device=device) * std).bfloat16()


@pytest.fixture(scope="module")
def up_projection(device):
    return bf16_normal((28672, 8192), 0.02, 9001, device)


@pytest.mark.parametrize("tokens", [1, 8, 32])
def test_bf16_decode_linear_28672x8192(device, up_projection, tokens):
    w = up_projection
    x = bf16_normal((tokens, 8192), 1.0, 9002 + tokens, device)
    y = _kernels.linear(x, w)
    assert y.shape == (tokens, 28672) and y.dtype == torch.bfloat16
    # sampled output features (rows of W): the workgroup seams at multiples of 112 rows included
    rows = sample(96, 28672, 1, seams=(112, 224, 28560, 14336))
    want = oracle.linear_bf16_f64(from_device_bf16(x), from_device_bf16(w[torch.from_numpy(rows).to(device)]))
    close_to(bf16_values(y)[:, rows], want)
    # scaling the input by a power of two scales every output exactly
    assert torch.equal(_kernels.linear(x * 4, w), y * 4)
    # a token's result depends on that token only: reversed batch, and the token alone
    if tokens > 1:
        assert torch.equal(_kernels.linear(x.flip(0).contiguous(), w), y.flip(0))
        alone = _kernels.linear(x[tokens - 1:].contiguous(), w)
        assert rel_frobenius(bf16_values(alone), bf16_values(y[tokens - 1:]).astype(np.float64)) <= 1e-2
    # zero input gives +0 everywhere; a NaN in one token poisons exactly that token
    assert not _kernels.linear(torch.zeros_like(x), w).view(torch.int16).any()
    poisoned = x.clone()
    poisoned[tokens - 1, 4097] = float("nan")
    out = _kernels.linear(poisoned, w)
    assert torch.isnan(out[tokens - 1]).all() and torch.equal(out[: tokens - 1], y[: tokens - 1])


def test_bf16_prefill_linear_4096x10240x8192(device):
    w = bf16_normal((10240, 8192), 0.02, 9101, device)
    x = bf16_normal((4096, 8192), 1.0, 9102, device)
    y = _kernels.linear(x, w)
    # sampled tokens against FP64, all 10240 features each (tile seams at 256 tokens / 320 rows)
    tokens = sample(12, 4096, 2, seams=(256, 2048, 3840))
    index = torch.from_numpy(tokens).to(device)
    want = oracle.linear_bf16_f64(from_device_bf16(x[index]), from_device_bf16(w))
    close_to(bf16_values(y[index]), want)
    assert torch.equal(_kernels.linear(x * 0.5, w), y * 0.5)
    # addmm with beta = 1 on a full-size C ~ N(0, 1): sampled tokens again
    c = bf16_normal((4096, 10240), 1.0, 9103, device)
    out = _kernels.matmul(x, w.t(), out=c.clone(), alpha=1.0, beta=1.0)
    want = want + bf16_values(c[index]).astype(np.float64)
    close_to(bf16_values(out[index]), want)
    # the addend read by the epilogue instead of first being cloned into the output: a full matrix
    # must reproduce the in-place form bit for bit, a bias row must hold the FP64 bar
    assert torch.equal(_kernels.addmm(c, x, w.t(), beta=1.0), out)
    row = bf16_normal((10240,), 1.0, 9104, device)
    biased = _kernels.addmm(row, x, w.t(), beta=1.0)
    close_to(bf16_values(biased[index]), want - bf16_values(c[index]).astype(np.float64) + bf16_values(row).astype(np.float64))
    # the same tokens as a small batch through the decode kernel agree to rounding
    small = _kernels.linear(x[index[:8]].contiguous(), w)
    assert rel_frobenius(bf16_values(small), bf16_values(y[index[:8]]).astype(np.float64)) <= 1e-2


def test_bf16_row_major_product_4096_cubed(device):
    # torch.mm(a, b) with a contiguous right operand ('N','N' through the ABI): the operand that is
    # not K-contiguous is transposed into the arena and the product runs on the linear-layer tiles.
    # Sampled rows against FP64; the transposed view of the same data ('T','N' directly, no copy)
    # must give the same bits, since the same kernel then multiplies the same K-contiguous rows.
    a = bf16_normal((4096, 4096), 1.0, 9110, device)
    b = bf16_normal((4096, 4096), 0.02, 9111, device)
    y = _kernels.matmul(a, b)
    rows = sample(10, 4096, 4, seams=(256, 2048))
    index = torch.from_numpy(rows).to(device)
    want = (a[index].double() @ b.double()).cpu().numpy()
    close_to(bf16_values(y[index]), want)
    assert torch.equal(_kernels.matmul(a, b.t().contiguous().t()), y)


@pytest.fixture(scope="module")
def fp8_weights(device):
    generator = torch.Generator(device=device).manual_seed(9201)
    # every byte pattern except the two NaN encodings
    w = torch.randint(0, 255, (18432, 7168), generator=generator, device=device, dtype=torch.uint8)
    w[w == 0x7F] = 0x7E
    scale = torch.exp(torch.empty((144, 56), device=device).uniform_(np.log(1e-4), np.log(1e-1), generator=generator))
    return w.view(torch.float8_e4m3fn), scale


@pytest.mark.parametrize("tokens", [1, 16, 256, 4096])
def test_fp8_block_linear_18432x7168(device, fp8_weights, tokens):
    w, w_scale = fp8_weights
    generator = torch.Generator(device=device).manual_seed(9300 + tokens)
    a = torch.randint(0, 255, (tokens, 7168), generator=generator, device=device, dtype=torch.uint8)
    a[a == 0x7F] = 0x7E
    a = a.view(torch.float8_e4m3fn)
    a_scale = torch.exp(torch.empty((tokens, 56), device=device).uniform_(np.log(1e-4), np.log(1e-1), generator=generator))
    out = _kernels.fp8_block_matmul(a, a_scale, w, w_scale)
    assert out.shape == (tokens, 18432) and out.dtype == torch.bfloat16
    # sampled tokens (all features) against the FP64 product of the dequantised operands
    picked = sample(4, tokens, 3, seams=(128, 256))
    index = torch.from_numpy(picked).to(device)
    want = oracle.fp8_block_matmul_f64(from_device_fp8(a[index]), a_scale[index].cpu().numpy(),
                                       from_device_fp8(w), w_scale.cpu().numpy())
    close_to(bf16_values(out[index]), want)
    # doubling every weight scale doubles every output exactly; so does doubling a token's scales
    assert torch.equal(_kernels.fp8_block_matmul(a, a_scale, w, w_scale * 2), out * 2)
    assert torch.equal(_kernels.fp8_block_matmul(a, a_scale * 0.5, w, w_scale), out * 0.5)
    # bit-exact block indexing: zeroing one 128 x 128 weight-scale block changes exactly the 128
    # features of that block row (and only through K group 17)
    masked = w_scale.clone()
    masked[77, 17] = 0
    changed = _kernels.fp8_block_matmul(a, a_scale, w, masked)
    differs = (changed.view(torch.int16) != out.view(torch.int16)).any(0).cpu().numpy()
    assert not differs[: 77 * 128].any() and not differs[78 * 128:].any() and differs[77 * 128: 78 * 128].any()
    # ... and zeroing one token's scale of group 17 changes exactly that token
    masked = a_scale.clone()
    masked[picked[-1], 17] = 0
    changed = _kernels.fp8_block_matmul(a, masked, w, w_scale)
    differs = (changed.view(torch.int16) != out.view(torch.int16)).any(1).cpu().numpy()
    assert differs[picked[-1]] and differs.sum() == 1
    # zero activations give +0; a NaN byte poisons exactly its token
    zero = torch.zeros_like(a.view(torch.uint8)).view(torch.float8_e4m3fn)
    assert not _kernels.fp8_block_matmul(zero, a_scale, w, w_scale).view(torch.int16).any()
    poisoned = a.view(torch.uint8).clone()
    poisoned[tokens - 1, 5000] = 0x7F
    result = _kernels.fp8_block_matmul(poisoned.view(torch.float8_e4m3fn), a_scale, w, w_scale)
    assert torch.isnan(result[tokens - 1]).all()
    assert torch.equal(result[: tokens - 1].view(torch.int16), out[: tokens - 1].view(torch.int16))


@pytest.mark.parametrize("tokens", [16, 4096])
def test_fp8_block_linear_on_the_distribution_the_configuration_states(device, tokens):
    # the configuration's own draw: x ~ N(0, 1) in BF16, quantised by the library's dynamic 1 x 128
    # quantiser; W ~ N(0, 0.02) quantised per 128 x 128 block to E4M3 with scale = amax / 448 (here
    # with PyTorch's own cast, an independent codec). Checked twice: against the FP64 product of the
    # dequantised operands (the kernel's own bar) and against the FP64 product of the unquantised
    # operands, where only the quantisation error of two 3-bit mantissas remains (about 4 %).
    outputs, inner = 18432, 7168
    x = bf16_normal((tokens, inner), 1.0, 9400 + tokens, device)
    w32 = bf16_normal((outputs, inner), 0.02, 9401, device).float()
    blocks = w32.view(outputs // 128, 128, inner // 128, 128)
    w_scale = (blocks.abs().amax(dim=(1, 3)) / 448.0).clamp_min(1e-12)
    w = (blocks / w_scale[:, None, :, None]).clamp(-448, 448).view(outputs, inner).to(torch.float8_e4m3fn)
    q, a_scale = _kernels.fp8_quantise_1x128(x)
    out = _kernels.fp8_block_matmul(q, a_scale, w, w_scale)
    assert torch.equal(out, _kernels.fp8_block_linear(x, w, w_scale))
    picked = sample(4, tokens, 5, seams=(128, 256))
    index = torch.from_numpy(picked).to(device)
    want = oracle.fp8_block_matmul_f64(from_device_fp8(q[index]), a_scale[index].cpu().numpy(),
                                       from_device_fp8(w), w_scale.cpu().numpy())
    close_to(bf16_values(out[index]), want)
    unquantised = (x[index].double() @ w32.double().t()).cpu().numpy()
    assert rel_frobenius(bf16_values(out[index]), unquantised) <= 6e-2


def test_decoder_layer_decode_llama70b_shape(device):
    # the oracle pipeline of the reduced-size layer test, at the size the benchmark runs
    from test_gpu_layer import device_layer, oracle_layer

    batch, hidden_size, q_heads, kv_heads, dim, ffn, context = 32, 8192, 64, 8, 128, 28672, 2048

    def bits(shape, std, seed, mean=0.0):
        generator = torch.Generator(device=device).manual_seed(seed)
        values = torch.randn(shape, generator=generator, device=device) * std + mean
        return from_device_bf16(values.bfloat16())

    weights = {
        "input_norm": bits((hidden_size,), 0.02, 9401, 1.0),
        "post_norm": bits((hidden_size,), 0.02, 9402, 1.0),
        "qkv": bits(((q_heads + 2 * kv_heads) * dim, hidden_size), 0.02, 9403),
        "o": bits((hidden_size, q_heads * dim), 0.02, 9404),
        "gate": bits((ffn, hidden_size), 0.02, 9405),
        "up": bits((ffn, hidden_size), 0.02, 9406),
        "down": bits((hidden_size, ffn), 0.02, 9407),
    }
    hidden, residual = bits((batch, hidden_size), 1.0, 9408), bits((batch, hidden_size), 1.0, 9409)
    k_cache = bits((batch, context, kv_heads, dim), 1.0, 9410)
    v_cache = bits((batch, context, kv_heads, dim), 1.0, 9411)
    # the benchmark's last slot for most sequences, shorter histories for a few
    positions = np.full(batch, context - 1, np.int32)
    positions[:4] = (0, 255, 256, 1000)
    inputs = (weights, hidden, residual, k_cache, v_cache, positions)
    want_out, want_res, want_k, want_v = oracle_layer(*inputs)
    out, res, kc, vc = device_layer(device, *inputs)
    assert rel_frobenius(bf16_values(res), oracle.bf16_to_f32(want_res)) <= 1e-2
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(want_out)) <= 2e-2
    untouched = np.ones((batch, context), bool)
    untouched[np.arange(batch), positions] = False
    assert np.array_equal(from_device_bf16(kc)[untouched], k_cache[untouched])
    assert np.array_equal(from_device_bf16(vc)[untouched], v_cache[untouched])
    appended = (np.arange(batch), positions)
    assert rel_frobenius(bf16_values(kc)[appended], oracle.bf16_to_f32(want_k)[appended]) <= 1e-2
    assert rel_frobenius(bf16_values(vc)[appended], oracle.bf16_to_f32(want_v)[appended]) <= 1e-2


@pytest.mark.parametrize("tokens", [16, 4096])
@pytest.mark.parametrize("packed", [False, True])
def test_e8m0_product_18432x7168(device, packed, tokens):
    # the benchmarked microscaling shape: weights [18432, 7168] E4M3 (scales per 32 x 32 block) or
    # packed E2M1 (scales per row and 32 inputs), at 16 tokens (weight-streaming kernel) and 4096
    # (tiled kernel); sampled 32-row blocks, and at 4096 sampled tokens, against FP64
    outputs, inner = 18432, 7168
    generator = torch.Generator(device=device).manual_seed(9500 + packed)
    x = torch.randint(0, 255, (tokens, inner), generator=generator, device=device, dtype=torch.uint8)
    x[x == 0x7F] = 0x7E
    sx = torch.randint(120, 130, (tokens, inner // 32), generator=generator, device=device, dtype=torch.uint8)
    if packed:
        w = torch.randint(0, 256, (outputs, inner // 2), generator=generator, device=device, dtype=torch.uint8)
        sw = torch.randint(118, 128, (outputs, inner // 32), generator=generator, device=device, dtype=torch.uint8)
    else:
        w = torch.randint(0, 255, (outputs, inner), generator=generator, device=device, dtype=torch.uint8)
        w[w == 0x7F] = 0x7E
        sw = torch.randint(118, 128, (outputs // 32, inner // 32), generator=generator, device=device, dtype=torch.uint8)
    weight = w if packed else w.view(torch.float8_e4m3fn)
    out = _kernels.quantized_matmul(x.view(torch.float8_e4m3fn), sx, weight, sw)
    assert out.shape == (tokens, outputs)
    blocks = sample(10, outputs // 32, 4, seams=(3, 288))  # workgroup seams at multiples of 96 rows
    rows = (blocks[:, None] * 32 + np.arange(32)).ravel()
    index = torch.from_numpy(rows).to(device)
    scale_rows = sw[index] if packed else sw[torch.from_numpy(blocks).to(device)]
    picked = np.unique(np.concatenate([np.arange(0, tokens, 37), np.arange(254, 259) % tokens, [tokens - 1]]))
    xd = oracle.mx_dequantise(x.cpu().numpy()[picked], sx.cpu().numpy()[picked], 32)
    wd = oracle.mx_dequantise(w[index].cpu().numpy(), scale_rows.cpu().numpy(), 32, packed, True)
    want = xd @ wd.T
    got = bf16_values(out)[np.ix_(picked, rows)]
    assert rel_frobenius(got, want) <= 4e-3
    assert (np.abs(got - want) <= 0.008 * np.abs(want) + (np.abs(xd) @ np.abs(wd).T) * 2.0 ** -13).all()
    # one more on every input scale doubles every output exactly (E8M0 scales are powers of two)
    assert torch.equal(_kernels.quantized_matmul(x.view(torch.float8_e4m3fn), sx + 1, weight, sw), out * 2)


@pytest.mark.parametrize("packed", [False, True])
def test_grouped_e8m0_products_at_an_expert_layer_size(device, packed):
    # a mixture-of-experts prefill: 8 groups of up to 300 rows through experts of [4096, 7168]
    # (gate and up of a 2048-wide expert), weights chosen through the device table; sampled rows
    # and outputs against FP64, zeros for clipped rows and invalid experts, exact doubling
    groups, weight_groups, rows, outputs, inner = 8, 5, 300, 4096, 7168
    generator = torch.Generator(device=device).manual_seed(9700 + packed)
    x = torch.randint(0, 255, (groups, rows, inner), generator=generator, device=device, dtype=torch.uint8)
    x[x == 0x7F] = 0x7E
    sx = torch.randint(120, 130, (groups, rows, inner // 32), generator=generator, device=device, dtype=torch.uint8)
    weights, scales = [], []
    for _ in range(weight_groups):
        if packed:
            weights.append(torch.randint(0, 256, (outputs, inner // 2), generator=generator, device=device, dtype=torch.uint8))
            scales.append(torch.randint(118, 128, (outputs, inner // 32), generator=generator, device=device, dtype=torch.uint8))
        else:
            w = torch.randint(0, 255, (outputs, inner), generator=generator, device=device, dtype=torch.uint8)
            w[w == 0x7F] = 0x7E
            weights.append(w)
            scales.append(torch.randint(118, 128, (outputs // 32, inner // 32), generator=generator, device=device, dtype=torch.uint8))
    metadata = torch.tensor([[w.data_ptr(), s.data_ptr()] for w, s in zip(weights, scales)],
                            dtype=torch.int64, device=device)
    active_host, counts_host = [4, 0, 2, 9, 1, 3, 0, -1], [300, 17, 256, 300, 0, 129, 999, 300]
    active = torch.tensor(active_host, dtype=torch.int32, device=device)
    counts = torch.tensor(counts_host, dtype=torch.int32, device=device)
    xt = x.view(torch.float8_e4m3fn)
    out = _kernels.grouped_quantized_matmul(xt, sx, metadata, active, counts, outputs=outputs, packed=packed)
    assert out.shape == (groups, rows, outputs)
    got_all = bf16_values(out)
    blocks = sample(6, outputs // 32, 11, seams=(8,))   # tile seams at multiples of 256 rows
    columns = (blocks[:, None] * 32 + np.arange(32)).ravel()
    for g, (index, count) in enumerate(zip(active_host, counts_host)):
        if not 0 <= index < weight_groups:
            assert not got_all[g].any()
            continue
        count = min(max(count, 0), rows)
        assert not got_all[g, count:].any()
        if count == 0:
            continue
        picked = np.unique(np.concatenate([np.arange(0, count, 41), [count - 1], np.arange(126, 131) % count]))
        xd = oracle.mx_dequantise(x[g].cpu().numpy()[picked], sx[g].cpu().numpy()[picked], 32)
        w_rows = weights[index][torch.from_numpy(columns).to(device)].cpu().numpy()
        s_rows = scales[index][torch.from_numpy(columns if packed else blocks).to(device)].cpu().numpy()
        wd = oracle.mx_dequantise(w_rows, s_rows, 32, packed, True)
        want = xd @ wd.T
        got = got_all[g][np.ix_(picked, columns)]
        assert rel_frobenius(got, want) <= 4e-3
        assert (np.abs(got - want) <= 0.008 * np.abs(want) + (np.abs(xd) @ np.abs(wd).T) * 2.0 ** -13).all()
    # one more on every input scale doubles every output exactly (E8M0 scales are powers of two)
    assert torch.equal(_kernels.grouped_quantized_matmul(xt, sx + 1, metadata, active, counts, outputs=outputs,
                                                         packed=packed), out * 2)
