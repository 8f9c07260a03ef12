"""SGLang plugin mirror on the GPU: each around-hook is called the way SGLang's registry would call
it (original callable first), inside and outside its guard. Routed results are compared with the
oracle or an FP64 product; everything outside a guard must reach the original untouched; the
dispatch counters follow camblas/sglang.py:11-19 of the reference."""

import types

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, sglang as plugin
from helpers import bf16_values, rel_frobenius, to_device_bf16, to_device_fp8

pytestmark = pytest.mark.gpu


class Original:
    """Stands for SGLang's own function: records that it was reached."""

    def __init__(self):
        self.calls = []

    def __call__(self, *arguments):
        self.calls.append(arguments)
        return "original"


def delta(before, name):
    return plugin.dispatch_counts().get(name, 0) - before.get(name, 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_hook_routes_and_falls_back(device, dtype):
    hook = plugin.build_hooks({"linear"})[plugin.LINEAR_TARGET]
    assert set(plugin.build_hooks({"linear"})) == {plugin.LINEAR_TARGET, plugin.BATCHED_LINEAR_TARGET}
    generator = torch.Generator().manual_seed(11)
    x = torch.randn((3, 5, 256), generator=generator).to(dtype).to(device)
    weight = (torch.randn((96, 256), generator=generator) * 0.05).to(dtype).to(device)
    bias = torch.randn((96,), generator=generator).to(dtype).to(device)
    layer = types.SimpleNamespace(weight=weight)
    original, before = Original(), plugin.dispatch_counts()
    for b in (None, bias):
        out = hook(original, object(), layer, x, b)
        want = x.double().cpu() @ weight.double().cpu().T + (0 if b is None else b.double().cpu())
        assert out.shape == (3, 5, 96) and out.dtype == dtype
        assert rel_frobenius(out.double().cpu().numpy(), want.numpy()) <= (1e-5 if dtype == torch.float32 else 1e-2)
    assert delta(before, "linear") == 2 and not original.calls
    # outside the guard: CPU tensors, mixed dtypes, strided input, FP16, gradients wanted
    refused = [
        (x.cpu(), types.SimpleNamespace(weight=weight.cpu()), None),
        (x, types.SimpleNamespace(weight=weight.double()), None),
        (x.transpose(0, 1), layer, None),
        (x.half(), types.SimpleNamespace(weight=weight.half()), None),
        (x[0, 0], layer, None),
    ]
    for value, owner, b in refused:
        assert hook(original, "method", owner, value, b) == "original"
    with torch.enable_grad():
        wanted = x.float().requires_grad_() if dtype == torch.float32 else x.clone().requires_grad_()
        assert hook(original, "method", layer, wanted, None) == "original"
    assert len(original.calls) == len(refused) + 1 and delta(before, "linear") == 2
    assert original.calls[0][0] == "method"


@pytest.mark.parametrize("rows", [1, 5, 200])
def test_fp8_block128_hook(device, rows):
    hooks = plugin.build_hooks({"fp8"})
    assert set(hooks) == {plugin.FP8_BLOCK128_TARGET, plugin.FP8_BLOCK32_PRODUCT_TARGET,
                          plugin.FP8_BLOCK32_LINEAR_TARGET, plugin.FP8_MOE_TARGET}
    hook = hooks[plugin.FP8_BLOCK128_TARGET]
    outputs, inner = 640, 1024
    x = oracle.fill_normal_bf16(910 + rows, (rows, inner))
    w, w_scale = oracle.fill_fp8_blocks(911, outputs, inner, 128)
    xt, wt, st = to_device_bf16(x, device), to_device_fp8(w, device), torch.from_numpy(w_scale).to(device)
    original, before = Original(), plugin.dispatch_counts()
    # like the reference's, this guard wants gradient mode off altogether (SGLang serves that way)
    assert hook(original, xt.view(1, rows, inner), wt, [128, 128], st) == "original"
    del original.calls[:]
    torch.set_grad_enabled(False)
    try:
        block128_checks(hook, original, before, device, rows, outputs, inner, x, w, w_scale, xt, wt, st)
    finally:
        torch.set_grad_enabled(True)


def block128_checks(hook, original, before, device, rows, outputs, inner, x, w, w_scale, xt, wt, st):
    out = hook(original, xt.view(1, rows, inner), wt, [128, 128], st)
    assert out.shape == (1, rows, outputs) and out.dtype == torch.bfloat16
    q, scale = oracle.quantise_1x128(x)
    assert rel_frobenius(bf16_values(out).reshape(rows, outputs),
                         oracle.fp8_block_matmul_f64(q, scale, w, w_scale)) <= 1e-2
    assert delta(before, "fp8") == 1 and delta(before, "fp8_dense_block128") == 1 and not original.calls
    # other block sizes, given input scales, a bias, FP16 activations, a wrong scale grid: original
    assert hook(original, xt, wt, [64, 64], st) == "original"
    assert hook(original, xt, wt, [128, 128], st, torch.ones((rows, inner // 128), device=device)) == "original"
    assert hook(original, xt, wt, [128, 128], st, None, torch.zeros(outputs, device=device)) == "original"
    assert hook(original, xt.half(), wt, [128, 128], st) == "original"
    assert hook(original, xt, wt, [128, 128], st[:, :-1].contiguous()) == "original"
    assert len(original.calls) == 5 and delta(before, "fp8") == 1
    assert len(original.calls[1]) == 6  # all six arguments are forwarded


def block32_case(seed, outputs, inner):
    rng = np.random.default_rng(seed)
    x = oracle.f32_to_e4m3((rng.standard_normal(inner) * 4).astype(np.float32))
    w = oracle.f32_to_e4m3((rng.standard_normal((outputs, inner)) * 4).astype(np.float32))
    sx = np.exp2(rng.integers(-6, 2, inner // 32)).astype(np.float32)
    sw = rng.uniform(0.01, 0.1, ((outputs + 31) // 32, inner // 32)).astype(np.float32)
    return x, sx, w, sw


def test_fp8_block32_hooks(device):
    hooks = plugin.build_hooks({"fp8"})
    product, linear = hooks[plugin.FP8_BLOCK32_PRODUCT_TARGET], hooks[plugin.FP8_BLOCK32_LINEAR_TARGET]
    outputs, inner = 1152, 5120
    x, sx, w, sw = block32_case(77, outputs, inner)
    A = to_device_fp8(x, device).view(1, inner)
    As = torch.from_numpy(sx).to(device).view(1, -1)
    B, Bs = to_device_fp8(w, device), torch.from_numpy(sw).to(device)
    original, before = Original(), plugin.dispatch_counts()
    out = product(original, A, B, As, Bs, [32, 32], torch.bfloat16)
    want = oracle.bf16_to_f32(oracle.fp8_block32_decode(x, sx, w, sw))
    assert out.shape == (1, outputs)
    assert (np.abs(bf16_values(out)[0] - want) <= 2.0 ** -7 * np.abs(want) + 1e-4 * np.abs(want).max()).all()
    assert delta(before, "fp8") == 1 and delta(before, f"fp8_decode:{outputs},{inner}") == 1
    # FP16 output (SGLang's default), two rows, another block size: original
    assert product(original, A, B, As, Bs, [32, 32]) == "original"
    two = torch.cat([A, A])
    assert product(original, two, B, torch.cat([As, As]), Bs, [32, 32], torch.bfloat16) == "original"
    assert product(original, A, B, As, Bs, [128, 128], torch.bfloat16) == "original"
    assert len(original.calls) == 3 and len(original.calls[0]) == 6

    activations = oracle.fill_normal_bf16(78, (1, inner), std=3.0)
    xt = to_device_bf16(activations, device)
    out = linear(original, xt, B, [32, 32], Bs, None, None, True, None)
    q, scale = oracle.quantise_block32(activations[0])
    want = oracle.bf16_to_f32(oracle.fp8_block32_decode(q, scale, w, sw))
    assert (np.abs(bf16_values(out)[0] - want) <= 2.0 ** -7 * np.abs(want) + 1e-4 * np.abs(want).max()).all()
    assert delta(before, "fp8_linear") == 1 and delta(before, f"fp8_linear:{outputs},{inner}") == 1
    assert delta(before, "fp8") == 2
    # without the power-of-two activation-scale policy the original quantiser must run
    assert linear(original, xt, B, [32, 32], Bs, None, None, False, None) == "original"
    assert linear(original, xt, B, [32, 32], Bs, torch.ones(1, device=device), None, True, None) == "original"
    assert len(original.calls) == 5 and len(original.calls[-1]) == 8


@pytest.mark.parametrize("shape", [(2048, 4096), (3392, 6144)])
@pytest.mark.parametrize("magnitude", [0.75, 80.0])
def test_fp8_block128_hook_on_the_reference_shapes(device, shape, magnitude):
    # ref: tests/test_sglang.py:74-117 — one BF16 token, dynamic 1x128 quantisation, a weight whose
    # row count is not a multiple of the 128-row scale block; FP64 product of the oracle-quantised
    # token as the yardstick (the reference compares with SGLang's own kernel bit for bit)
    outputs, inner = shape
    hook = plugin.build_hooks({"fp8"})[plugin.FP8_BLOCK128_TARGET]
    x = oracle.fill_normal_bf16(717, (1, inner), std=magnitude)
    w, w_scale = oracle.fill_fp8_blocks(718, outputs, inner, 128)
    w_scale = (w_scale * 1.25).astype(np.float32)
    original = Original()
    with torch.no_grad():
        out = hook(original, to_device_bf16(x, device), to_device_fp8(w, device), [128, 128],
                   torch.from_numpy(w_scale).to(device))
    assert not original.calls and out.shape == (1, outputs)
    q, scale = oracle.quantise_1x128(x)
    assert rel_frobenius(bf16_values(out), oracle.fp8_block_matmul_f64(q, scale, w, w_scale)) <= 1e-2


def moe_configuration(experts, **changes):
    """The runner configuration the reference's guard accepts (camblas/sglang.py:376-396)."""
    fields = dict(activation="silu", is_gated=True, no_combine=False, apply_router_weight_on_input=False,
                  swiglu_limit=10, gemm1_alpha=None, gemm1_clamp_limit=None, num_experts=experts,
                  num_local_experts=experts, inplace=False, routed_scaling_factor=2.5)
    fields.update(changes)
    return types.SimpleNamespace(**fields)


def test_fp8_moe_hook(device):
    # ref: camblas/sglang.py:340-455 — the single-token FP8 expert step behind
    # fused_moe.fused_experts: routed inside the guard (also in place), the original outside it
    hooks = plugin.build_hooks({"fp8"})
    hook = hooks[plugin.FP8_MOE_TARGET]
    experts, choices, hidden, width = 12, 9, 512, 256
    rng = np.random.default_rng(3)
    x = oracle.f32_to_bf16((rng.standard_normal(hidden) * 3).astype(np.float32))
    w1 = oracle.f32_to_e4m3((rng.standard_normal((experts, 2 * width, hidden)) * 0.6).astype(np.float32))
    w2 = oracle.f32_to_e4m3((rng.standard_normal((experts, hidden, width)) * 0.6).astype(np.float32))
    s1 = (rng.random((experts, 2 * width // 128, hidden // 128)) * 0.002 + 0.001).astype(np.float32)
    s2 = (rng.random((experts, hidden // 128, width // 128)) * 0.002 + 0.001).astype(np.float32)
    ids = rng.permutation(experts)[:choices].astype(np.int32)
    routing = np.linspace(0.05, 1.0, choices).astype(np.float32)
    want = oracle.fp8_moe_decode_f64(x, w1, s1, w2, s2, ids, routing, 2.5)

    xt = to_device_bf16(x.reshape(1, -1), device)
    w1t, w2t = to_device_fp8(w1, device), to_device_fp8(w2, device)
    topk = types.SimpleNamespace(topk_ids=torch.from_numpy(ids).to(device).view(1, -1),
                                 topk_weights=torch.from_numpy(routing).to(device).view(1, -1))
    keywords = dict(w1_scale=torch.from_numpy(s1).to(device), w2_scale=torch.from_numpy(s2).to(device),
                    use_fp8_w8a8=True, block_shape=[128, 128])
    original, before = Original(), plugin.dispatch_counts()

    class KeywordOriginal(Original):
        def __call__(self, *arguments, **kwargs):
            return super().__call__(*arguments)

    original = KeywordOriginal()
    with torch.no_grad():
        out = hook(original, xt, w1t, w2t, topk, moe_configuration(experts), **keywords)
        assert out is not xt and out.shape == (1, hidden) and out.dtype == torch.bfloat16
        assert rel_frobenius(bf16_values(out)[0], want) <= 1e-2
        same = xt.clone()
        inplace = hook(original, same, w1t, w2t, topk, moe_configuration(experts, inplace=True), **keywords)
        assert inplace is same and torch.equal(inplace, out)
        unscaled = hook(original, xt, w1t, w2t, topk, moe_configuration(experts, routed_scaling_factor=None), **keywords)
        assert rel_frobenius(bf16_values(unscaled)[0], want / 2.5) <= 1e-2
        assert delta(before, "fp8") == 3 and delta(before, "fp8_moe") == 3 and not original.calls
        # outside the guard: two tokens, another activation or limit, router weights on the input,
        # a bias, a static activation scale, another block shape, int64 expert IDs, 17 choices,
        # experts sharded over ranks, extra positional arguments
        two = torch.cat([xt, xt])
        refused = [
            ((two, w1t, w2t, topk, moe_configuration(experts)), keywords),
            ((xt, w1t, w2t, topk, moe_configuration(experts, activation="gelu")), keywords),
            ((xt, w1t, w2t, topk, moe_configuration(experts, swiglu_limit=7)), keywords),
            ((xt, w1t, w2t, topk, moe_configuration(experts, apply_router_weight_on_input=True)), keywords),
            ((xt, w1t, w2t, topk, moe_configuration(experts, num_local_experts=experts // 2)), keywords),
            ((xt, w1t, w2t, topk, moe_configuration(experts)), dict(keywords, b1=keywords["w1_scale"])),
            ((xt, w1t, w2t, topk, moe_configuration(experts)), dict(keywords, a1_scale=keywords["w1_scale"])),
            ((xt, w1t, w2t, topk, moe_configuration(experts)), dict(keywords, block_shape=[64, 64])),
            ((xt, w1t, w2t, types.SimpleNamespace(topk_ids=topk.topk_ids.long(), topk_weights=topk.topk_weights),
              moe_configuration(experts)), keywords),
            ((xt, w1t, w2t, types.SimpleNamespace(topk_ids=torch.zeros((1, 17), dtype=torch.int32, device=device),
                                                  topk_weights=torch.ones((1, 17), device=device)),
              moe_configuration(experts)), keywords),
            ((xt, w1t, w2t, topk, moe_configuration(experts), "extra"), keywords),
        ]
        for arguments, kwargs in refused:
            assert hook(original, *arguments, **kwargs) == "original"
    assert hook(original, xt, w1t, w2t, topk, moe_configuration(experts), **keywords) == "original"  # grad mode on
    assert len(original.calls) == len(refused) + 1 and delta(before, "fp8_moe") == 3


@pytest.mark.parametrize("batch,rows,inner,outputs", [(2, 1, 128, 2048), (3, 5, 256, 520), (16, 2, 64, 24)])
def test_batched_linear_hook(device, batch, rows, inner, outputs):
    # ref: camblas/sglang.py:294-336 (its single shape is the first case): BF16 projections per batch
    # with FP32 accumulation and one rounding; anything else reaches the original
    hook = plugin.build_hooks({"linear"})[plugin.BATCHED_LINEAR_TARGET]
    generator = torch.Generator().manual_seed(21 + batch)
    x = torch.randn((batch, rows, inner), generator=generator).to(torch.bfloat16).to(device)
    weight = (torch.randn((batch, outputs, inner), generator=generator) * 0.1).to(torch.bfloat16).to(device)
    layer = types.SimpleNamespace(weight=weight)
    original, before = Original(), plugin.dispatch_counts()
    # the hook serves callers that asked for full-precision BF16 reductions (torch's default allows
    # reduced precision; the reference's guard, and this one, then leave the product to the original)
    previous = torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction
    torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = False
    try:
        routed_and_refused(hook, original, before, layer, x, weight, batch, rows, inner, outputs)
    finally:
        torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = previous


def routed_and_refused(hook, original, before, layer, x, weight, batch, rows, inner, outputs):
    with torch.no_grad():
        out = hook(original, layer, x)
        assert out.shape == (batch, rows, outputs) and out.dtype == torch.bfloat16
        want = torch.einsum("brk,bnk->brn", x.double().cpu(), weight.double().cpu())
        assert rel_frobenius(out.double().cpu().numpy(), want.numpy()) <= 1e-2
        assert delta(before, "bmm") == 1 and not original.calls
        refused = [
            (types.SimpleNamespace(weight=weight.float()), x.float()),
            (types.SimpleNamespace(weight=weight[:, :, : inner // 2]), x[:, :, : inner // 2]),   # strided
            (types.SimpleNamespace(weight=weight[0]), x),
            (types.SimpleNamespace(weight=weight[:1]), x),
            (types.SimpleNamespace(weight=weight.cpu()), x.cpu()),
        ]
        for owner, value in refused:
            assert hook(original, owner, value) == "original"
        torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = True
        try:
            assert hook(original, layer, x) == "original"
        finally:
            torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = False
    assert hook(original, layer, x) == "original"  # grad mode on
    assert len(original.calls) == len(refused) + 2 and delta(before, "bmm") == 1


def test_hooks_leave_what_the_entry_points_refuse_to_the_original(device):
    # the guards stop where the C entry points do: more than 65535 rows for the block-128 product,
    # more than 512 (choice, 128-wide group) pairs for the fused expert step; both must reach
    # SGLang's own function instead of raising inside the hook
    hooks = plugin.build_hooks({"fp8"})
    original = Original()
    rows, outputs, inner = 65536, 128, 128
    x = torch.zeros((rows, inner), dtype=torch.bfloat16, device=device)
    w = torch.zeros((outputs, inner), dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    scale = torch.ones((1, 1), dtype=torch.float32, device=device)
    with torch.no_grad():
        assert hooks[plugin.FP8_BLOCK128_TARGET](original, x, w, [128, 128], scale) == "original"
        out = hooks[plugin.FP8_BLOCK128_TARGET](original, x[:65535], w, [128, 128], scale)
    assert out.shape == (65535, outputs) and len(original.calls) == 1

    class KeywordOriginal(Original):
        def __call__(self, *arguments, **kwargs):
            return super().__call__(*arguments)

    original = KeywordOriginal()
    experts, choices, hidden, width = 16, 16, 128, 128 * 33        # 16 * 33 = 528 pairs
    xt = torch.zeros((1, hidden), dtype=torch.bfloat16, device=device)
    w1 = torch.zeros((experts, 2 * width, hidden), dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    w2 = torch.zeros((experts, hidden, width), dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    topk = types.SimpleNamespace(topk_ids=torch.arange(choices, dtype=torch.int32, device=device).view(1, -1),
                                 topk_weights=torch.ones((1, choices), dtype=torch.float32, device=device))
    keywords = dict(w1_scale=torch.ones((experts, 2 * width // 128, 1), device=device),
                    w2_scale=torch.ones((experts, 1, width // 128), device=device),
                    use_fp8_w8a8=True, block_shape=[128, 128])
    with torch.no_grad():
        assert hooks[plugin.FP8_MOE_TARGET](original, xt, w1, w2, topk, moe_configuration(experts), **keywords) == "original"
        with pytest.raises(RuntimeError):
            _kernels.fp8_moe_decode(xt, w1, w2, keywords["w1_scale"], keywords["w2_scale"],
                                    topk.topk_ids.view(-1), topk.topk_weights.view(-1))
    assert len(original.calls) == 1
