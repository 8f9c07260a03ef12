"""Opt-in routing of SGLang's linear and block-scaled FP8 products to libcamblas_hip.so.

Host-side mirror of the reference plugin (camblas/sglang.py:11-747): the same entry point
(`install`, registered under `sglang.srt.plugins`), the same environment contract, the same hook
targets in SGLang's `HookRegistry`, the same `dispatch_counts()` keys, and the same rule that any
call outside a guard goes to SGLang's original function untouched.

    CAMBLAS_SGLANG_OPS=linear,fp8   operations to route (unknown names raise ValueError)
    CAMBLAS_SGLANG_ALGORITHM=auto   GEMM policy for the routed products
    CAMBLAS_SGLANG_STABLE_MOE=1     repeatable token order inside expert blocks at prefill

What differs from the reference, on purpose: its block-128 FP8 guard admits one token and a list
of eleven weight shapes, because its kernel is a single-token Triton kernel for Hopper; the kernels
here cover any token count and any [N, K] with K a multiple of 128, so the guard checks layout and
dtypes only. The block-32 guards keep the single-token rule (that is what the entry points
compute) but drop the shape list for the same reason. The fused single-token FP8 expert step
keeps every condition of the reference on the runner configuration and drops only the fixed
289-expert shapes: any expert count and any widths in multiples of 128 with at most 16 choices.
The batched BF16 projection hook takes any [batch, rows, inner] x [batch, outputs, inner] with
at most 16 batches (one product per batch) instead of the single [2, 1, 128] x [2, 2048, 128]
shape. The Triton tile tables of CAMBLAS_SGLANG_FP8_TILES configure SGLang's own Triton kernels
and have no counterpart.

The hook bodies are plain functions of (original, *arguments) returned by `build_hooks`, so they
can be exercised without SGLang; `install` only hands them to the registry.
"""

import os

_calls = {}

LINEAR_TARGET = "sglang.srt.layers.quantization.unquant.UnquantizedLinearMethod.apply"
BATCHED_LINEAR_TARGET = "sglang.srt.layers.linear.ColumnParallelBatchedLinear.forward"
FP8_BLOCK128_TARGET = ("sglang.srt.layers.quantization.fp8_utils."
                       "deepgemm_w8a8_block_fp8_linear_with_fallback")
FP8_BLOCK32_PRODUCT_TARGET = "sglang.kernels.ops.quantization.fp8_kernel.w8a8_block_fp8_matmul_triton"
FP8_BLOCK32_LINEAR_TARGET = "sglang.srt.layers.quantization.fp8_utils.triton_w8a8_block_fp8_linear"
FP8_MOE_TARGET = "sglang.srt.layers.moe.moe_runner.triton_utils.fused_moe.fused_experts"
MOE_ALIGN_TARGET = ("sglang.srt.layers.moe.moe_runner.triton_utils."
                    "moe_align_block_size.moe_align_block_size")
OPERATIONS = ("linear", "fp8")


def dispatch_counts():
    """Copy of the per-operation and per-shape host dispatch counts of this process; work replayed
    from a captured graph is not counted (ref: camblas/sglang.py:11-19)."""
    return dict(_calls)


def _count(*names):
    for name in names:
        _calls[name] = _calls.get(name, 0) + 1


def canonical_moe_tokens(token_ids, expert_ids, count, block_size, choices):
    """Sort the token choices inside each expert block, keeping every choice in its block and the
    padding at the end (ref: camblas/sglang.py:122-152; known answer in tests/test_sglang.py:19-39).

    token_ids: 1-D choice indices including padded capacity; expert_ids: expert label per block;
    count: scalar tensor, entries inside live blocks; choices: number of token choices, which is
    also the padding value. Returns a new tensor of token_ids' dtype.
    """
    import torch

    span = choices + 1
    labels = expert_ids.to(torch.int64).repeat_interleave(block_size)[: token_ids.numel()]
    # one sortable key per entry: (expert + 1, token); entries past `count` sort last
    keys = (labels + 1) * span + token_ids.to(torch.int64)
    live = torch.arange(token_ids.numel(), device=token_ids.device) < count
    last = torch.iinfo(torch.int64).max
    keys = torch.where(live, keys, last).sort().values
    return torch.where(keys == last, choices, keys % span).to(token_ids.dtype)


def _inference(*tensors):
    import torch

    return not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors))


def _tracing():
    import torch

    compiling = getattr(getattr(torch, "_dynamo", None), "is_compiling", None)
    return bool(compiling and compiling())


def build_hooks(selected):
    """{hook target: around-function} for the selected operations. Every function takes SGLang's
    original callable first and falls back to it whenever its guard does not hold."""
    import torch

    from . import _kernels

    hooks = {}

    def linear(original, method, layer, x, bias=None):
        # ref: camblas/sglang.py:250-286 (same predicate)
        weight = layer.weight
        operands = (x, weight) if bias is None else (x, weight, bias)
        if (x.is_cuda and x.ndim >= 2 and weight.ndim == 2
                and x.dtype in (torch.float32, torch.bfloat16)
                and all(t.is_contiguous() and t.device == x.device and t.dtype == x.dtype for t in operands)
                and x.shape[-1] == weight.shape[1] and _inference(*operands)):
            _count("linear")
            return _kernels.linear(x, weight, bias)
        return original(method, layer, x, bias)

    def batched(original, layer, input):
        # ref: camblas/sglang.py:294-336; FP32 accumulation, one BF16 rounding
        weight = layer.weight
        if (input.is_cuda and input.ndim == 3 and weight.ndim == 3 and 1 <= input.shape[0] <= 16
                and input.shape[0] == weight.shape[0] and input.shape[2] == weight.shape[2]
                and input.shape[1] >= 1 and input.dtype == weight.dtype == torch.bfloat16
                and input.is_contiguous() and weight.is_contiguous() and weight.device == input.device
                and not torch.is_grad_enabled() and not _tracing()
                and not torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction):
            output = torch.empty((input.shape[0], input.shape[1], weight.shape[1]), dtype=torch.bfloat16,
                                 device=input.device)
            for index in range(input.shape[0]):
                _kernels.matmul(input[index], weight[index].t(), out=output[index])
            _count("bmm")
            return output
        return original(layer, input)

    def fp8_block128(original, input, weight, block_size, weight_scale, input_scale=None, bias=None):
        # ref: camblas/sglang.py:472-544; dynamic 1x128 activation quantisation, any row count
        if (input.is_cuda and input.ndim >= 2 and weight.ndim == 2
                and input.dtype == torch.bfloat16 and weight.dtype == torch.float8_e4m3fn
                and list(block_size) == [128, 128] and weight_scale.dtype == torch.float32
                and input.shape[-1] == weight.shape[1] and weight.shape[1] % 128 == 0
                and input.numel() > 0 and input.numel() // input.shape[-1] <= 65535
                and tuple(weight_scale.shape) == ((weight.shape[0] + 127) // 128, weight.shape[1] // 128)
                and input_scale is None and bias is None
                and all(t.is_contiguous() and t.device == input.device
                        for t in (input, weight, weight_scale))
                and not torch.is_grad_enabled() and not _tracing()):
            _count("fp8", "fp8_dense_block128")
            return _kernels.fp8_block_linear(input, weight, weight_scale)
        return original(input, weight, block_size, weight_scale, input_scale, bias)

    def block32_shape(rows_input, weight):
        inner, outputs = weight.shape[1], weight.shape[0]
        return (rows_input.numel() == rows_input.shape[-1] == inner and 32 <= inner <= 8192
                and inner % 32 == 0 and outputs >= 16 and outputs % 16 == 0)

    def fp8_block32_product(original, A, B, As, Bs, block_size, output_dtype=torch.float16):
        # ref: camblas/sglang.py:578-640
        operands = (A, B, As, Bs)
        if (not _tracing() and A.is_cuda and A.ndim >= 2 and B.ndim == 2 and As.ndim == A.ndim
                and Bs.ndim == 2 and list(block_size) == [32, 32] and output_dtype == torch.bfloat16
                and A.dtype == B.dtype == torch.float8_e4m3fn and As.dtype == Bs.dtype == torch.float32
                and block32_shape(A, B) and A.is_contiguous() and B.is_contiguous()
                and tuple(Bs.shape) == ((B.shape[0] + 31) // 32, B.shape[1] // 32)
                and tuple(As.shape) == tuple(A.shape[:-1]) + (A.shape[-1] // 32,)
                and all(t.device == A.device for t in operands)
                and all(0 < stride <= 2147483647 for stride in (As.stride(-1), *Bs.stride()))
                and _inference(*operands) and _kernels.fp8_decode_supported(A.device)):
            _count("fp8", f"fp8_decode:{B.shape[0]},{B.shape[1]}")
            return _kernels.fp8_decode(A, As, B, Bs)
        return original(A, B, As, Bs, block_size, output_dtype)

    def fp8_block32_linear(original, input, weight, block_size, weight_scale, input_scale=None,
                           bias=None, act_scale_ue8m0=False, weight_bf16=None):
        # ref: camblas/sglang.py:648-741; power-of-two activation scales (the UE8M0 policy)
        operands = (input, weight, weight_scale)
        if (not _tracing() and input.is_cuda and input.ndim >= 2 and weight.ndim == 2
                and weight_scale.ndim == 2 and list(block_size) == [32, 32] and act_scale_ue8m0
                and input_scale is None and bias is None and input.dtype == torch.bfloat16
                and weight.dtype == torch.float8_e4m3fn and weight_scale.dtype == torch.float32
                and block32_shape(input, weight) and input.is_contiguous() and weight.is_contiguous()
                and tuple(weight_scale.shape) == ((weight.shape[0] + 31) // 32, weight.shape[1] // 32)
                and all(t.device == input.device for t in operands)
                and all(0 < stride <= 2147483647 for stride in weight_scale.stride())
                and _inference(*operands) and _kernels.fp8_decode_supported(input.device)):
            _count("fp8", "fp8_linear", f"fp8_linear:{weight.shape[0]},{weight.shape[1]}")
            return _kernels.fp8_linear(input, weight, weight_scale)
        return original(input, weight, block_size, weight_scale, input_scale, bias, act_scale_ue8m0,
                        weight_bf16)

    def fp8_moe_fused(original, hidden_states, w1, w2, topk_output, moe_runner_config, *args, **kwargs):
        # ref: camblas/sglang.py:340-455; one token, silu-gated experts with the limit 10, FP8
        # weights with 128 x 128 block scales, no biases, zero points or static activation scales
        cfg = moe_runner_config
        ids, routing = topk_output.topk_ids, topk_output.topk_weights
        scales = (kwargs.get("w1_scale"), kwargs.get("w2_scale"))
        if (not args and not _tracing() and hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16
                and hidden_states.ndim == 2 and hidden_states.shape[0] == 1
                and w1.ndim == 3 and w2.ndim == 3 and w1.dtype == w2.dtype == torch.float8_e4m3fn
                and w1.shape[0] == w2.shape[0] and w1.shape[2] == hidden_states.shape[1] == w2.shape[1]
                and w1.shape[1] == 2 * w2.shape[2] and w1.shape[2] % 128 == 0 and w2.shape[2] % 128 == 0
                and cfg.activation == "silu" and cfg.is_gated and not cfg.no_combine
                and not cfg.apply_router_weight_on_input and cfg.swiglu_limit == 10
                and cfg.gemm1_alpha is None and cfg.gemm1_clamp_limit is None
                and cfg.num_experts == cfg.num_local_experts == w1.shape[0]
                and kwargs.get("use_fp8_w8a8") and kwargs.get("block_shape") == [128, 128]
                and not any(kwargs.get(k, False) for k in ("use_int8_w8a8", "use_int8_w8a16", "use_int4_w4a16",
                                                           "per_channel_quant", "fuse_swiglu_interleaved"))
                and all(kwargs.get(k) is None for k in ("b1", "b2", "w1_zp", "w2_zp", "a1_scale", "a2_scale", "a1_q"))
                and ids.dtype == torch.int32 and ids.ndim == 2 and ids.shape[0] == 1 and 1 <= ids.shape[1] <= 16
                and ids.shape[1] * (w2.shape[2] // 128) <= 512
                and routing.dtype == torch.float32 and routing.shape == ids.shape
                and all(t is not None and t.dtype == torch.float32 for t in scales)
                and tuple(scales[0].shape) == (w1.shape[0], w1.shape[1] // 128, w1.shape[2] // 128)
                and tuple(scales[1].shape) == (w2.shape[0], w2.shape[1] // 128, w2.shape[2] // 128)
                and all(t.is_contiguous() and t.device == hidden_states.device
                        for t in (hidden_states, w1, w2, ids, routing, *scales))
                and not torch.is_grad_enabled()):
            output = hidden_states if cfg.inplace else torch.empty_like(hidden_states)
            factor = 1.0 if cfg.routed_scaling_factor is None else cfg.routed_scaling_factor
            _kernels.fp8_moe_decode(hidden_states, w1, w2, scales[0], scales[1], ids, routing,
                                    factor=factor, out=output)
            _count("fp8", "fp8_moe")
            return output
        return original(hidden_states, w1, w2, topk_output, moe_runner_config, *args, **kwargs)

    if "linear" in selected:
        hooks[LINEAR_TARGET] = linear
        hooks[BATCHED_LINEAR_TARGET] = batched
    if "fp8" in selected:
        hooks[FP8_BLOCK128_TARGET] = fp8_block128
        hooks[FP8_BLOCK32_PRODUCT_TARGET] = fp8_block32_product
        hooks[FP8_BLOCK32_LINEAR_TARGET] = fp8_block32_linear
        hooks[FP8_MOE_TARGET] = fp8_moe_fused
    return hooks


def stable_moe_hook(original, topk_ids, block_size, num_experts, *args, **kwargs):
    """Around-hook of SGLang's moe_align_block_size: prefill batches (more than one token) get the
    token choices of each expert block in ascending order; decode is untouched
    (ref: camblas/sglang.py:155-196)."""
    ids, experts, count = original(topk_ids, block_size, num_experts, *args, **kwargs)
    if topk_ids.shape[0] > 1:
        ids = canonical_moe_tokens(ids, experts, count, block_size, topk_ids.numel())
    return ids, experts, count


def selected_operations(environment=None):
    """Parse CAMBLAS_SGLANG_OPS (ref: camblas/sglang.py:213-217)."""
    environment = os.environ if environment is None else environment
    selected = set(filter(None, environment.get("CAMBLAS_SGLANG_OPS", "").split(",")))
    if selected - set(OPERATIONS):
        raise ValueError(f"Unknown CAMBLAS SGLang operations: {sorted(selected)}")
    return selected


def install():
    """Entry point of the `sglang.srt.plugins` group: register the selected hooks
    (ref: camblas/sglang.py:199-747). Without CAMBLAS_SGLANG_OPS and CAMBLAS_SGLANG_STABLE_MOE this
    does nothing and does not import SGLang."""
    stable = os.environ.get("CAMBLAS_SGLANG_STABLE_MOE") == "1"
    selected = selected_operations()
    if not stable and not selected:
        return
    from sglang.srt.plugins.hook_registry import HookRegistry, HookType

    if stable:
        HookRegistry.register(MOE_ALIGN_TARGET, stable_moe_hook, HookType.AROUND)
    if not selected:
        return
    from . import _kernels

    algorithm = os.environ.get("CAMBLAS_SGLANG_ALGORITHM", "auto")
    _kernels.set_algorithm(algorithm)
    if "linear" in selected:
        # torch.mm / addmm / F.linear outside the hooked method as well (ref: camblas/sglang.py:245-248)
        from . import _native

        module = _native.tensor_module()
        if module is not None and hasattr(module, "install_torch_backend"):
            module.install_torch_backend(_native.ALGORITHMS[algorithm])
    for target, function in build_hooks(selected).items():
        HookRegistry.register(target, function, HookType.AROUND)
