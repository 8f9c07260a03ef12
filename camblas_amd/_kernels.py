"""Tensor-level operators of the linear path on top of the C ABI.

Host-side mirror of the reference's operator table (camblas/_kernels.py:34-59 and the binding
functions in src/cuda/torch_bindings.cpp): same names, argument meaning and error behaviour for
matmul / linear / rms_norm / add_rms_norm / silu_multiply / swiglu / gated_mlp / qkv_linear, plus
the block-128 FP8 linear, rotary embedding, GQA decode attention and the decoder-layer decode step
this backend adds. torch supplies device memory and streams only; every product and fusion runs in
libcamblas_hip.so. Nothing here computes on the CPU or falls back to torch kernels.
"""

import ctypes as ct

import torch

from . import _native
from ._native import algorithm, set_algorithm, stats, tensor_module  # noqa: F401 (re-exported)

_DTYPE_CODE = {torch.float32: 0, torch.float64: 1, torch.bfloat16: 2}
INT_MAX = 2**31 - 1


def _require(condition, message):
    if not condition:
        raise RuntimeError(message)


def _validate(tensor, reference, allow_bfloat16=True):
    # ref: src/cuda/torch_bindings.cpp:122-138
    allowed = (torch.float32, torch.float64) + ((torch.bfloat16,) if allow_bfloat16 else ())
    _require(
        tensor.is_cuda and tensor.dtype in allowed,
        "CAMBLAS matmul requires CUDA FP32, FP64 or BF16 tensors"
        if allow_bfloat16
        else "CAMBLAS CUDA requires CUDA FP32 or FP64 tensors",
    )
    _require(
        tensor.device == reference.device and tensor.dtype == reference.dtype,
        "All operands must have the same device and dtype",
    )
    _require(all(size <= INT_MAX for size in tensor.shape), "LP64 dimension overflow")
    _require(all(stride <= INT_MAX for stride in tensor.stride()), "LP64 stride overflow")


def _operand(tensor):
    """Row-major 2-D tensor -> (tensor, transpose flag, leading dimension) of the column-major view.

    ref: src/cuda/torch_bindings.cpp:146-153
    """
    rows, columns = tensor.shape
    stride0, stride1 = tensor.stride()
    if stride1 == 1 and stride0 >= max(1, columns):
        return tensor, b"N", stride0
    if stride0 == 1 and stride1 >= max(1, rows):
        return tensor, b"T", stride1
    return tensor.contiguous(), b"N", max(1, columns)


def _pointer(tensor):
    return ct.c_void_p(tensor.data_ptr()) if tensor is not None else None


def matmul(a, b, out=None, alpha=1.0, beta=0.0):
    """alpha * a @ b + beta * out for 2-D FP32 or BF16 device tensors.

    ref: src/cuda/torch_bindings.cpp:155-199 (row-major operands become the swapped column-major
    call).
    """
    _validate(a, a)
    _validate(b, a)
    _require(
        a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0],
        "matmul requires compatible rank-two operands",
    )
    m, k = a.shape
    n = b.shape[1]
    if out is not None:
        _validate(out, a)
        _require(
            out.dim() == 2 and out.shape[0] == m and out.shape[1] == n and out.is_contiguous(),
            "Output must have the product shape and contiguous row storage",
        )
        _require(
            out.untyped_storage().data_ptr() != a.untyped_storage().data_ptr()
            and out.untyped_storage().data_ptr() != b.untyped_storage().data_ptr(),
            "GEMM output cannot alias an input",
        )
        c = out
    else:
        _require(beta == 0, "beta requires an existing output tensor")
        c = torch.empty((m, n), dtype=a.dtype, device=a.device)
    left, left_trans, left_ld = _operand(b)
    right, right_trans, right_ld = _operand(a)
    native = _native.context(a.device)
    name = {torch.float32: "sgemm", torch.float64: "dgemm", torch.bfloat16: "bgemm"}[a.dtype]
    scalar = ct.c_double if a.dtype == torch.float64 else ct.c_float
    with torch.cuda.device(a.device):
        native.call(
            name, left_trans, right_trans, n, m, k, scalar(alpha), _pointer(left), left_ld,
            _pointer(right), right_ld, scalar(beta), _pointer(c), max(1, n),
        )
    return c


def linear(x, weight, bias=None):
    """x @ weight.T (+ bias) with x [..., inputs] and weight [outputs, inputs].

    ref: src/cuda/torch_bindings.cpp:244-270. The bias add is a torch elementwise op there as well.
    """
    _validate(x, x)
    _validate(weight, x)
    _require(
        x.dim() >= 1 and weight.dim() == 2 and x.shape[-1] == weight.shape[1],
        "linear requires matching input and [outputs, inputs] weight dimensions",
    )
    rows = 1
    for size in x.shape[:-1]:
        rows *= size
    _require(rows <= INT_MAX, "LP64 flattened row overflow")
    if bias is not None:
        _validate(bias, x)
        _require(
            bias.dim() == 1 and bias.shape[0] == weight.shape[0],
            "linear bias must have the output width",
        )
    result = matmul(x.reshape(rows, x.shape[-1]), weight.t())
    if bias is not None:
        result = result.add(bias)
    return result.reshape(*x.shape[:-1], weight.shape[0])


def _epilogue_addend(bias, a, rows, columns):
    """(pointer holder, row pitch) of a BF16 bias the product can read where it lies, else None:
    one row for all output rows ([n], [1, n]) or a full [rows, n] matrix, unit stride along n."""
    if (a.dtype != torch.bfloat16 or bias.dtype != torch.bfloat16 or bias.device != a.device or bias.dim() not in (1, 2)
            or bias.shape[-1] != columns or (columns > 1 and bias.stride(-1) != 1)):
        return None
    if bias.dim() == 1 or bias.shape[0] == 1:
        return bias, 0
    if bias.shape[0] != rows or (rows > 1 and bias.stride(0) < columns):
        return None
    return bias, (bias.stride(0) if rows > 1 else 0)


def addmm(bias, a, b, beta=1.0, alpha=1.0):
    """beta * bias + alpha * a @ b, rounded once.

    A BF16 bias row or matrix with unit stride along the output features is read by the product's
    epilogue (camblas_cuda_bgemm_add); any other broadcast form is expanded and cloned, then updated
    in place, as the reference does for every form (ref: src/cuda/torch_backend.cuh:59-71).
    """
    m, n = a.shape[0], b.shape[1]
    if beta == 0:
        return matmul(a, b, None, alpha, 0.0)
    addend = _epilogue_addend(bias, a, m, n) if m > 0 and n > 0 and a.shape[1] > 0 else None
    if addend is not None:
        _validate(a, a)
        _validate(b, a)
        _require(a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0],
                 "matmul requires compatible rank-two operands")
        out = torch.empty((m, n), dtype=a.dtype, device=a.device)
        left, left_trans, left_ld = _operand(b)
        right, right_trans, right_ld = _operand(a)
        with torch.cuda.device(a.device):
            _native.context(a.device).call(
                "bgemm_add", left_trans, right_trans, n, m, a.shape[1], ct.c_float(alpha), _pointer(left), left_ld,
                _pointer(right), right_ld, ct.c_float(beta), _pointer(addend[0]), addend[1], _pointer(out), max(1, n))
        return out
    out = bias.expand(m, n).clone(memory_format=torch.contiguous_format)
    return matmul(a, b, out, alpha, beta)


def _dense(tensor, reference):
    _validate(tensor, reference, allow_bfloat16=False)
    return tensor.contiguous()


def _affine_forward(x, weight, bias, relu, out=None):
    # ref: affine, src/cuda/torch_bindings.cpp:737-771
    x, weight, bias = _dense(x, x), _dense(weight, x), _dense(bias, x)
    _require(x.dim() == 2 and weight.dim() == 2 and bias.dim() == 1 and x.shape[1] == weight.shape[0]
             and weight.shape[1] == bias.shape[0], "Invalid affine operand shapes")
    rows, inner = x.shape
    columns = weight.shape[1]
    if out is not None:
        _validate(out, x, allow_bfloat16=False)
        _require(out.dim() == 2 and tuple(out.shape) == (rows, columns) and out.is_contiguous(),
                 "Invalid affine output shape or strides")
        storage = out.untyped_storage().data_ptr()
        _require(all(storage != t.untyped_storage().data_ptr() for t in (x, weight, bias)),
                 "Affine output cannot alias an input")
    else:
        out = torch.empty((rows, columns), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _native.context(x.device).call("affine", _DTYPE_CODE[x.dtype], rows, inner, columns, _pointer(x),
                                       _pointer(weight), _pointer(bias), int(bool(relu)), _pointer(out))
    return out


class _Affine(torch.autograd.Function):
    """ref: AffineAutograd, src/cuda/torch_bindings.cpp:773-801 — the gradients are products through
    this library; with ReLU the incoming gradient is masked where the output is not positive."""

    @staticmethod
    def forward(ctx, x, weight, bias, relu):
        output = _affine_forward(x, weight, bias, relu)
        ctx.save_for_backward(x, weight, output)
        ctx.relu = relu
        return output

    @staticmethod
    def backward(ctx, gradient):
        x, weight, output = ctx.saved_tensors
        if ctx.relu:
            gradient = torch.where(output <= 0, torch.zeros_like(gradient), gradient)
        dx = matmul_autograd(gradient, weight.t()) if ctx.needs_input_grad[0] else None
        dw = matmul_autograd(x.t(), gradient) if ctx.needs_input_grad[1] else None
        db = gradient.sum(0) if ctx.needs_input_grad[2] else None
        return dx, dw, db, None


class _Matmul(torch.autograd.Function):
    """a @ b with both gradients as products of this library (ref: MatmulAutograd,
    src/cuda/torch_bindings.cpp:201-242); differentiable to any order."""

    @staticmethod
    def forward(ctx, a, b):
        ctx.save_for_backward(a, b)
        return matmul(a, b)

    @staticmethod
    def backward(ctx, gradient):
        a, b = ctx.saved_tensors
        da = matmul_autograd(gradient, b.t()) if ctx.needs_input_grad[0] else None
        db = matmul_autograd(a.t(), gradient) if ctx.needs_input_grad[1] else None
        return da, db


def matmul_autograd(a, b):
    """matmul that records gradients when any operand needs them."""
    if torch.is_grad_enabled() and (a.requires_grad or b.requires_grad):
        return _Matmul.apply(a, b)
    return matmul(a, b)


def affine(x, weight, bias, relu=False, out=None):
    """x @ weight + bias with optional ReLU for FP32 / FP64 (ref: affine_public,
    src/cuda/torch_bindings.cpp:803-813; C entry include/camblas_cuda.h:71-75)."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in (x, weight, bias)):
        _require(out is None, "Autograd affine does not support an out tensor")
        return _Affine.apply(x, weight, bias, bool(relu))
    return _affine_forward(x, weight, bias, relu, out)


def _mlp_forward(x, w1, b1, w2, b2):
    # ref: mlp, src/cuda/torch_bindings.cpp:815-841; returns (output, hidden activations)
    x, w1, b1, w2, b2 = (_dense(t, x) for t in (x, w1, b1, w2, b2))
    _require(x.dim() == 2 and w1.dim() == 2 and w2.dim() == 2 and b1.dim() == 1 and b2.dim() == 1
             and x.shape[1] == w1.shape[0] and w1.shape[1] == w2.shape[0]
             and b1.shape[0] == w1.shape[1] and b2.shape[0] == w2.shape[1], "Invalid MLP operand shapes")
    rows, inputs = x.shape
    hidden, outputs = w2.shape
    h = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    out = torch.empty((rows, outputs), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _native.context(x.device).call("mlp", _DTYPE_CODE[x.dtype], rows, inputs, hidden, outputs,
                                       _pointer(x), _pointer(w1), _pointer(b1), _pointer(w2), _pointer(b2),
                                       _pointer(h), _pointer(out))
    return out, h


def mlp_backward(x, w1, w2, hidden, gradient, needed=(True,) * 5):
    """Gradients (dx, dw1, db1, dw2, db2) of mlp; entries not `needed` are None
    (ref: mlp_backward_tensors, src/cuda/torch_bindings.cpp:925-966; C entry
    include/camblas_cuda.h:87-94)."""
    x, w1, w2, hidden, gradient = (_dense(t, x) for t in (x, w1, w2, hidden, gradient))
    _require(x.dim() == 2 and w1.dim() == 2 and w2.dim() == 2 and hidden.dim() == 2 and gradient.dim() == 2
             and x.shape[1] == w1.shape[0] and w1.shape[1] == w2.shape[0]
             and tuple(hidden.shape) == (x.shape[0], w1.shape[1])
             and tuple(gradient.shape) == (x.shape[0], w2.shape[1]), "Invalid backward operand shapes")
    rows, inputs = x.shape
    width, outputs = w2.shape

    def empty(wanted, *shape):
        return torch.empty(shape, dtype=x.dtype, device=x.device) if wanted else None

    dh = empty(any(needed[:3]), rows, width)
    dx, dw1, db1 = empty(needed[0], rows, inputs), empty(needed[1], inputs, width), empty(needed[2], width)
    dw2, db2 = empty(needed[3], width, outputs), empty(needed[4], outputs)
    with torch.cuda.device(x.device):
        _native.context(x.device).call(
            "mlp_backward", _DTYPE_CODE[x.dtype], rows, inputs, width, outputs, _pointer(x), _pointer(w1),
            _pointer(w2), _pointer(hidden), _pointer(gradient), _pointer(dh), _pointer(dx), _pointer(dw1),
            _pointer(db1), _pointer(dw2), _pointer(db2))
    return dx, dw1, db1, dw2, db2


class _Mlp(torch.autograd.Function):
    """ref: MlpAutograd, src/cuda/torch_bindings.cpp:978-1002 — first derivatives only."""

    @staticmethod
    def forward(ctx, x, w1, b1, w2, b2):
        output, hidden = _mlp_forward(x, w1, b1, w2, b2)
        ctx.save_for_backward(x, w1, w2, hidden)
        return output

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gradient):
        x, w1, w2, hidden = ctx.saved_tensors
        return mlp_backward(x, w1, w2, hidden, gradient, tuple(ctx.needs_input_grad[:5]))


def mlp(x, w1, b1, w2, b2):
    """relu(x @ w1 + b1) @ w2 + b2 for FP32 / FP64 (ref: mlp_public,
    src/cuda/torch_bindings.cpp:1003-1014; C entry include/camblas_cuda.h:76-78)."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in (x, w1, b1, w2, b2)):
        return _Mlp.apply(x, w1, b1, w2, b2)
    return _mlp_forward(x, w1, b1, w2, b2)[0]


def attention(q, k, v, scale=None):
    """softmax(scale * q @ k.T) @ v, dense and single-head, FP32 / FP64 (ref: attention_public,
    src/cuda/torch_bindings.cpp:903-923; C entry include/camblas_cuda.h:80-85). With gradients
    enabled the result is composed from differentiable products, as the reference does."""
    _require(q.dim() == 2 and (scale is not None or q.shape[1] > 0),
             "Attention requires a rank-two query and positive depth for the default scale")
    value = float(scale) if scale is not None else 1.0 / float(q.shape[1]) ** 0.5
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v)):
        scores = matmul_autograd(q, k.t()).mul(value)
        return matmul_autograd(torch.softmax(scores, -1), v)
    q, k, v = _dense(q, q), _dense(k, q), _dense(v, q)
    _require(k.dim() == 2 and v.dim() == 2 and q.shape[1] == k.shape[1] and k.shape[0] == v.shape[0],
             "Invalid attention operand shapes")
    out = torch.empty((q.shape[0], v.shape[1]), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        _native.context(q.device).call("attention", _DTYPE_CODE[q.dtype], q.shape[0], k.shape[0],
                                       q.shape[1], v.shape[1], ct.c_double(value), _pointer(q), _pointer(k),
                                       _pointer(v), _pointer(out))
    return out


def _elementwise_pair(gate, up, name):
    _require(
        gate.is_cuda and gate.dtype in (torch.float32, torch.bfloat16),
        f"{name} requires CUDA FP32 or BF16 tensors",
    )
    _require(
        up.device == gate.device and up.dtype == gate.dtype and up.shape == gate.shape,
        f"{name} operands must share device, dtype and shape",
    )
    _require(gate.is_contiguous() and up.is_contiguous(), f"{name} operands must be contiguous")


def silu_multiply(gate, up, out=None):
    """round(silu(gate)) * up with storage rounding in between (ref: inference_fusion.cuh:19-28)."""
    _elementwise_pair(gate, up, "silu_multiply")
    out = torch.empty_like(gate) if out is None else out
    _native.context(gate.device).call(
        "silu_multiply", _DTYPE_CODE[gate.dtype], gate.numel(), _pointer(gate), _pointer(up),
        _pointer(out),
    )
    return out


def swiglu(gate, up, limit=0.0, routing=None, out=None):
    """silu(gate) * up in FP32 with optional clamp and per-row routing (ref: :30-51)."""
    _elementwise_pair(gate, up, "swiglu")
    out = torch.empty_like(gate) if out is None else out
    width = gate.shape[-1] if gate.dim() else 1
    if routing is not None:
        _require(
            routing.dtype == torch.float32 and routing.is_contiguous()
            and routing.numel() * width == gate.numel(),
            "routing must hold one FP32 value per row",
        )
    _native.context(gate.device).call(
        "swiglu", _DTYPE_CODE[gate.dtype], gate.numel(), max(1, width), ct.c_float(limit),
        _pointer(gate), _pointer(up), _pointer(routing), _pointer(out),
    )
    return out


def rms_norm(x, weight, epsilon=1e-6, round_before_weight=True):
    """RMS normalisation over the last dimension (ref: src/cuda/torch_bindings.cpp:602-673)."""
    _require(x.is_cuda and x.dtype in (torch.float32, torch.bfloat16), "rms_norm needs FP32/BF16")
    _require(x.is_contiguous() and weight.is_contiguous(), "rms_norm operands must be contiguous")
    width = x.shape[-1]
    _require(weight.numel() == width, "rms_norm weight must match the last dimension")
    rows = x.numel() // max(1, width)
    out = torch.empty_like(x)
    _native.context(x.device).call(
        "add_rms_norm_rows", _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype], rows, width,
        ct.c_float(epsilon), int(round_before_weight), _pointer(x), None, _pointer(weight), None,
        _pointer(out),
    )
    return out


def add_rms_norm(x, residual, weight, epsilon=1e-6, round_before_weight=True):
    """(x + residual rounded to storage, its RMS norm) (ref: torch_bindings.cpp:675-701)."""
    _require(x.is_cuda and x.dtype in (torch.float32, torch.bfloat16), "add_rms_norm needs FP32/BF16")
    _require(
        residual.shape == x.shape and residual.dtype == x.dtype and residual.device == x.device,
        "residual must match the input",
    )
    _require(
        x.is_contiguous() and residual.is_contiguous() and weight.is_contiguous(),
        "add_rms_norm operands must be contiguous",
    )
    width = x.shape[-1]
    _require(weight.numel() == width, "add_rms_norm weight must match the last dimension")
    rows = x.numel() // max(1, width)
    added, out = torch.empty_like(x), torch.empty_like(x)
    _native.context(x.device).call(
        "add_rms_norm_rows", _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype], rows, width,
        ct.c_float(epsilon), int(round_before_weight), _pointer(x), _pointer(residual),
        _pointer(weight), _pointer(added), _pointer(out),
    )
    return added, out


def gated_linear(x, gate_weight, up_weight):
    """silu_multiply(gate(x), up(x)) for a BF16 decode batch x [rows <= 64, inner] in one pass over both
    weight matrices [outputs, inner]; the same rounding points as the three separate calls."""
    _require(x.dtype == gate_weight.dtype == up_weight.dtype == torch.bfloat16 and x.is_cuda,
             "gated_linear takes BF16 device tensors")
    _require(x.dim() == 2 and gate_weight.dim() == 2 and gate_weight.shape == up_weight.shape
             and x.shape[1] == gate_weight.shape[1] and x.shape[0] <= 64, "gated_linear shapes")
    _require(x.stride(1) == 1 and gate_weight.stride(1) == 1 and up_weight.stride(1) == 1
             and gate_weight.stride(0) == up_weight.stride(0), "gated_linear needs row-major operands")
    rows, inner = x.shape
    outputs = gate_weight.shape[0]
    out = torch.empty((rows, outputs), dtype=torch.bfloat16, device=x.device)
    _native.context(x.device).call(
        "bf16_gated_linear", rows, outputs, inner, _pointer(x), x.stride(0), _pointer(gate_weight),
        _pointer(up_weight), gate_weight.stride(0), _pointer(out), outputs)
    return out


def _gated_linear_takes(x, gate_weight, up_weight):
    return (x.dtype == torch.bfloat16 and x.dim() == 2 and 0 < x.shape[0] <= 64 and x.stride(1) == 1
            and gate_weight.stride(1) == 1 and up_weight.stride(1) == 1
            and gate_weight.stride(0) == up_weight.stride(0)
            and all(t.data_ptr() % 16 == 0 for t in (x, gate_weight, up_weight))
            and all(s % 8 == 0 for s in (x.shape[1], x.stride(0), gate_weight.stride(0))))


def gated_mlp(x, gate_weight, up_weight, down_weight):
    """down(silu_multiply(gate(x), up(x))) (ref: src/cuda/torch_bindings.cpp:703-723). A BF16 decode
    batch takes the one-pass front end; anything else the three separate calls."""
    if _gated_linear_takes(x, gate_weight, up_weight):
        return linear(gated_linear(x, gate_weight, up_weight), down_weight)
    gate = linear(x, gate_weight)
    up = linear(x, up_weight)
    silu_multiply(gate, up, out=gate)
    return linear(gate, down_weight)


def qkv_linear(x, q_weight, k_weight, v_weight):
    """Three independent linears with distinct outputs (ref: torch_bindings.cpp:725-736)."""
    return linear(x, q_weight), linear(x, k_weight), linear(x, v_weight)


def fp8_block_matmul(a, a_scale, weight, weight_scale, out=None):
    """E4M3fn a [M,K] x weight [N,K]^T with 1x128 / 128x128 FP32 scales -> BF16 [M,N]."""
    _require(a.dtype == torch.float8_e4m3fn and weight.dtype == torch.float8_e4m3fn,
             "fp8_block_matmul requires float8_e4m3fn operands")
    _require(a.is_cuda and a.is_contiguous() and weight.is_contiguous(), "contiguous device operands")
    rows, inner = a.shape
    outputs = weight.shape[0]
    groups = inner // 128
    _require(weight.shape[1] == inner and inner % 128 == 0, "inner must be a multiple of 128")
    _require(
        a_scale.dtype == torch.float32 and tuple(a_scale.shape) == (rows, groups)
        and a_scale.is_contiguous(),
        "activation scales must be FP32 [rows, inner/128]",
    )
    _require(
        weight_scale.dtype == torch.float32
        and tuple(weight_scale.shape) == ((outputs + 127) // 128, groups)
        and weight_scale.is_contiguous(),
        "weight scales must be FP32 [ceil(outputs/128), inner/128]",
    )
    out = torch.empty((rows, outputs), dtype=torch.bfloat16, device=a.device) if out is None else out
    _native.context(a.device).call(
        "fp8_block_matmul", rows, outputs, inner, _pointer(a), _pointer(a_scale), _pointer(weight),
        _pointer(weight_scale), _pointer(out),
    )
    return out


def fp8_quantise_1x128(x):
    """BF16 [M,K] -> (E4M3fn [M,K], FP32 scales [M,K/128]) (ref: camblas/_hopper.py:82-98)."""
    _require(x.dtype == torch.bfloat16 and x.is_cuda and x.is_contiguous() and x.dim() == 2,
             "fp8_quantise_1x128 requires a contiguous 2-D BF16 device tensor")
    rows, inner = x.shape
    q = torch.empty((rows, inner), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((rows, inner // 128), dtype=torch.float32, device=x.device)
    _native.context(x.device).call(
        "fp8_quantise_1x128", rows, inner, _pointer(x), _pointer(q), _pointer(scale)
    )
    return q, scale


def fp8_block_linear(x, weight, weight_scale):
    """BF16 activations quantised on the fly, then the block-scaled product."""
    q, scale = fp8_quantise_1x128(x.reshape(-1, x.shape[-1]))
    out = fp8_block_matmul(q, scale, weight, weight_scale)
    return out.reshape(*x.shape[:-1], weight.shape[0])


def fp8_moe_decode(x, w1, w2, w1_scale, w2_scale, expert_ids, routing, *, factor=1.0, out=None):
    """One BF16 token [1, hidden] through a block-scaled FP8 mixture-of-experts layer
    (ref: camblas/_hopper.py:329-401 `fused`): w1 E4M3 [experts, 2*width, hidden] (gate rows, then
    up rows), w2 E4M3 [experts, hidden_out, width], FP32 scales per 128 x 128 block, expert_ids
    int32 and routing FP32 with at most 16 entries. Returns BF16 [1, hidden_out]; `out` may be x."""
    experts, doubled, hidden = w1.shape
    hidden_out, width = w2.shape[1], w2.shape[2]
    choices = expert_ids.numel()
    _require(x.is_cuda and x.dtype == torch.bfloat16 and x.numel() == hidden and x.is_contiguous()
             and w1.dtype == w2.dtype == torch.float8_e4m3fn and w1.is_contiguous() and w2.is_contiguous()
             and w2.shape[0] == experts and doubled == 2 * width,
             "FP8 expert step needs one contiguous BF16 token and E4M3 weights [experts, 2*width, hidden] / [experts, hidden_out, width]")
    _require(hidden % 128 == 0 and width % 128 == 0 and hidden_out % 16 == 0 and 1 <= choices <= 16
             and choices * (width // 128) <= 512,
             "FP8 expert step needs hidden and width in multiples of 128, outputs of 16 and 1..16 choices")
    _require(w1_scale.dtype == w2_scale.dtype == torch.float32 and w1_scale.is_contiguous()
             and w2_scale.is_contiguous()
             and tuple(w1_scale.shape) == (experts, doubled // 128, hidden // 128)
             and tuple(w2_scale.shape) == (experts, (hidden_out + 127) // 128, width // 128),
             "FP8 expert scale shapes do not match their 128 x 128 blocks")
    _require(expert_ids.dtype == torch.int32 and routing.dtype == torch.float32
             and routing.numel() == choices and expert_ids.is_contiguous() and routing.is_contiguous()
             and all(t.device == x.device for t in (w1, w2, w1_scale, w2_scale, expert_ids, routing)),
             "FP8 expert step needs int32 expert IDs and FP32 routing weights on the token's device")
    if out is None:
        out = torch.empty((1, hidden_out), dtype=torch.bfloat16, device=x.device)
    _require(out.dtype == torch.bfloat16 and out.numel() == hidden_out and out.is_contiguous()
             and out.device == x.device, "FP8 expert output must be contiguous BF16 [1, hidden_out]")
    _native.context(x.device).call(
        "fp8_moe_decode", experts, choices, hidden, width, hidden_out, _pointer(x), _pointer(w1),
        _pointer(w1_scale), _pointer(w2), _pointer(w2_scale), _pointer(expert_ids), _pointer(routing),
        float(factor), _pointer(out))
    return out


def _bytes(tensor):
    return tensor if tensor.dtype == torch.uint8 else tensor.view(torch.uint8)


def quantized_matmul(x, x_scale, weight, weight_scale, *, activation_block=32):
    """E8M0 block-scaled linear (ref: quantized_matmul_public, src/cuda/torch_bindings.cpp:328-378):
    x E4M3 [.., inner] with scales [.., inner/activation_block]; weight E4M3 [outputs, inner] with
    scales [ceil(outputs/32), inner/32], or packed E2M1 [outputs, inner/2] (uint8 or
    float4_e2m1fn_x2) with scales [outputs, inner/32]. Returns BF16 [.., outputs]."""
    packed = weight.dtype != torch.float8_e4m3fn
    _require(x.is_cuda and x.dtype == torch.float8_e4m3fn and x.is_contiguous()
             and weight.is_contiguous() and x_scale.is_contiguous() and weight_scale.is_contiguous(),
             "quantized matmul requires contiguous GPU operands with E4M3 input")
    _require(not torch.is_grad_enabled() or not any(t.requires_grad for t in (x, x_scale, weight_scale)),
             "quantized matmul supports inference only")
    inner = x.shape[-1]
    rows = x.numel() // max(inner, 1)
    outputs = weight.shape[0]
    _require(weight.dim() == 2 and weight.shape[1] * (2 if packed else 1) == inner
             and inner % 32 == 0 and outputs % 8 == 0 and outputs >= 8
             and activation_block in ((32, 128) if packed else (32,)) and inner % activation_block == 0,
             "Invalid quantized matrix dimensions")
    _require(x_scale.numel() == rows * (inner // activation_block)
             and tuple(weight_scale.shape) == ((outputs if packed else (outputs + 31) // 32), inner // 32),
             "Quantized scale shapes do not match their blocks")
    out = torch.empty(tuple(x.shape[:-1]) + (outputs,), dtype=torch.bfloat16, device=x.device)
    _native.context(x.device).call(
        "quantized_matmul", int(packed), rows, outputs, inner, activation_block, _pointer(x),
        _pointer(_bytes(x_scale)), _pointer(_bytes(weight)), _pointer(_bytes(weight_scale)),
        _pointer(out))
    return out


def grouped_quantized_matmul(x, x_scale, metadata, active, counts, *, outputs, packed,
                             activation_block=32):
    """Batched E8M0 block-scaled products (ref: include/camblas_cuda.h:156-167): x E4M3
    [groups, rows, inner]; metadata uint64 [weight_groups, 2] (weight, scale addresses); active and
    counts int32 [groups]. Returns BF16 [groups, rows, outputs]; inactive groups and padding rows
    are zero."""
    groups, rows, inner = x.shape
    _require(x.is_contiguous() and x_scale.is_contiguous() and metadata.dtype in (torch.int64, torch.uint64)
             and metadata.dim() == 2 and metadata.shape[1] == 2 and active.dtype == torch.int32
             and counts.dtype == torch.int32 and active.numel() == groups == counts.numel(),
             "Invalid grouped operands")
    out = torch.empty((groups, rows, outputs), dtype=torch.bfloat16, device=x.device)
    _native.context(x.device).call(
        "grouped_quantized_matmul", int(packed), groups, metadata.shape[0], rows, outputs, inner,
        activation_block, _pointer(x), _pointer(_bytes(x_scale)), _pointer(metadata),
        _pointer(active), _pointer(counts), _pointer(out))
    return out


def route_groups(experts, active, *, first_expert=0, rows):
    """Slots, reverse mapping and counts for expert/choice IDs (ref: route_groups_public,
    src/cuda/torch_bindings.cpp:465-530): experts int64 [tokens, choices], active int32 [groups].
    Excess rows are discarded and unassigned slots are -1; runs on the current stream."""
    _require(experts.is_cuda and experts.dtype == torch.int64 and experts.dim() == 2
             and experts.is_contiguous() and active.dtype == torch.int32 and active.dim() == 1
             and active.is_contiguous() and active.device == experts.device,
             "routing needs contiguous GPU int64 expert IDs [tokens, choices] and int32 active IDs")
    tokens, choices = experts.shape
    groups = active.numel()
    counts = torch.empty(groups, dtype=torch.int32, device=experts.device)
    slots = torch.empty((groups, rows), dtype=torch.int32, device=experts.device)
    reverse = torch.empty((tokens, max(choices, 1)), dtype=torch.int32, device=experts.device)
    _native.context(experts.device).call(
        "route_groups", tokens, choices, first_expert, groups, rows, _pointer(experts),
        _pointer(active), _pointer(counts), _pointer(slots), _pointer(reverse))
    return slots, reverse, counts


def reduce_groups(grouped, experts, reverse):
    """Sum BF16 contributions [grouped_rows, width] into FP32 [tokens, width] in expert/choice
    order (ref: reduce_groups_public, src/cuda/torch_bindings.cpp:532-600)."""
    _require(grouped.is_cuda and grouped.dtype == torch.bfloat16 and grouped.dim() == 2
             and grouped.is_contiguous() and experts.dtype == torch.int64 and experts.is_contiguous()
             and reverse.dtype == torch.int32 and reverse.is_contiguous()
             and reverse.shape == experts.shape,
             "grouped reduction needs contiguous BF16 rows, int64 experts and int32 reverse")
    tokens, choices = experts.shape
    out = torch.empty((tokens, grouped.shape[1]), dtype=torch.float32, device=grouped.device)
    _native.context(grouped.device).call(
        "reduce_groups", tokens, choices, grouped.shape[1], grouped.shape[0], _pointer(experts),
        _pointer(reverse), _pointer(grouped), _pointer(out))
    return out


def fp8_decode_supported(device=None):
    """Whether the block-32 single-token FP8 product runs on this device (ref: fp8_decode_supported
    in src/cuda/torch_bindings.cpp:380-387)."""
    native = _native.context(device)
    return bool(_native.library().camblas_cuda_fp8_decode_supported(native.handle))


def _fp8_block32(x, x_scale, weight, weight_scale):
    # ref: src/cuda/torch_bindings.cpp:389-445 (same checks, same messages' meaning)
    quantise = x_scale is None
    _require(x.is_cuda and x.dtype == (torch.bfloat16 if quantise else torch.float8_e4m3fn)
             and weight.dtype == torch.float8_e4m3fn,
             "FP8 linear requires GPU BF16/FP8 input and E4M3 weight")
    _require(x.dim() >= 1 and weight.dim() == 2 and weight_scale.dim() == 2 and x.is_contiguous()
             and weight.is_contiguous(),
             "FP8 linear requires contiguous matrices and rank-two weight scales")
    _require(weight_scale.dtype == torch.float32, "FP8 weight scales must be FP32")
    for tensor in (x, weight, weight_scale):
        _require(tensor.device == x.device
                 and not (torch.is_grad_enabled() and tensor.requires_grad),
                 "FP8 operands must share a GPU and support inference only")
    inner, outputs = x.shape[-1], weight.shape[0]
    _require(32 <= inner <= 8192 and inner % 32 == 0 and outputs >= 16 and outputs % 16 == 0
             and x.numel() == inner and weight.shape[1] == inner,
             "Invalid FP8 linear matrix dimensions")
    _require(tuple(weight_scale.shape) == ((outputs + 31) // 32, inner // 32),
             "FP8 weight scale shape does not match its blocks")
    sx, sn, sk = 1, weight_scale.stride(0), weight_scale.stride(1)
    if not quantise:
        _require(x_scale.device == x.device and x_scale.dtype == torch.float32
                 and x_scale.dim() == x.dim()
                 and not (torch.is_grad_enabled() and x_scale.requires_grad),
                 "FP8 input scales require matching device/rank and FP32 inference storage")
        _require(tuple(x_scale.shape[:-1]) == tuple(x.shape[:-1])
                 and x_scale.shape[-1] == inner // 32, "FP8 input scale shape mismatch")
        sx = x_scale.stride(-1)
    _require(sx > 0 and sn > 0 and sk > 0, "FP8 scale strides must be positive")
    out = torch.empty(tuple(x.shape[:-1]) + (outputs,), dtype=torch.bfloat16, device=x.device)
    native = _native.context(x.device)
    if quantise:
        native.call("fp8_linear", outputs, inner, _pointer(x), _pointer(weight),
                    _pointer(weight_scale), sn, sk, None, 0, _pointer(out))
    else:
        native.call("fp8_decode", outputs, inner, _pointer(x), _pointer(x_scale), _pointer(weight),
                    _pointer(weight_scale), sx, sn, sk, None, 0, _pointer(out))
    return out


def fp8_decode(x, x_scale, weight, weight_scale):
    """One E4M3 token [.., inner] with FP32 block-32 scales times E4M3 weights [outputs, inner] with
    FP32 scales [ceil(outputs/32), inner/32] (any positive strides); BF16 [.., outputs]."""
    return _fp8_block32(x, x_scale, weight, weight_scale)


def fp8_linear(x, weight, weight_scale):
    """One BF16 token, quantised per 32 values with a power-of-two scale, then fp8_decode."""
    return _fp8_block32(x, None, weight, weight_scale)


def rope(x, positions, theta=500000.0):
    """In-place rotate-half rotary embedding on BF16 x [tokens, heads, dim]."""
    _require(x.dtype == torch.bfloat16 and x.is_cuda and x.dim() == 3, "rope needs BF16 [T,H,D]")
    _require(x.stride(2) == 1 and x.stride(1) == x.shape[2], "rope needs dense heads")
    _require(positions.dtype == torch.int32 and positions.numel() == x.shape[0], "int32 positions")
    tokens, heads, dim = x.shape
    _native.context(x.device).call(
        "rope", tokens, heads, dim, x.stride(0), ct.c_float(theta), _pointer(positions), _pointer(x)
    )
    return x


def gqa_decode_attention(q, k_cache, v_cache, lengths=None, scale=None):
    """One-token-per-sequence grouped-query attention against BF16 caches [B, C, Hkv, 128]."""
    _require(q.dtype == torch.bfloat16 and q.is_cuda and q.dim() == 3, "q must be BF16 [B,H,D]")
    _require(q.stride(2) == 1 and q.stride(1) == q.shape[2], "q heads must be dense")
    _require(k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape,
             "caches must be contiguous and equal-shaped")
    batch, q_heads, dim = q.shape
    _, context_length, kv_heads, _ = k_cache.shape
    scale = dim**-0.5 if scale is None else scale
    out = torch.empty((batch, q_heads, dim), dtype=torch.bfloat16, device=q.device)
    _native.context(q.device).call(
        "gqa_decode_attention", batch, q_heads, kv_heads, dim, context_length, _pointer(lengths),
        ct.c_float(scale), _pointer(q), q.stride(0), _pointer(k_cache), _pointer(v_cache),
        _pointer(out),
    )
    return out


def kv_append(k_new, v_new, k_cache, v_cache, positions):
    """Write the new token's K/V heads [B, Hkv, D] (views of a fused activation are fine) into the
    caches [B, C, Hkv, D] at positions[B]."""
    batch, kv_heads, dim = k_new.shape
    _require(k_new.stride(2) == 1 and k_new.stride(1) == dim and v_new.stride(1) == dim
             and k_new.stride(0) == v_new.stride(0), "new K/V heads must be dense rows of one stride")
    _require(k_cache.is_contiguous() and v_cache.is_contiguous(), "caches must be contiguous")
    _native.context(k_new.device).call(
        "kv_append", batch, kv_heads, dim, k_cache.shape[1], _pointer(positions), _pointer(k_new),
        _pointer(v_new), k_new.stride(0), _pointer(k_cache), _pointer(v_cache),
    )


def rope_kv_append(qkv, positions, k_cache, v_cache, *, q_heads, kv_heads, theta=500000.0):
    """rope() on the q and k heads of a fused QKV activation [B, Hq + 2 Hkv, D] and kv_append() of
    its k and v heads, in one launch."""
    _require(qkv.dtype == torch.bfloat16 and qkv.is_cuda and qkv.dim() == 3
             and qkv.shape[1] == q_heads + 2 * kv_heads, "qkv must be BF16 [B, Hq + 2 Hkv, D]")
    _require(qkv.stride(2) == 1 and qkv.stride(1) == qkv.shape[2], "qkv heads must be dense")
    _require(k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
             and k_cache.shape[2:] == (kv_heads, qkv.shape[2]), "caches must be [B, C, Hkv, D]")
    _native.context(qkv.device).call(
        "rope_kv_append", qkv.shape[0], q_heads, kv_heads, qkv.shape[2], qkv.stride(0),
        ct.c_float(theta), _pointer(positions), _pointer(qkv), k_cache.shape[1], _pointer(k_cache),
        _pointer(v_cache),
    )
    return qkv


def rope_angles(positions, dim=128, theta=500000.0):
    """FP32 [batch, 2, dim / 2]: sines and cosines of positions * theta^(-2i/dim), the angles of one decode
    step (the same for every layer), for rope_append_attention / decoder_layer_decode."""
    _require(positions.is_cuda and positions.dtype == torch.int32 and positions.dim() == 1, "positions: int32 [batch]")
    angles = torch.empty((positions.shape[0], 2, dim // 2), dtype=torch.float32, device=positions.device)
    _native.context(positions.device).call("rope_angles", positions.shape[0], dim, ct.c_float(theta),
                                           _pointer(positions), _pointer(angles))
    return angles


def rope_append_attention(qkv, positions, k_cache, v_cache, *, q_heads, kv_heads, theta=500000.0, scale=None,
                          angles=None):
    """rope_kv_append() and gqa_decode_attention() over positions + 1 entries in one call (two launches
    instead of three): the attention's partition kernel rotates the queries and the new K row itself and
    appends the new K and V rows to the caches. qkv [B, Hq + 2 Hkv, D] is left unrotated. Bit for bit the
    result and the caches of the two separate calls."""
    _require(qkv.dtype == torch.bfloat16 and qkv.is_cuda and qkv.dim() == 3
             and qkv.shape[1] == q_heads + 2 * kv_heads, "qkv must be BF16 [B, Hq + 2 Hkv, D]")
    _require(qkv.stride(2) == 1 and qkv.stride(1) == qkv.shape[2], "qkv heads must be dense")
    _require(k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
             and k_cache.shape[2:] == (kv_heads, qkv.shape[2]), "caches must be [B, C, Hkv, D]")
    batch, _, dim = qkv.shape
    _require(angles is None or (angles.dtype == torch.float32 and angles.is_contiguous()
                                and tuple(angles.shape) == (batch, 2, dim // 2)), "angles: what rope_angles returns")
    scale = dim**-0.5 if scale is None else scale
    out = torch.empty((batch, q_heads, dim), dtype=torch.bfloat16, device=qkv.device)
    _native.context(qkv.device).call(
        "rope_append_gqa_decode_attention", batch, q_heads, kv_heads, dim, k_cache.shape[1], _pointer(positions),
        ct.c_float(theta), ct.c_float(scale), _pointer(qkv), qkv.stride(0), _pointer(k_cache), _pointer(v_cache),
        _pointer(angles), _pointer(out))
    return out


def decoder_layer_decode(hidden, residual, weights, k_cache, v_cache, positions, lengths, *,
                         q_heads, kv_heads, head_dim=128, epsilon=1e-5, theta=500000.0, angles=None):
    """One Llama-shaped decoder layer for one new token per sequence.

    residual-add + RMSNorm -> fused QKV linear -> RoPE on q and k with cache append and GQA decode
    attention (one call) -> o-proj -> residual-add + RMSNorm -> SwiGLU MLP. Returns (mlp output, residual).
    `weights` holds input_norm, qkv [ (Hq+2Hkv)*D, hidden ], o, post_norm, gate, up, down.
    `positions` (int32 [batch]) is the cache slot the new token is written to and rotated for;
    `lengths` (int32 [batch]) the number of valid cache positions afterwards (positions + 1).
    `angles` (optional): rope_angles(positions, head_dim, theta), made once per decode step for all layers.
    Every step is a call into libcamblas_hip.so, so the whole function can be captured in a graph
    after one warm-up call on the capture stream.
    """
    batch = hidden.shape[0]
    residual, normed = add_rms_norm(hidden, residual, weights["input_norm"], epsilon)
    qkv = linear(normed, weights["qkv"]).view(batch, q_heads + 2 * kv_heads, head_dim)
    # (rotary embedding, cache append and attention over positions + 1 entries: `lengths` is what that gives)
    attended = rope_append_attention(qkv, positions, k_cache, v_cache, q_heads=q_heads, kv_heads=kv_heads,
                                     theta=theta, angles=angles)
    projected = linear(attended.view(batch, q_heads * head_dim), weights["o"])
    residual, normed = add_rms_norm(projected, residual, weights["post_norm"], epsilon)
    return gated_mlp(normed, weights["gate"], weights["up"], weights["down"]), residual


def add_residual_squares(x, residual):
    """(added, squares, count): added = bf16(x + residual) and its rows' sums of squares, the state the
    fused decode linears pass along (count partial sums per row; here one)."""
    _require(x.is_cuda and x.dtype == residual.dtype == torch.bfloat16 and x.shape == residual.shape
             and x.dim() == 2 and x.is_contiguous() and residual.is_contiguous(),
             "add_residual_squares takes two contiguous BF16 [rows, width] device tensors")
    rows, width = x.shape
    added = torch.empty_like(x)
    squares = torch.empty((1, rows), dtype=torch.float32, device=x.device)
    _native.context(x.device).call("add_residual_squares", rows, width, _pointer(x), _pointer(residual),
                                   _pointer(added), _pointer(squares))
    return added, squares, 1


def _fused_linear_takes(x, weight):
    return (x.dtype == weight.dtype == torch.bfloat16 and x.is_cuda and x.dim() == 2 and weight.dim() == 2
            and 0 < x.shape[0] <= 64 and x.shape[1] == weight.shape[1] and x.stride(1) == 1
            and weight.stride(1) == 1 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0
            and weight.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def linear_residual(x, weight, residual):
    """(added, squares, count) with added = bf16(bf16(x weight^T) + residual): a decode linear with the
    residual add of the RMSNorm that follows it in its epilogue, plus per-workgroup partial sums of
    squares of the rows of `added` (squares[:count]) for the linear after that norm."""
    _require(_fused_linear_takes(x, weight), "linear_residual takes a BF16 decode batch (at most 64 rows)")
    rows, inner = x.shape
    outputs = weight.shape[0]
    _require(residual.dtype == torch.bfloat16 and tuple(residual.shape) == (rows, outputs)
             and residual.stride(1) == 1, "residual must be BF16 [rows, outputs]")
    added = torch.empty((rows, outputs), dtype=torch.bfloat16, device=x.device)
    capacity = (outputs + 15) // 16
    squares = torch.empty((capacity, rows), dtype=torch.float32, device=x.device)
    count = ct.c_int(0)
    _native.context(x.device).call(
        "bf16_linear_residual", rows, outputs, inner, _pointer(x), x.stride(0), _pointer(weight), weight.stride(0),
        _pointer(residual), residual.stride(0), _pointer(added), outputs, _pointer(squares), rows, capacity,
        ct.byref(count))
    return added, squares, count.value


def rms_linear(x, squares, count, norm_weight, epsilon, weight):
    """bf16(rms_norm(x) weight^T) for a BF16 decode batch, the normalisation done while the linear
    stages its tokens; x, squares, count as linear_residual / add_residual_squares return them."""
    _require(_fused_linear_takes(x, weight), "rms_linear takes a BF16 decode batch (at most 64 rows)")
    rows, inner = x.shape
    outputs = weight.shape[0]
    _require(norm_weight.dtype == torch.bfloat16 and norm_weight.numel() == inner and norm_weight.is_contiguous()
             and squares.dtype == torch.float32 and squares.dim() == 2 and squares.shape[1] >= rows
             and squares.stride(1) == 1 and 1 <= count <= squares.shape[0], "rms_linear norm operands")
    out = torch.empty((rows, outputs), dtype=torch.bfloat16, device=x.device)
    _native.context(x.device).call(
        "bf16_rms_linear", rows, outputs, inner, _pointer(x), x.stride(0), _pointer(squares), squares.stride(0),
        count, _pointer(norm_weight), ct.c_float(epsilon), _pointer(weight), weight.stride(0), _pointer(out), outputs)
    return out


def rms_gated_linear(x, squares, count, norm_weight, epsilon, gate_weight, up_weight):
    """gated_linear(rms_norm(x), gate, up) with the normalisation fused into the staging of x."""
    _require(_gated_linear_takes(x, gate_weight, up_weight), "rms_gated_linear takes a BF16 decode batch")
    rows, inner = x.shape
    outputs = gate_weight.shape[0]
    _require(norm_weight.dtype == torch.bfloat16 and norm_weight.numel() == inner and norm_weight.is_contiguous()
             and squares.dtype == torch.float32 and squares.dim() == 2 and squares.shape[1] >= rows
             and squares.stride(1) == 1 and 1 <= count <= squares.shape[0], "rms_gated_linear norm operands")
    out = torch.empty((rows, outputs), dtype=torch.bfloat16, device=x.device)
    _native.context(x.device).call(
        "bf16_rms_gated_linear", rows, outputs, inner, _pointer(x), x.stride(0), _pointer(squares),
        squares.stride(0), count, _pointer(norm_weight), ct.c_float(epsilon), _pointer(gate_weight),
        _pointer(up_weight), gate_weight.stride(0), _pointer(out), outputs)
    return out


def decoder_layer_decode_fused(state, weights, k_cache, v_cache, positions, lengths, *,
                               q_heads, kv_heads, head_dim=128, epsilon=1e-5, theta=500000.0, angles=None):
    """decoder_layer_decode with both residual-add + RMSNorm steps fused into the linears around them.

    `state` = (added, squares, count): the residual stream after the add that precedes this layer's
    input norm, with its rows' partial sums of squares (add_residual_squares makes it for the first
    layer; every layer returns the next one's). Six launches: QKV linear (normalising its input),
    rotary embedding + cache append, attention (two), o-proj (adding the residual), gate + up +
    SiLU-multiply (normalising its input), down projection (adding the residual). The values equal
    decoder_layer_decode's up to the order in which the sums of squares are added.
    """
    added, squares, count = state
    batch = added.shape[0]
    qkv = rms_linear(added, squares, count, weights["input_norm"], epsilon, weights["qkv"])
    qkv = qkv.view(batch, q_heads + 2 * kv_heads, head_dim)
    attended = rope_append_attention(qkv, positions, k_cache, v_cache, q_heads=q_heads, kv_heads=kv_heads,
                                     theta=theta, angles=angles)
    added, squares, count = linear_residual(attended.view(batch, q_heads * head_dim), weights["o"], added)
    hidden = rms_gated_linear(added, squares, count, weights["post_norm"], epsilon, weights["gate"], weights["up"])
    return linear_residual(hidden, weights["down"], added)


def __getattr__(name):
    """`QuantizedGroups` (captured expert weights, ref: camblas/_kernels.py:55) lives in the tensor
    binding; it is looked up on first use so that importing this module needs no built binding."""
    if name == "QuantizedGroups":
        module = _native.tensor_module()
        if module is None or not hasattr(module, "QuantizedGroups"):
            raise RuntimeError("QuantizedGroups requires the tensor binding (python camblas_amd/_build.py)")
        return module.QuantizedGroups
    raise AttributeError(name)
