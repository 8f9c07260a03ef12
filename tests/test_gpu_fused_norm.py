"""The residual-add + RMSNorm of a decoder layer fused into the decode linears around it.

The norm's arithmetic is the reference's (src/cuda/inference_fusion.cuh:136-191; closed form quoted in
its tests/test_residual_rms.py:46-80): added = bf16(x + r), scale = rsqrt(mean(added^2) + eps),
out = bf16(bf16(added * scale) * w). Here the linear before the norm does the add in its epilogue and
leaves per-workgroup sums of squares, and the linear after it forms the scale and normalises its input
while staging it. What is checked:
  * `added` equals, bit for bit, what the separate calls give (same linear kernel, same rounding
    points), and the partial sums of squares add up to the row sums (FP64 yardstick), run to run
    identically;
  * with values whose squares and sums are exact in FP32 (so that the order of the sum cannot
    matter) the fused linears equal the separate norm + linear bit for bit;
  * on ordinary data they meet the BF16 bar (relative Frobenius error <= 1e-2) against the oracle
    pipeline in FP64 and stay within one BF16 rounding step of the separate calls;
  * a whole fused layer step against the unfused one and the oracle; graph replay against eager.
"""

import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import bf16_values, from_device_bf16, ptr, rel_frobenius, to_device_bf16
from test_gpu_layer import BATCH, DIM, HIDDEN, KV_HEADS, Q_HEADS, make_inputs, oracle_layer

pytestmark = pytest.mark.gpu

EPSILON = 1e-5
SHAPES = [(1, 512, 1024), (7, 300, 328), (32, 1152, 2048), (32, 4096, 1024), (17, 8192, 512), (64, 2048, 1024),
          (33, 640, 4096)]


def operands(device, seed, tokens, outputs, inner):
    x = oracle.fill_normal_bf16(seed, (tokens, inner))
    w = oracle.fill_normal_bf16(seed + 1, (outputs, inner), std=0.03)
    r = oracle.fill_normal_bf16(seed + 2, (tokens, outputs))
    return (x, w, r), tuple(to_device_bf16(v, device) for v in (x, w, r))


@pytest.mark.parametrize("tokens,outputs,inner", SHAPES)
def test_linear_residual_against_the_separate_calls(device, tokens, outputs, inner):
    (x, w, r), (xd, wd, rd) = operands(device, 7100 + tokens, tokens, outputs, inner)
    added, squares, count = _kernels.linear_residual(xd, wd, rd)
    again = _kernels.linear_residual(xd, wd, rd)
    torch.cuda.synchronize()
    assert 1 <= count <= (outputs + 15) // 16
    # the oracle's pipeline in FP64 with the same rounding points
    product = oracle.f32_to_bf16(oracle.linear_bf16_f64(x, w).astype(np.float32))
    want = oracle.f32_to_bf16(oracle.bf16_to_f32(product) + oracle.bf16_to_f32(r))
    assert rel_frobenius(bf16_values(added), oracle.bf16_to_f32(want)) <= 1e-2
    # sums of squares: the partial sums add up to the rows' sums (of the values the kernel wrote)
    got = bf16_values(added).astype(np.float64)
    total = squares[:count].double().sum(0).cpu().numpy()
    assert np.allclose(total, (got * got).sum(1), rtol=1e-5, atol=0)
    # bit for bit what the plain linear followed by the norm kernel's add gives, wherever the plain linear
    # runs the same kernel (the planner sends 33 to 64 tokens on narrow projections to other tiles)
    plain = _kernels.linear(xd, wd)
    separate, _ = _kernels.add_rms_norm(plain, rd, torch.ones(outputs, dtype=torch.bfloat16, device=device), EPSILON)
    torch.cuda.synchronize()
    if tokens <= 32:
        assert np.array_equal(from_device_bf16(added), from_device_bf16(separate))
    else:
        assert rel_frobenius(bf16_values(added), bf16_values(separate)) <= 1e-2
    # and the same on a second run, partial sums included
    assert again[2] == count
    assert np.array_equal(from_device_bf16(added), from_device_bf16(again[0]))
    assert torch.equal(squares[:count], again[1][:count])


def exact_state(device, seed, tokens, width):
    # rows of values from {-2, -1, -0.5, 0.5, 1, 2}: squares and their sums are exact in FP32 in any order
    rng = np.random.default_rng(seed)
    values = rng.choice(np.array([-2, -1, -0.5, 0.5, 1, 2], np.float32), size=(tokens, width))
    x = oracle.f32_to_bf16(values)
    zero = oracle.f32_to_bf16(np.zeros((tokens, width), np.float32))
    return x, _kernels.add_residual_squares(to_device_bf16(x, device), to_device_bf16(zero, device))


@pytest.mark.parametrize("tokens,outputs,inner", SHAPES)
def test_rms_linear_equals_norm_then_linear_when_the_sums_are_exact(device, tokens, outputs, inner):
    x, (added, squares, count) = exact_state(device, 7200 + tokens, tokens, inner)
    assert count == 1 and np.array_equal(from_device_bf16(added), x)
    values = oracle.bf16_to_f32(x).astype(np.float64)
    assert np.array_equal(squares[0].cpu().numpy(), (values * values).sum(1).astype(np.float32))
    norm_weight = to_device_bf16(oracle.fill_normal_bf16(7300, (inner,), mean=1.0, std=0.1), device)
    w = to_device_bf16(oracle.fill_normal_bf16(7301 + tokens, (outputs, inner), std=0.03), device)
    fused = _kernels.rms_linear(added, squares, count, norm_weight, EPSILON, w)
    normed = _kernels.rms_norm(added, norm_weight, EPSILON)
    separate = _kernels.linear(normed, w)
    torch.cuda.synchronize()
    if tokens <= 32:
        assert np.array_equal(from_device_bf16(fused), from_device_bf16(separate))
    else:
        assert rel_frobenius(bf16_values(fused), bf16_values(separate)) <= 1e-2
    # several partial sums per row instead of one: split each row's sum into pieces (still exact)
    pieces = 5
    split = torch.zeros((pieces, tokens), dtype=torch.float32, device=device)
    split[0] = squares[0] - 3.0
    split[2] = 1.0
    split[4] = 2.0
    spread = _kernels.rms_linear(added, split, pieces, norm_weight, EPSILON, w)
    torch.cuda.synchronize()
    assert np.array_equal(from_device_bf16(spread), from_device_bf16(fused))


@pytest.mark.parametrize("tokens,outputs,inner", [(1, 512, 1024), (32, 1024, 2048), (48, 1408, 1024), (9, 264, 520)])
def test_rms_gated_linear_equals_norm_then_gated_linear_when_the_sums_are_exact(device, tokens, outputs, inner):
    x, (added, squares, count) = exact_state(device, 7400 + tokens, tokens, inner)
    norm_weight = to_device_bf16(oracle.fill_normal_bf16(7500, (inner,), mean=1.0, std=0.1), device)
    gate = to_device_bf16(oracle.fill_normal_bf16(7501, (outputs, inner), std=0.03), device)
    up = to_device_bf16(oracle.fill_normal_bf16(7502, (outputs, inner), std=0.03), device)
    fused = _kernels.rms_gated_linear(added, squares, count, norm_weight, EPSILON, gate, up)
    separate = _kernels.gated_linear(_kernels.rms_norm(added, norm_weight, EPSILON), gate, up)
    torch.cuda.synchronize()
    assert np.array_equal(from_device_bf16(fused), from_device_bf16(separate))


@pytest.mark.parametrize("tokens,outputs,inner", [(32, 1152, 2048), (5, 304, 328), (64, 2048, 1024)])
def test_chain_of_fused_linears_on_ordinary_data(device, tokens, outputs, inner):
    # o-proj-like linear with the residual add, then the linear that consumes its state
    (x, w, r), (xd, wd, rd) = operands(device, 7600 + tokens, tokens, outputs, inner)
    norm = oracle.fill_normal_bf16(7700, (outputs,), mean=1.0, std=0.05)
    w2 = oracle.fill_normal_bf16(7701, (520, outputs), std=0.03)
    added, squares, count = _kernels.linear_residual(xd, wd, rd)
    fused = _kernels.rms_linear(added, squares, count, to_device_bf16(norm, device), EPSILON, to_device_bf16(w2, device))
    separate = _kernels.linear(_kernels.rms_norm(added, to_device_bf16(norm, device), EPSILON), to_device_bf16(w2, device))
    torch.cuda.synchronize()
    # oracle: the norm (FP64 sums) of the device's own `added`, then the linear in FP64
    normed = oracle.rms_norm(2, 2, EPSILON, np.ascontiguousarray(from_device_bf16(added)), norm)
    want = oracle.linear_bf16_f64(normed, w2)
    assert rel_frobenius(bf16_values(fused), want) <= 1e-2
    # the scale can differ from the row kernel's in its last bit, which moves single outputs by a rounding step
    difference = np.abs(bf16_values(fused) - bf16_values(separate))
    assert (difference <= 2.0 ** -7 * np.abs(bf16_values(separate)) + 1e-30).all()


def test_refusals(device):
    native = _native.context(device)
    x = torch.zeros((65, 256), dtype=torch.bfloat16, device=device)
    w = torch.zeros((64, 256), dtype=torch.bfloat16, device=device)
    r = torch.zeros((65, 64), dtype=torch.bfloat16, device=device)
    squares = torch.zeros((4, 65), dtype=torch.float32, device=device)
    count = ct.c_int(-1)
    with pytest.raises(RuntimeError, match="invalid fused linear dimensions"):  # more than 64 tokens
        native.call("bf16_linear_residual", 65, 64, 256, ptr(x), 256, ptr(w), 256, ptr(r), 64, ptr(r), 64,
                    ptr(squares), 65, 4, ct.byref(count))
    assert count.value == 0
    with pytest.raises(RuntimeError, match="room for the partial sums of squares"):
        native.call("bf16_linear_residual", 8, 64, 256, ptr(x), 256, ptr(w), 256, ptr(r), 64, ptr(r[8:]), 64,
                    ptr(squares), 65, 0, ct.byref(count))
    with pytest.raises(RuntimeError, match="invalid fused linear dimensions"):  # no partial sums to add
        native.call("bf16_rms_linear", 8, 64, 256, ptr(x), 256, ptr(squares), 65, 0, ptr(w), ct.c_float(1e-5),
                    ptr(w), 256, ptr(r), 64)
    torch.cuda.synchronize()


def fused_layer(device, weights, hidden, residual, k_cache, v_cache, positions):
    w = {name: to_device_bf16(value, device) for name, value in weights.items()}
    kc, vc = to_device_bf16(k_cache, device), to_device_bf16(v_cache, device)
    pos = torch.from_numpy(positions).to(device)
    lengths = torch.from_numpy(positions + 1).to(device)
    state = _kernels.add_residual_squares(to_device_bf16(hidden, device), to_device_bf16(residual, device))
    nxt = _kernels.decoder_layer_decode_fused(state, w, kc, vc, pos, lengths, q_heads=Q_HEADS, kv_heads=KV_HEADS,
                                              head_dim=DIM)
    torch.cuda.synchronize()
    return state, nxt, kc, vc


def test_fused_layer_step_against_the_oracle_and_the_unfused_step(device):
    inputs = make_inputs(3000)
    weights, hidden, residual, k_cache, v_cache, positions = inputs
    want_out, want_res, want_k, want_v = oracle_layer(*inputs)
    state, (added, squares, count), kc, vc = fused_layer(device, *inputs)
    # the state that enters the next layer is the residual stream plus this layer's MLP output
    want_next = oracle.f32_to_bf16(oracle.bf16_to_f32(want_out) + oracle.bf16_to_f32(want_res))
    assert rel_frobenius(bf16_values(added), oracle.bf16_to_f32(want_next)) <= 2e-2
    assert rel_frobenius(bf16_values(vc), oracle.bf16_to_f32(want_v)) <= 1e-2
    assert rel_frobenius(bf16_values(kc), oracle.bf16_to_f32(want_k)) <= 1e-2
    got = bf16_values(added).astype(np.float64)
    assert np.allclose(squares[:count].double().sum(0).cpu().numpy(), (got * got).sum(1), rtol=1e-5)
    # against the unfused step on the same device: same kernels apart from where the norm happens
    w = {name: to_device_bf16(value, device) for name, value in weights.items()}
    kc2, vc2 = to_device_bf16(k_cache, device), to_device_bf16(v_cache, device)
    pos = torch.from_numpy(positions).to(device)
    out, res = _kernels.decoder_layer_decode(to_device_bf16(hidden, device), to_device_bf16(residual, device), w,
                                             kc2, vc2, pos, pos + 1, q_heads=Q_HEADS, kv_heads=KV_HEADS, head_dim=DIM)
    torch.cuda.synchronize()
    unfused_next = oracle.f32_to_bf16(bf16_values(out) + bf16_values(res))
    assert rel_frobenius(bf16_values(added), oracle.bf16_to_f32(unfused_next)) <= 1e-2
    assert np.array_equal(from_device_bf16(state[0]),
                          oracle.f32_to_bf16(oracle.bf16_to_f32(hidden) + oracle.bf16_to_f32(residual)))


def test_fused_layer_graph_replay_equals_eager(device):
    weights, hidden, residual, k_cache, v_cache, positions = make_inputs(4100)
    w = {name: to_device_bf16(value, device) for name, value in weights.items()}
    kc, vc = to_device_bf16(k_cache, device), to_device_bf16(v_cache, device)
    pos = torch.from_numpy(positions).to(device)
    lengths = torch.from_numpy(positions + 1).to(device)
    static_hidden = to_device_bf16(hidden, device)
    static_residual = to_device_bf16(residual, device)

    def run():
        state = _kernels.add_residual_squares(static_hidden, static_residual)
        return _kernels.decoder_layer_decode_fused(state, w, kc, vc, pos, lengths, q_heads=Q_HEADS,
                                                   kv_heads=KV_HEADS, head_dim=DIM)

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        run()  # warm-up on the capture stream: creates the context, sizes its scratch
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        graph_added, graph_squares, graph_count = run()
    for replay in range(3):
        fresh = oracle.fill_normal_bf16(5100 + replay, (BATCH, HIDDEN))
        static_hidden.copy_(to_device_bf16(fresh, device))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_added, got_squares = from_device_bf16(graph_added).copy(), graph_squares[:graph_count].clone()
        eager_added, eager_squares, eager_count = run()
        torch.cuda.synchronize()
        assert eager_count == graph_count
        assert np.array_equal(got_added, from_device_bf16(eager_added)), replay
        assert torch.equal(got_squares, eager_squares[:eager_count]), replay
