"""Decoder-layer decode step (residual-add+RMSNorm -> QKV -> RoPE -> cache append -> GQA decode
attention -> o-proj -> RMSNorm -> SwiGLU MLP) against the same pipeline assembled from the CPU
oracle, eagerly and replayed from a captured graph.

Every stage rounds to BF16, so the composite tolerance is looser than a single operator's: relative
Frobenius <= 2e-2 on the MLP output (each stage alone meets 1e-2), <= 1e-2 on the residual stream.
Graph replays are checked against the eager result after every replay, with the inputs changed and
the stream synchronised in between.
"""

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels
from helpers import bf16_values, from_device_bf16, rel_frobenius, to_device_bf16

pytestmark = pytest.mark.gpu

BATCH, HIDDEN, Q_HEADS, KV_HEADS, DIM, FFN, CONTEXT = 4, 1024, 8, 2, 128, 2048, 300


def bf16_linear(x_bits, w_bits):
    return oracle.f32_to_bf16(oracle.linear_bf16_f64(x_bits, w_bits).astype(np.float32))


def make_inputs(seed, batch=BATCH):
    weights = {
        "input_norm": oracle.fill_normal_bf16(seed + 1, (HIDDEN,), mean=1.0, std=0.02),
        "post_norm": oracle.fill_normal_bf16(seed + 2, (HIDDEN,), mean=1.0, std=0.02),
        "qkv": oracle.fill_normal_bf16(seed + 3, ((Q_HEADS + 2 * KV_HEADS) * DIM, HIDDEN), std=0.03),
        "o": oracle.fill_normal_bf16(seed + 4, (HIDDEN, Q_HEADS * DIM), std=0.03),
        "gate": oracle.fill_normal_bf16(seed + 5, (FFN, HIDDEN), std=0.03),
        "up": oracle.fill_normal_bf16(seed + 6, (FFN, HIDDEN), std=0.03),
        "down": oracle.fill_normal_bf16(seed + 7, (HIDDEN, FFN), std=0.03),
    }
    hidden = oracle.fill_normal_bf16(seed + 8, (batch, HIDDEN))
    residual = oracle.fill_normal_bf16(seed + 9, (batch, HIDDEN))
    k_cache = oracle.fill_normal_bf16(seed + 10, (batch, CONTEXT, KV_HEADS, DIM))
    v_cache = oracle.fill_normal_bf16(seed + 11, (batch, CONTEXT, KV_HEADS, DIM))
    positions = np.array([CONTEXT - 1, 0, 17, 256], np.int32)
    if batch != BATCH:
        positions = np.random.default_rng(seed).integers(0, CONTEXT, batch).astype(np.int32)
    return weights, hidden, residual, k_cache, v_cache, positions


def oracle_layer(weights, hidden, residual, k_cache, v_cache, positions):
    # sizes come from the operands, so the same pipeline serves the full-size configuration
    BATCH, HIDDEN = hidden.shape
    KV_HEADS, DIM = k_cache.shape[2:]
    Q_HEADS = weights["qkv"].shape[0] // DIM - 2 * KV_HEADS
    k_cache, v_cache = k_cache.copy(), v_cache.copy()
    residual, normed = oracle.rms_norm(2, 2, 1e-5, hidden, weights["input_norm"], residual=residual)
    qkv = bf16_linear(normed, weights["qkv"]).reshape(BATCH, Q_HEADS + 2 * KV_HEADS, DIM)
    rotated = oracle.rope(qkv[:, : Q_HEADS + KV_HEADS], positions, 5e5)
    for b in range(BATCH):
        k_cache[b, positions[b]] = rotated[b, Q_HEADS:]
        v_cache[b, positions[b]] = qkv[b, Q_HEADS + KV_HEADS:]
    attended = oracle.gqa_decode(np.ascontiguousarray(rotated[:, :Q_HEADS]), k_cache, v_cache,
                                 positions + 1, DIM**-0.5)
    projected = bf16_linear(attended.reshape(BATCH, Q_HEADS * DIM), weights["o"])
    residual, normed = oracle.rms_norm(2, 2, 1e-5, projected, weights["post_norm"], residual=residual)
    gate, up = bf16_linear(normed, weights["gate"]), bf16_linear(normed, weights["up"])
    return bf16_linear(oracle.silu_multiply(2, gate, up), weights["down"]), residual, k_cache, v_cache


def device_layer(device, weights, hidden, residual, k_cache, v_cache, positions):
    KV_HEADS, DIM = k_cache.shape[2:]
    Q_HEADS = weights["qkv"].shape[0] // DIM - 2 * KV_HEADS
    w = {name: to_device_bf16(value, device) for name, value in weights.items()}
    kc, vc = to_device_bf16(k_cache, device), to_device_bf16(v_cache, device)
    pos = torch.from_numpy(positions).to(device)
    lengths = torch.from_numpy(positions + 1).to(device)
    out, res = _kernels.decoder_layer_decode(
        to_device_bf16(hidden, device), to_device_bf16(residual, device), w, kc, vc, pos, lengths,
        q_heads=Q_HEADS, kv_heads=KV_HEADS, head_dim=DIM)
    torch.cuda.synchronize()
    return out, res, kc, vc


@pytest.mark.parametrize("batch", [BATCH, 17, 40, 64, 80])
def test_layer_matches_oracle_pipeline(device, batch):
    # (the batches take the streaming linears with one to four token tiles, the gated launch included)
    inputs = make_inputs(3000 + batch, batch)
    want_out, want_res, want_k, want_v = oracle_layer(*inputs)
    out, res, kc, vc = device_layer(device, *inputs)
    assert rel_frobenius(bf16_values(res), oracle.bf16_to_f32(want_res)) <= 1e-2
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(want_out)) <= 2e-2
    # the cache rows that were not appended are untouched; the appended V row is a pure copy of a
    # linear output and the K row a rotation of one
    untouched = np.ones((batch, CONTEXT), bool)
    untouched[np.arange(batch), inputs[5]] = False
    assert np.array_equal(from_device_bf16(kc)[untouched], inputs[3][untouched])
    assert np.array_equal(from_device_bf16(vc)[untouched], inputs[4][untouched])
    assert rel_frobenius(bf16_values(vc), oracle.bf16_to_f32(want_v)) <= 1e-2
    assert rel_frobenius(bf16_values(kc), oracle.bf16_to_f32(want_k)) <= 1e-2


def test_layer_graph_replay_equals_eager(device):
    weights, hidden, residual, k_cache, v_cache, positions = make_inputs(4000)
    w = {name: to_device_bf16(value, device) for name, value in weights.items()}
    kc, vc = to_device_bf16(k_cache, device), to_device_bf16(v_cache, device)
    pos = torch.from_numpy(positions).to(device)
    lengths = torch.from_numpy(positions + 1).to(device)
    static_hidden = to_device_bf16(hidden, device)
    static_residual = to_device_bf16(residual, device)

    def run():
        return _kernels.decoder_layer_decode(static_hidden, static_residual, w, kc, vc, pos, lengths,
                                             q_heads=Q_HEADS, kv_heads=KV_HEADS, head_dim=DIM)

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        run()  # warm-up on the capture stream: creates the context, sizes its scratch
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        graph_out, graph_res = run()
    for replay in range(3):
        fresh = oracle.fill_normal_bf16(5000 + replay, (BATCH, HIDDEN))
        static_hidden.copy_(to_device_bf16(fresh, device))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_out, got_res = from_device_bf16(graph_out).copy(), from_device_bf16(graph_res).copy()
        eager_out, eager_res = run()
        torch.cuda.synchronize()
        assert np.array_equal(got_out, from_device_bf16(eager_out)), replay
        assert np.array_equal(got_res, from_device_bf16(eager_res)), replay
