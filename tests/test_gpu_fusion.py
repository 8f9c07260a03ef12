"""Decode epilogues (SiLU*up, SwiGLU, RMSNorm family, rotary embedding, GQA decode attention) and
the decoder-layer decode step against the CPU oracle.

The elementwise/RMS oracles restate src/cuda/inference_fusion.cuh; as in the reference's
tolerance-form tests (tests/test_residual_rms.py:64-69, tests/test_inference_fusion.py:64-101) the
GPU result may differ from the CPU one by one unit in the last place of the storage type where
expf/rsqrt or the reduction order differ; residual sums (pure BF16 adds) must be bit-exact.
RoPE and attention have no reference code: FP64 textbook formulas, relative Frobenius <= 1e-2.
"""

import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import (bf16_ulp_distance, bf16_values, from_device_bf16, ptr, rel_frobenius,
                     to_device_bf16)

pytestmark = pytest.mark.gpu


def close_bf16(got_bits, want_bits, ulps=1, exact_fraction=0.97):
    distance = bf16_ulp_distance(got_bits, want_bits)
    assert distance.max() <= ulps, distance.max()
    assert (distance == 0).mean() >= exact_fraction, (distance == 0).mean()


@pytest.mark.parametrize("count", [8 * 1000, 1001])
def test_silu_multiply_bf16(device, count):
    gate = oracle.fill_normal_bf16(1, (count,), std=3.0)
    up = oracle.fill_normal_bf16(2, (count,))
    out = _kernels.silu_multiply(to_device_bf16(gate, device), to_device_bf16(up, device))
    close_bf16(from_device_bf16(out), oracle.silu_multiply(2, gate, up))


def test_silu_multiply_f32_and_in_place(device):
    gate = oracle.fill_normal(3, (4099,), std=3.0)
    up = oracle.fill_normal(4, (4099,))
    g = torch.from_numpy(gate).to(device)
    out = _kernels.silu_multiply(g, torch.from_numpy(up).to(device), out=g)
    want = oracle.silu_multiply(0, gate, up)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-6, atol=1e-7)


@pytest.mark.parametrize("limit", [0.0, 1.5])
@pytest.mark.parametrize("routed", [False, True])
@pytest.mark.parametrize("width", [520, 515])  # eight values per thread, or one by one
def test_swiglu_bf16(device, limit, routed, width):
    rows = 7
    gate = oracle.fill_normal_bf16(5, (rows, width), std=2.0)
    up = oracle.fill_normal_bf16(6, (rows, width), std=2.0)
    routing = oracle.fill_uniform(7, (rows,), 0.1, 1.0) if routed else None
    out = _kernels.swiglu(to_device_bf16(gate, device), to_device_bf16(up, device), limit,
                          torch.from_numpy(routing).to(device) if routed else None)
    close_bf16(from_device_bf16(out), oracle.swiglu(2, width, limit, gate, up, routing))
    # NaN inputs survive the clamp (comparisons, not fmin/fmax)
    gate[0, 0] = 0x7FC0
    out = _kernels.swiglu(to_device_bf16(gate, device), to_device_bf16(up, device), limit)
    assert np.isnan(bf16_values(out)[0, 0])


@pytest.mark.parametrize("rows,width", [(32, 8192), (1, 2048), (3, 4104), (5, 1000), (2, 16384),
                                        (2, 32768), (1, 40008)])
@pytest.mark.parametrize("round_before_weight", [True, False])
def test_add_rms_norm_rows_bf16(device, rows, width, round_before_weight):
    x = oracle.fill_normal_bf16(10, (rows, width))
    r = oracle.fill_normal_bf16(11, (rows, width))
    w = oracle.fill_normal_bf16(12, (width,), mean=1.0, std=0.02)
    added, out = _kernels.add_rms_norm(to_device_bf16(x, device), to_device_bf16(r, device),
                                       to_device_bf16(w, device), 1e-5, round_before_weight)
    want_added, want_out = oracle.rms_norm(2, 2, 1e-5, x, w, residual=r,
                                           round_before_weight=round_before_weight)
    assert np.array_equal(from_device_bf16(added), want_added)
    close_bf16(from_device_bf16(out), want_out)
    plain = _kernels.rms_norm(to_device_bf16(x, device), to_device_bf16(w, device), 1e-5,
                              round_before_weight)
    close_bf16(from_device_bf16(plain),
               oracle.rms_norm(2, 2, 1e-5, x, w, round_before_weight=round_before_weight))


def test_reference_single_row_entry_points(device):
    width = 4096
    x = oracle.fill_normal_bf16(13, (1, width))
    r = oracle.fill_normal_bf16(14, (1, width))
    w = oracle.fill_normal_bf16(15, (width,), mean=1.0, std=0.1)
    native = _native.context(device)
    xt, rt, wt = (to_device_bf16(v, device) for v in (x, r, w))
    added, out = torch.empty_like(xt), torch.empty_like(xt)
    native.call("add_rms_norm", 2, width, ct.c_float(1e-6), ptr(xt), ptr(rt), ptr(wt), ptr(added),
                ptr(out))
    want_added, want_out = oracle.rms_norm(2, 2, 1e-6, x, w, residual=r)
    assert np.array_equal(from_device_bf16(added), want_added)
    close_bf16(from_device_bf16(out), want_out)
    wf = torch.from_numpy(oracle.bf16_to_f32(w)).to(device)
    native.call("rms_norm_decode", 2, 0, width, ct.c_float(1e-6), 0, 1, ptr(xt), ptr(wf), ptr(out))
    close_bf16(from_device_bf16(out),
               oracle.rms_norm(2, 0, 1e-6, x, oracle.bf16_to_f32(w), round_before_weight=False))
    native.call("rms_norm", 2, 1, width, ct.c_float(1e-6), ptr(xt), ptr(wt), ptr(out))
    close_bf16(from_device_bf16(out), oracle.rms_norm(2, 2, 1e-6, x, w))
    lib = _native.library()
    assert lib.camblas_cuda_add_rms_norm(native.handle, 2, 100, 1e-6, ptr(xt), ptr(rt), ptr(wt),
                                         ptr(added), ptr(out)) == -1
    assert b"invalid residual RMS arguments" in lib.camblas_cuda_error(native.handle)
    # squares + scale helpers keep the framework's own mean (ref: torch_bindings.cpp:654-666)
    squares = torch.empty((1, width), dtype=torch.float32, device=device)
    native.call("bfloat16_square", width, ptr(xt), ptr(squares))
    values = oracle.bf16_to_f32(x)
    assert np.array_equal(squares.cpu().numpy(), values * values)
    means = squares.mean(dim=1)
    native.call("rms_scale", 2, width, width, ct.c_float(1e-6), ptr(xt), ptr(wt), ptr(means),
                ptr(out))
    close_bf16(from_device_bf16(out), oracle.rms_norm(2, 2, 1e-6, x, w))


def test_rms_norm_f32(device):
    rows, width = 4, 3000
    x = oracle.fill_normal(16, (rows, width))
    w = oracle.fill_normal(17, (width,), mean=1.0, std=0.1)
    out = _kernels.rms_norm(torch.from_numpy(x).to(device), torch.from_numpy(w).to(device), 1e-6)
    np.testing.assert_allclose(out.cpu().numpy(), oracle.rms_norm(0, 0, 1e-6, x, w), rtol=3e-6)


def test_rope(device):
    tokens, heads, dim = 5, 9, 128
    x = oracle.fill_normal_bf16(20, (tokens, heads, dim))
    positions = np.array([0, 1, 17, 2047, 100000], np.int32)
    out = _kernels.rope(to_device_bf16(x, device), torch.from_numpy(positions).to(device), 5e5)
    want = oracle.rope(x, positions, 5e5)
    assert np.array_equal(from_device_bf16(out)[0], x[0])  # position 0 is the identity
    distance = bf16_ulp_distance(from_device_bf16(out)[:3], want[:3])
    assert distance.max() <= 1 and (distance == 0).mean() > 0.97
    wanted = oracle.bf16_to_f32(want)
    assert (np.abs(bf16_values(out) - wanted)[:4] <= 0.01 * np.abs(wanted[:4]) + 2e-3).all()
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(want)) <= 1e-2


def test_rope_over_many_tokens_equals_rope_over_few(device):
    # from 64 tokens on one workgroup per token works the angles out once for all heads; the result
    # must equal, bit for bit, the same tokens rotated 50 at a time by the kernel with one thread per
    # (token, head, pair); views with a token stride (the q and k heads of a fused activation) included
    tokens, heads, dim = 150, 9, 128
    x = oracle.fill_normal_bf16(21, (tokens, heads + 2, dim))
    positions = torch.from_numpy(np.arange(tokens, dtype=np.int32) * 37 % 5000).to(device)
    many, few = to_device_bf16(x, device), to_device_bf16(x, device)
    _kernels.rope(many[:, :heads], positions)
    for first in range(0, tokens, 50):
        _kernels.rope(few[first:first + 50, :heads], positions[first:first + 50])
    torch.cuda.synchronize()
    differing = np.argwhere(from_device_bf16(many) != from_device_bf16(few))
    assert len(differing) == 0, (len(differing), differing[:5])
    assert np.array_equal(from_device_bf16(many)[:, heads:], x[:, heads:])
    want = oracle.rope(x[:, :heads], positions.cpu().numpy(), 5e5)
    assert rel_frobenius(bf16_values(many[:, :heads]), oracle.bf16_to_f32(want)) <= 1e-2


@pytest.mark.parametrize("batch,q_heads,kv_heads,context", [(3, 16, 2, 700), (2, 8, 8, 256),
                                                            (2, 12, 4, 300), (1, 64, 8, 2048),
                                                            (3, 32, 2, 520), (2, 5, 5, 65)])
def test_gqa_decode_attention(device, batch, q_heads, kv_heads, context):
    dim = 128
    q = oracle.fill_normal_bf16(30, (batch, q_heads, dim))
    k = oracle.fill_normal_bf16(31, (batch, context, kv_heads, dim))
    v = oracle.fill_normal_bf16(32, (batch, context, kv_heads, dim))
    lengths = np.array([context, 1, 257][:batch], np.int32)
    scale = dim**-0.5
    out = _kernels.gqa_decode_attention(to_device_bf16(q, device), to_device_bf16(k, device),
                                        to_device_bf16(v, device),
                                        torch.from_numpy(lengths).to(device), scale)
    want = oracle.gqa_decode(q, k, v, lengths, scale)
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(want)) <= 1e-2
    wanted = oracle.bf16_to_f32(want)
    assert (np.abs(bf16_values(out) - wanted) <= 0.01 * np.abs(wanted) + 2e-3).all()
    # a single valid position returns that value row exactly
    if batch > 1:
        group = q_heads // kv_heads
        expect = np.repeat(v[1, 0], group, axis=0)
        assert np.array_equal(from_device_bf16(out)[1], expect)
    full = _kernels.gqa_decode_attention(to_device_bf16(q, device), to_device_bf16(k, device),
                                         to_device_bf16(v, device), None, scale)
    want_full = oracle.gqa_decode(q, k, v, None, scale)
    assert rel_frobenius(bf16_values(full), oracle.bf16_to_f32(want_full)) <= 1e-2


def test_gqa_decode_attention_empty_and_partial_partitions(device):
    # lengths 0 (no position: zeros), 64 and 65 (wavefront boundary), 256 and 259 (partition boundary)
    batch, q_heads, kv_heads, context, dim = 5, 16, 2, 600, 128
    q = oracle.fill_normal_bf16(40, (batch, q_heads, dim))
    k = oracle.fill_normal_bf16(41, (batch, context, kv_heads, dim))
    v = oracle.fill_normal_bf16(42, (batch, context, kv_heads, dim))
    lengths = np.array([0, 64, 65, 256, 259], np.int32)
    out = _kernels.gqa_decode_attention(to_device_bf16(q, device), to_device_bf16(k, device),
                                        to_device_bf16(v, device),
                                        torch.from_numpy(lengths).to(device), dim**-0.5)
    want = oracle.gqa_decode(q, k, v, np.maximum(lengths, 1), dim**-0.5)
    got = from_device_bf16(out)
    assert not got[0].any()
    wanted = oracle.bf16_to_f32(want)[1:]
    assert (np.abs(bf16_values(out)[1:] - wanted) <= 0.01 * np.abs(wanted) + 2e-3).all()


def test_gqa_decode_attention_short_sequences_in_a_long_cache(device):
    """Sixteen partitions per sequence, of which a sequence uses none to all: partitions past a
    sequence's length are neither computed nor read, whatever an earlier call left in the scratch
    (a first call with NaN queries over the whole cache leaves NaN in every partition record)."""
    batch, q_heads, kv_heads, context, dim = 6, 16, 2, 4096, 128
    q = oracle.fill_normal_bf16(43, (batch, q_heads, dim))
    k = oracle.fill_normal_bf16(44, (batch, context, kv_heads, dim))
    v = oracle.fill_normal_bf16(45, (batch, context, kv_heads, dim))
    k_device, v_device = to_device_bf16(k, device), to_device_bf16(v, device)
    poison = torch.full((batch, q_heads, dim), float("nan"), dtype=torch.bfloat16, device=device)
    _kernels.gqa_decode_attention(poison, k_device, v_device, None, dim**-0.5)
    lengths = np.array([0, 1, 255, 700, 2049, 4096], np.int32)
    out = _kernels.gqa_decode_attention(to_device_bf16(q, device), k_device, v_device,
                                        torch.from_numpy(lengths).to(device), dim**-0.5)
    want = oracle.gqa_decode(q, k, v, np.maximum(lengths, 1), dim**-0.5)
    assert not from_device_bf16(out)[0].any()
    wanted = oracle.bf16_to_f32(want)[1:]
    assert (np.abs(bf16_values(out)[1:] - wanted) <= 0.01 * np.abs(wanted) + 2e-3).all()


def test_rope_kv_append_equals_rope_then_append(device):
    # the fused launch must give bit-identical activations and caches, including a sequence whose
    # position lies outside the cache (rotated, not written)
    batch, q_heads, kv_heads, dim, context = 4, 6, 2, 128, 40
    qkv = oracle.fill_normal_bf16(50, (batch, q_heads + 2 * kv_heads, dim))
    k_cache = oracle.fill_normal_bf16(51, (batch, context, kv_heads, dim))
    v_cache = oracle.fill_normal_bf16(52, (batch, context, kv_heads, dim))
    positions = torch.tensor([0, 39, 17, 40], dtype=torch.int32, device=device)
    fused, kf, vf = (to_device_bf16(t, device) for t in (qkv, k_cache, v_cache))
    _kernels.rope_kv_append(fused, positions, kf, vf, q_heads=q_heads, kv_heads=kv_heads)
    split, ks, vs = (to_device_bf16(t, device) for t in (qkv, k_cache, v_cache))
    _kernels.rope(split[:, : q_heads + kv_heads], positions)
    _kernels.kv_append(split[:, q_heads : q_heads + kv_heads], split[:, q_heads + kv_heads :], ks, vs,
                       positions)
    torch.cuda.synchronize()
    assert np.array_equal(from_device_bf16(fused), from_device_bf16(split))
    assert np.array_equal(from_device_bf16(kf), from_device_bf16(ks))
    assert np.array_equal(from_device_bf16(vf), from_device_bf16(vs))
    assert np.array_equal(from_device_bf16(kf)[3], k_cache[3])  # position 40 is outside the cache
    want = oracle.rope(qkv[:, : q_heads + kv_heads], positions.cpu().numpy(), 5e5)
    assert rel_frobenius(bf16_values(fused[:, : q_heads + kv_heads]), oracle.bf16_to_f32(want)) <= 1e-2


@pytest.mark.parametrize("rows,outputs,inner,pairs", [(1, 100, 256, None), (7, 130, 264, 1), (32, 300, 512, 2),
                                                        (33, 70, 136, 3), (64, 257, 1024, 4), (32, 1024, 2048, None),
                                                        (40, 130, 264, 1), (48, 300, 512, 2), (47, 257, 1024, 4),
                                                        (48, 1024, 2048, None)])
def test_gated_linear_equals_the_three_call_composition(device, rows, outputs, inner, pairs):
    # one pass over both weight matrices against linear, linear, silu_multiply: the rounding points
    # are the same and only the order of the FP32 sums inside a product may differ (the planner is
    # free to give the separate products another kernel), so the two agree to a few BF16 units in
    # a few places; and the oracle's composition holds within the BF16 bar
    from camblas_amd import _native

    x = oracle.fill_normal_bf16(500 + rows, (rows, inner))
    gate = oracle.fill_normal_bf16(501, (outputs, inner), std=0.05)
    up = oracle.fill_normal_bf16(502, (outputs, inner), std=0.05)
    xt, gt, ut = (to_device_bf16(v, device) for v in (x, gate, up))
    native = _native.context(device)
    if pairs is not None:
        native.call("hip_set_plan_override", pairs, 0)
    try:
        fused = _kernels.gated_linear(xt, gt, ut)
    finally:
        native.call("hip_set_plan_override", -1, 0)
    g, u = _kernels.linear(xt, gt), _kernels.linear(xt, ut)
    composed = _kernels.silu_multiply(g, u)
    torch.cuda.synchronize()
    assert rel_frobenius(bf16_values(fused), bf16_values(composed)) <= 4e-3
    want_g = oracle.f32_to_bf16(oracle.linear_bf16_f64(x, gate).astype(np.float32))
    want_u = oracle.f32_to_bf16(oracle.linear_bf16_f64(x, up).astype(np.float32))
    want = oracle.bf16_to_f32(oracle.silu_multiply(2, want_g, want_u))
    assert rel_frobenius(bf16_values(fused), want) <= 2e-2  # two BF16-rounded products, then two roundings


def test_gated_linear_refuses_what_it_does_not_take(device):
    import ctypes as ct

    from camblas_amd import _native
    from helpers import ptr

    native, lib = _native.context(device), _native.library()
    x = torch.zeros((65, 64), dtype=torch.bfloat16, device=device)
    w = torch.zeros((32, 64), dtype=torch.bfloat16, device=device)
    out = torch.zeros((65, 32), dtype=torch.bfloat16, device=device)
    call = lib.camblas_cuda_bf16_gated_linear
    assert call(native.handle, 65, 32, 64, ptr(x), 64, ptr(w), ptr(w), 64, ptr(out), 32) == -1
    assert b"invalid gated linear dimensions" in lib.camblas_cuda_error(native.handle)
    assert call(native.handle, 8, 32, 60, ptr(x), 64, ptr(w), ptr(w), 64, ptr(out), 32) == -1
    assert call(native.handle, 8, 32, 64, ptr(x), 64, ptr(w), ptr(w), 64, ptr(x), 32) == -1
    assert b"invalid gated linear buffers" in lib.camblas_cuda_error(native.handle)
    assert call(native.handle, 0, 32, 64, None, 64, None, None, 64, None, 32) == 0
