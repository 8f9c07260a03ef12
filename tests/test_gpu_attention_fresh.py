"""Rotary embedding + cache append folded into the decode attention's partition kernel, against the
separate calls (rope_kv_append, then gqa_decode_attention over positions + 1 entries) and the oracle.

The two routes run the same arithmetic (one shared rotation routine, the same products), so outputs
and caches must agree bit for bit: slots at the start and end of wavefronts (64 positions) and of
partitions (256), the first and the last slot of the cache, every query-group size, slots outside the
cache, and caches whose unused part holds NaN (nothing beyond a sequence's length may reach a sum).
"""

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels
from helpers import bf16_values, from_device_bf16, rel_frobenius, to_device_bf16

pytestmark = pytest.mark.gpu
DIM = 128


def case(device, seed, batch, q_heads, kv_heads, context, positions, poison=True):
    qkv = oracle.fill_normal_bf16(seed, (batch, q_heads + 2 * kv_heads, DIM))
    k = oracle.fill_normal_bf16(seed + 1, (batch, context, kv_heads, DIM))
    v = oracle.fill_normal_bf16(seed + 2, (batch, context, kv_heads, DIM))
    positions = np.asarray(positions, np.int32)
    if poison:  # everything from the new token's slot on is garbage until it is appended
        for b, slot in enumerate(positions):
            k[b, max(slot, 0):] = 0x7fc0
            v[b, max(slot, 0):] = 0x7fc0
    return qkv, k, v, positions


def both_routes(device, qkv, k, v, positions, q_heads, kv_heads):
    pos = torch.from_numpy(positions).to(device)
    a_qkv, a_k, a_v = (to_device_bf16(t, device) for t in (qkv, k, v))
    _kernels.rope_kv_append(a_qkv, pos, a_k, a_v, q_heads=q_heads, kv_heads=kv_heads)
    separate = _kernels.gqa_decode_attention(a_qkv[:, :q_heads], a_k, a_v, pos + 1)
    b_qkv, b_k, b_v = (to_device_bf16(t, device) for t in (qkv, k, v))
    folded = _kernels.rope_append_attention(b_qkv, pos, b_k, b_v, q_heads=q_heads, kv_heads=kv_heads)
    # the same with the step's angles handed in instead of worked out by every workgroup
    c_k, c_v = to_device_bf16(k, device), to_device_bf16(v, device)
    tabled = _kernels.rope_append_attention(b_qkv, pos, c_k, c_v, q_heads=q_heads, kv_heads=kv_heads,
                                            angles=_kernels.rope_angles(pos))
    torch.cuda.synchronize()
    assert np.array_equal(from_device_bf16(b_qkv), qkv)  # the activation itself is left as it was
    assert np.array_equal(from_device_bf16(tabled), from_device_bf16(folded))
    assert np.array_equal(from_device_bf16(c_k), from_device_bf16(b_k))
    assert np.array_equal(from_device_bf16(c_v), from_device_bf16(b_v))
    return (separate, a_k, a_v), (folded, b_k, b_v)


@pytest.mark.parametrize("q_heads,kv_heads", [(8, 1), (16, 4), (4, 4), (16, 1)])
@pytest.mark.parametrize("context,positions", [
    (300, [0, 63, 64, 255, 256, 299]),
    (1024, [1023, 511, 512, 767, 1, 700]),
    (257, [256, 255, 128, 0, 200, 17]),
])
def test_folded_route_equals_the_separate_calls(device, q_heads, kv_heads, context, positions):
    qkv, k, v, positions = case(device, 8100 + context, len(positions), q_heads, kv_heads, context, positions)
    (separate, a_k, a_v), (folded, b_k, b_v) = both_routes(device, qkv, k, v, positions, q_heads, kv_heads)
    assert not np.isnan(bf16_values(folded)).any()
    assert np.array_equal(from_device_bf16(folded), from_device_bf16(separate))
    assert np.array_equal(from_device_bf16(b_k), from_device_bf16(a_k))
    assert np.array_equal(from_device_bf16(b_v), from_device_bf16(a_v))


def test_folded_route_against_the_oracle(device):
    q_heads, kv_heads, context = 16, 2, 600
    positions = [599, 0, 300, 255]
    qkv, k, v, positions = case(device, 8300, 4, q_heads, kv_heads, context, positions, poison=False)
    pos = torch.from_numpy(positions).to(device)
    dk, dv = to_device_bf16(k, device), to_device_bf16(v, device)
    out = _kernels.rope_append_attention(to_device_bf16(qkv, device), pos, dk, dv, q_heads=q_heads, kv_heads=kv_heads)
    torch.cuda.synchronize()
    rotated = oracle.rope(qkv[:, : q_heads + kv_heads], positions, 5e5)
    for b in range(4):
        k[b, positions[b]] = rotated[b, q_heads:]
        v[b, positions[b]] = qkv[b, q_heads + kv_heads:]
    want = oracle.gqa_decode(np.ascontiguousarray(rotated[:, :q_heads]), k, v, positions + 1, DIM**-0.5)
    assert rel_frobenius(bf16_values(out), oracle.bf16_to_f32(want)) <= 1e-2
    assert np.array_equal(from_device_bf16(dv), v)
    assert rel_frobenius(bf16_values(dk), oracle.bf16_to_f32(k)) <= 1e-2


def test_slots_outside_the_cache_append_nothing(device):
    q_heads, kv_heads, context = 8, 2, 320
    qkv, k, v, positions = case(device, 8400, 3, q_heads, kv_heads, context, [-1, 320, 5000], poison=False)
    (separate, a_k, a_v), (folded, b_k, b_v) = both_routes(device, qkv, k, v, positions, q_heads, kv_heads)
    assert np.array_equal(from_device_bf16(b_k), k) and np.array_equal(from_device_bf16(b_v), v)
    # slot -1: no entries, zeros; slots past the cache: the whole cache, no new token
    assert not bf16_values(folded)[0].any()
    assert np.array_equal(from_device_bf16(folded), from_device_bf16(separate))
