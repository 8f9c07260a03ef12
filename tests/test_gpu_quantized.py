"""E8M0 block-scaled (microscaling) linear through the C ABI: E4M3 and packed E2M1 weights, scale
extremes and NaN, the grouped form. Strategy and tolerances of the reference's
tests/test_quantized.py:12-158 and :243-320: an independent FP64 byte decoder (oracle.mx_dequantise),
rtol 0.008 / atol 0.02 for random operands, exact equality (NaN included) where every product is
exactly representable."""

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import bf16_values

pytestmark = pytest.mark.gpu


def operands(seed, rows, outputs, inner, packed, block):
    rng = np.random.default_rng(seed)
    x = oracle.f32_to_e4m3((rng.standard_normal((rows, inner)) * 8).astype(np.float32))
    if packed:
        weight = rng.integers(0, 256, (outputs, inner // 2), dtype=np.uint8)
    else:
        weight = oracle.f32_to_e4m3((rng.standard_normal((outputs, inner)) * 4).astype(np.float32))
    sx = rng.integers(122, 129, (rows, inner // block), dtype=np.uint8)
    sw = rng.integers(121, 128, (outputs if packed else (outputs + 31) // 32, inner // 32), dtype=np.uint8)
    return x, sx, weight, sw


def run(device, x, sx, weight, sw, packed, block):
    xt = torch.from_numpy(x).to(device).view(torch.float8_e4m3fn)
    wt = torch.from_numpy(weight).to(device)
    if not packed:
        wt = wt.view(torch.float8_e4m3fn)
    out = _kernels.quantized_matmul(xt, torch.from_numpy(sx).to(device), wt, torch.from_numpy(sw).to(device),
                                    activation_block=block)
    torch.cuda.synchronize()
    return bf16_values(out)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,outputs,inner", [(1, 8, 32), (3, 40, 256), (7, 40, 256), (8, 40, 256),
                                               (17, 40, 256), (33, 40, 256), (128, 40, 256),
                                               (1, 2304, 5120), (1, 5120, 2304), (70, 264, 416)])
def test_random_operands_and_individual_mutations(device, packed, rows, outputs, inner):
    # every operand is changed separately so that a stale or mis-indexed buffer cannot hide
    # (ref: tests/test_quantized.py:110-158); 416 = 3.25 groups of 128 exercises the K tail
    block = 128 if packed and inner % 128 == 0 and rows > 1 else 32
    x, sx, weight, sw = operands(700 + rows, rows, outputs, inner, packed, block)
    for changed in ("original", "input", "weight", "input_scale", "weight_scale"):
        if changed == "input":
            x ^= 128
        elif changed == "weight":
            weight ^= 17 if packed else 128
            if not packed:
                weight[(weight & 0x7F) == 0x7F] = 0x38  # keep the weights finite
        elif changed == "input_scale":
            sx -= 1
        elif changed == "weight_scale":
            sw += 1
        got = run(device, x, sx, weight, sw, packed, block)
        want = oracle.mx_matmul_f64(x, sx, weight, sw, block, packed)
        assert got.shape == want.shape
        assert (np.abs(got - want) <= 0.02 + 0.008 * np.abs(want)).all(), changed


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,outputs,inner", [(16, 18440, 256), (20, 18440, 160), (40, 12296, 96)])
def test_wide_workgroups_and_unaligned_scales(device, packed, rows, outputs, inner):
    # enough outputs for workgroups of several row tiles, a last workgroup that is cut short, and
    # scale arrays that start at an odd address (they are byte arrays: nothing aligns them)
    x, sx, weight, sw = operands(4100 + rows, rows, outputs, inner, packed, 32)
    xt = torch.from_numpy(x).to(device).view(torch.float8_e4m3fn)
    wt = torch.from_numpy(weight).to(device)
    if not packed:
        wt = wt.view(torch.float8_e4m3fn)

    def shifted(array, shift):
        buffer = torch.zeros(array.size + 16, dtype=torch.uint8, device=device)
        view = buffer[shift:shift + array.size].view(array.shape)
        view.copy_(torch.from_numpy(array).to(device))
        return view

    out = _kernels.quantized_matmul(xt, shifted(sx, 3), wt, shifted(sw, 5), activation_block=32)
    torch.cuda.synchronize()
    got = bf16_values(out)
    xd = oracle.mx_dequantise(x, sx, 32)
    wd = oracle.mx_dequantise(weight, sw, 32, packed, True)
    want = xd @ wd.T
    # Among 300 000 outputs a few sums cancel to nearly nothing, so the reference's fixed absolute
    # tolerance gives way to one that follows the size of the terms: FP32 accumulation may lose
    # 2^-13 of the sum of the products' magnitudes (measured worst case about 2^-15).
    magnitude = np.abs(xd) @ np.abs(wd).T
    assert (np.abs(got - want) <= 0.008 * np.abs(want) + magnitude * 2.0 ** -13).all()
    assert np.linalg.norm(got - want) <= 4e-3 * np.linalg.norm(want)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows", [1, 8, 17])
def test_scale_extremes_and_nan(device, packed, rows):
    # ones times ones with unit weight scales: exact for input scales 2^-127, 1, 2^127 and NaN for
    # the scale byte 255; a NaN input or weight byte poisons exactly its row / column
    # (ref: tests/test_quantized.py:243-280)
    outputs, inner = 40, 64
    x = np.full((rows, inner), 0x38, np.uint8)
    weight = np.full((outputs, inner // 2), 0x22, np.uint8) if packed else np.full((outputs, inner), 0x38, np.uint8)
    sw = np.full((outputs if packed else 2, inner // 32), 127, np.uint8)
    for exponent in (0, 127, 254, 255):
        sx = np.full((rows, inner // 32), exponent, np.uint8)
        got = run(device, x, sx, weight, sw, packed, 32)
        with np.errstate(over="ignore"):
            want = oracle.bf16_to_f32(oracle.f32_to_bf16(
                oracle.mx_matmul_f64(x, sx, weight, sw, 32, packed).astype(np.float32)))
        assert np.array_equal(got, want, equal_nan=True), exponent
    sx = np.full((rows, inner // 32), 127, np.uint8)
    poisoned = x.copy()
    poisoned[rows - 1, 5] = 0x7F
    got = run(device, poisoned, sx, weight, sw, packed, 32)
    assert np.isnan(got[rows - 1]).all() and (got[: rows - 1] == inner).all()
    if not packed:
        bad = weight.copy()
        bad[3, 40] = 0xFF
        got = run(device, x, sx, bad, sw, packed, 32)
        assert np.isnan(got[:, 3]).all() and (np.delete(got, 3, axis=1) == inner).all()


@pytest.mark.parametrize("packed", [False, True])
def test_grouped_products(device, packed):
    # ref: include/camblas_cuda.h:156-167 — weights chosen per group through a device table, an
    # invalid index gives zeros, counts clip the rows, padding rows are zero
    groups, weight_groups, rows, outputs, inner = 5, 3, 20, 48, 256
    rng = np.random.default_rng(9)
    x = oracle.f32_to_e4m3((rng.standard_normal((groups, rows, inner)) * 8).astype(np.float32))
    sx = rng.integers(122, 129, (groups, rows, inner // 32), dtype=np.uint8)
    weights, scales = [], []
    for g in range(weight_groups):
        _, _, w, sw = operands(800 + g, 1, outputs, inner, packed, 32)
        weights.append(torch.from_numpy(w).to(device))
        scales.append(torch.from_numpy(sw).to(device))
    metadata = torch.tensor([[w.data_ptr(), s.data_ptr()] for w, s in zip(weights, scales)],
                            dtype=torch.int64, device=device)
    active = torch.tensor([2, 0, 7, 1, -1], dtype=torch.int32, device=device)
    counts = torch.tensor([20, 5, 20, 99, 3], dtype=torch.int32, device=device)
    out = _kernels.grouped_quantized_matmul(
        torch.from_numpy(x).to(device).view(torch.float8_e4m3fn), torch.from_numpy(sx).to(device),
        metadata, active, counts, outputs=outputs, packed=packed)
    torch.cuda.synchronize()
    got = bf16_values(out)
    for g, (index, count) in enumerate(zip(active.tolist(), counts.tolist())):
        if not 0 <= index < weight_groups:
            assert not got[g].any()
            continue
        count = min(max(count, 0), rows)
        want = oracle.mx_matmul_f64(x[g], sx[g], weights[index].cpu().numpy(), scales[index].cpu().numpy(), 32, packed)
        assert (np.abs(got[g, :count] - want[:count]) <= 0.02 + 0.008 * np.abs(want[:count])).all()
        assert not got[g, count:].any()


@pytest.mark.parametrize("packed", [False, True])
def test_grouped_decode_with_many_groups_uses_wide_workgroups(device, packed):
    # 40 groups of a few rows: the streaming kernel sizes its workgroups with all groups counted
    # (eight 16-row tiles each here, the last workgroup of a group cut short at 1032 outputs)
    groups, weight_groups, rows, outputs, inner = 40, 4, 5, 1032, 256
    rng = np.random.default_rng(29)
    x = oracle.f32_to_e4m3((rng.standard_normal((groups, rows, inner)) * 8).astype(np.float32))
    sx = rng.integers(122, 129, (groups, rows, inner // 32), dtype=np.uint8)
    weights, scales = [], []
    for g in range(weight_groups):
        _, _, w, sw = operands(820 + g, 1, outputs, inner, packed, 32)
        weights.append(torch.from_numpy(w).to(device))
        scales.append(torch.from_numpy(sw).to(device))
    metadata = torch.tensor([[w.data_ptr(), s.data_ptr()] for w, s in zip(weights, scales)],
                            dtype=torch.int64, device=device)
    active_host = [int(v) for v in rng.integers(-1, weight_groups + 1, groups)]
    counts_host = [int(v) for v in rng.integers(0, rows + 2, groups)]
    out = _kernels.grouped_quantized_matmul(
        torch.from_numpy(x).to(device).view(torch.float8_e4m3fn), torch.from_numpy(sx).to(device), metadata,
        torch.tensor(active_host, dtype=torch.int32, device=device),
        torch.tensor(counts_host, dtype=torch.int32, device=device), outputs=outputs, packed=packed)
    torch.cuda.synchronize()
    got = bf16_values(out)
    for g, (index, count) in enumerate(zip(active_host, counts_host)):
        if not 0 <= index < weight_groups:
            assert not got[g].any()
            continue
        count = min(max(count, 0), rows)
        want = oracle.mx_matmul_f64(x[g], sx[g], weights[index].cpu().numpy(), scales[index].cpu().numpy(), 32, packed)
        assert (np.abs(got[g, :count] - want[:count]) <= 0.02 + 0.008 * np.abs(want[:count])).all()
        assert not got[g, count:].any()


def test_invalid_arguments(device):
    native, lib = _native.context(device), _native.library()
    for arguments in ((2, 1, 8, 32, 32), (0, 1, 12, 32, 32), (0, 1, 8, 48, 32), (0, 1, 8, 128, 128),
                      (1, 1, 8, 160, 128), (0, 70000, 8, 32, 32)):
        status = lib.camblas_cuda_quantized_matmul(native.handle, *arguments, None, None, None, None, None)
        assert status == -1 and b"invalid quantized matrix dimensions" in lib.camblas_cuda_error(native.handle)
    assert lib.camblas_cuda_quantized_matmul(native.handle, 0, 0, 8, 32, 32, None, None, None, None, None) == 0
    status = lib.camblas_cuda_quantized_matmul(native.handle, 0, 1, 8, 32, 32, None, None, None, None, None)
    assert status == -1 and b"invalid quantized matrix buffers" in lib.camblas_cuda_error(native.handle)
    status = lib.camblas_cuda_grouped_quantized_matmul(native.handle, 0, 1, 0, 1, 8, 32, 32, None, None, None, None, None, None)
    assert status == -1 and b"invalid grouped matrix dimensions" in lib.camblas_cuda_error(native.handle)


# ---------------------------------------------------------------- expert routing (index work: exact)
@pytest.mark.parametrize("tokens,choices,groups,rows", [(1, 8, 4, 4), (37, 8, 16, 8), (300, 6, 40, 70),
                                                        (5, 1, 3, 2), (0, 4, 3, 2)])
def test_route_groups_is_exact(device, tokens, choices, groups, rows):
    rng = np.random.default_rng(tokens * 7 + groups)
    first = 10
    experts = rng.integers(first - 3, first + groups + 4, (tokens, choices)).astype(np.int64)
    if tokens:
        experts[0, 0] = -5
        experts[-1, -1] = 2**40                      # outside [first, INT_MAX): ignored
    active = rng.permutation(groups + 2)[:groups].astype(np.int32)
    if groups > 2:
        active[-1] = active[0]                       # duplicate: the first group wins
    slots, reverse, counts = _kernels.route_groups(
        torch.from_numpy(experts).to(device).reshape(tokens, choices), torch.from_numpy(active).to(device),
        first_expert=first, rows=rows)
    torch.cuda.synchronize()
    want_counts, want_slots, want_reverse = oracle.route_groups(experts, active, first, rows)
    assert np.array_equal(counts.cpu().numpy(), want_counts)
    assert np.array_equal(slots.cpu().numpy(), want_slots)
    assert np.array_equal(reverse.cpu().numpy()[:, :choices], want_reverse.reshape(tokens, choices))
    # invariants of the contract, independent of the oracle
    got_slots, got_reverse = slots.cpu().numpy(), reverse.cpu().numpy().reshape(-1)[: tokens * choices]
    for group in range(groups):
        taken = got_slots[group][got_slots[group] >= 0]
        assert len(taken) == min(int(counts[group]), rows) and len(set(taken)) == len(taken)
        for row, slot in enumerate(taken):
            assert got_reverse[slot] == group * rows + row
            assert experts.reshape(-1)[slot] - first == active[group]


@pytest.mark.parametrize("tokens,choices,width", [(1, 8, 7168), (9, 4, 257), (3, 64, 40), (5, 12, 4104), (2, 3, 20480)])
def test_reduce_groups_is_exact(device, tokens, choices, width):
    rng = np.random.default_rng(tokens + choices)
    grouped_rows = 50
    grouped = oracle.fill_normal_bf16(900 + width, (grouped_rows, width))
    experts = rng.integers(-2, 12, (tokens, choices)).astype(np.int64)   # duplicates, negatives
    reverse = rng.integers(-3, grouped_rows + 3, (tokens, choices)).astype(np.int32)
    out = _kernels.reduce_groups(torch.from_numpy(grouped.view(np.int16)).view(torch.bfloat16).to(device),
                                 torch.from_numpy(experts).to(device), torch.from_numpy(reverse).to(device))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.reduce_groups(grouped, experts, reverse))
