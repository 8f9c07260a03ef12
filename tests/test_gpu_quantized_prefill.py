"""E8M0 block-scaled products at prefill row counts (more than 32 rows: the tiled kernel that uses
the matrix cores' hardware scales), through the C ABI, against the independent FP64 byte decoder
of the oracle. Strategy of the reference's tests/test_quantized.py:110-158 and :243-320 (every
operand mutated separately, scale extremes and NaN, grouped weights with clipped counts), plus
products chosen so that every partial sum is exact in FP32: there the kernel must equal the
oracle bit for bit, which pins the operand layout and which scale byte goes with which block."""

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import bf16_values

pytestmark = pytest.mark.gpu

KERNELS = {"auto": -1, "stream": 0, "tile256x256": 20, "tile256x128": 21, "tile192x256": 22, "tile128x128": 23,
           "wave4-192x256": 24}


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


def shifted(device, array, shift):
    """Device copy of a byte array that starts `shift` bytes after an aligned address."""
    buffer = torch.zeros(array.size + 16, dtype=torch.uint8, device=device)
    view = buffer[shift:shift + array.size].view(array.shape)
    view.copy_(torch.from_numpy(array).to(device))
    return view


def run(device, x, sx, weight, sw, packed, block, kernel="auto", shifts=(0, 0), shares=0):
    xt = torch.from_numpy(x).to(device).view(torch.float8_e4m3fn)
    wt = torch.from_numpy(weight).to(device)
    if not packed:
        wt = wt.view(torch.float8_e4m3fn)
    native = _native.context(device)
    native.call("hip_set_plan_override", KERNELS[kernel], shares)
    try:
        out = _kernels.quantized_matmul(xt, shifted(device, sx, shifts[0]), wt, shifted(device, sw, shifts[1]),
                                        activation_block=block)
        torch.cuda.synchronize()
    finally:
        native.call("hip_set_plan_override", -1, 0)
    return bf16_values(out)


def close(got, x, sx, weight, sw, packed, block):
    # FP32 accumulation inside the matrix instruction may lose 2^-13 of the sum of the products'
    # magnitudes (measured about 2^-15.6); BF16 rounding of the result is the 0.008
    xd = oracle.mx_dequantise(x, sx, block)
    wd = oracle.mx_dequantise(weight, sw, 32, packed, True)
    want = xd @ wd.T
    magnitude = np.abs(xd) @ np.abs(wd).T
    assert got.shape == want.shape
    assert (np.abs(got - want) <= 0.008 * np.abs(want) + magnitude * 2.0 ** -13).all()
    assert np.linalg.norm(got - want) <= 4e-3 * np.linalg.norm(want)


# (the 192-row tile exists for E4M3 weights only)
FORMATS = [(kernel, packed, block) for kernel in ("auto", "tile256x256", "tile256x128", "tile192x256", "tile128x128")
           for packed, block in ((False, 32), (True, 32), (True, 128)) if not (packed and kernel == "tile192x256")]


@pytest.mark.parametrize("kernel,packed,block", FORMATS)
@pytest.mark.parametrize("rows,outputs,inner", [(33, 264, 256), (65, 264, 256), (128, 520, 384),
                                               (300, 776, 1024), (513, 40, 128)])
def test_random_operands_and_individual_mutations(device, kernel, packed, block, rows, outputs, inner):
    x, sx, weight, sw = operands(900 + rows, rows, outputs, inner, packed, block)
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
        close(run(device, x, sx, weight, sw, packed, block, kernel), x, sx, weight, sw, packed, block)


@pytest.mark.parametrize("kernel,packed,block", [f for f in FORMATS if f[0] != "auto"])
@pytest.mark.parametrize("shifts", [(0, 0), (1, 3), (2, 1), (3, 2)])
def test_exact_products_with_every_scale_alignment(device, kernel, packed, block, shifts):
    # Inputs in {0, +-0.5, +-1, +-2}, weights in {0, +-0.5 .. +-2} (E2M1: any nibble up to 2), scales
    # 2^-2 .. 2^2 drawn per block: every product is a multiple of 2^-6 below 2^6 and a sum of 640 of
    # them is exact in FP32, so the result must be the BF16 rounding of the exact product, and a
    # scale byte applied to the wrong block or row would change it. Scale arrays start at every
    # offset inside a 4-byte word (they are byte arrays; nothing aligns them).
    rows, outputs, inner = 150, 328, 640
    rng = np.random.default_rng(31 + shifts[0])
    levels = np.array([0x00, 0x30, 0x38, 0x40, 0xB0, 0xB8, 0xC0], np.uint8)  # E4M3 0, .5, 1, 2, -.5, -1, -2
    x = levels[rng.integers(0, len(levels), (rows, inner))]
    if packed:
        nibbles = np.array([0, 1, 2, 3, 4, 9, 10, 11, 12], np.uint8)  # 0, .5, 1, 1.5, 2 and negatives
        pairs = nibbles[rng.integers(0, len(nibbles), (outputs, inner // 2, 2))]
        weight = (pairs[..., 0] | (pairs[..., 1] << 4)).astype(np.uint8)
    else:
        weight = levels[rng.integers(0, len(levels), (outputs, inner))]
    sx = rng.integers(125, 130, (rows, inner // block), dtype=np.uint8)
    sw = rng.integers(125, 130, (outputs if packed else (outputs + 31) // 32, inner // 32), dtype=np.uint8)
    got = run(device, x, sx, weight, sw, packed, block, kernel, shifts)
    want = oracle.mx_matmul_f64(x, sx, weight, sw, block, packed)
    assert np.abs(want).max() < 2.0 ** 24 and (want * 64 == np.round(want * 64)).all()
    want = oracle.bf16_to_f32(oracle.f32_to_bf16(want.astype(np.float32)))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,outputs,inner", [(70, 296, 2048), (513, 456, 3072), (300, 840, 4096)])
def test_four_wavefront_tile_random_operands(device, packed, rows, outputs, inner):
    # 192 x 256 tiles on four wavefronts with the K loop in generated assembly (a scale per 32 inputs; E4M3
    # weights with a scale per 32 x 32 block, or packed E2M1 weights with a scale per row and 32 inputs):
    # partial tiles in both directions, a partial last scale block, two to four slabs of eight K groups,
    # operands and scales mutated one at a time
    x, sx, weight, sw = operands(950 + rows, rows, outputs, inner, packed, 32)
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
        close(run(device, x, sx, weight, sw, packed, 32, "wave4-192x256"), x, sx, weight, sw, packed, 32)


@pytest.mark.parametrize("packed", [False, True])
def test_four_wavefront_tile_exact_products(device, packed):
    # exact arithmetic as in test_exact_products_with_every_scale_alignment over 24 K groups (three slabs):
    # a scale byte of the wrong block, row, group or slab buffer changes the bits
    rows, outputs, inner = 300, 840, 24 * 128
    rng = np.random.default_rng(77)
    levels = np.array([0x00, 0x30, 0x38, 0x40, 0xB0, 0xB8, 0xC0], np.uint8)
    x = levels[rng.integers(0, len(levels), (rows, inner))]
    if packed:
        nibbles = np.array([0, 1, 2, 3, 4, 9, 10, 11, 12], np.uint8)  # 0, .5, 1, 1.5, 2 and negatives
        pairs = nibbles[rng.integers(0, len(nibbles), (outputs, inner // 2, 2))]
        weight = (pairs[..., 0] | (pairs[..., 1] << 4)).astype(np.uint8)
    else:
        weight = levels[rng.integers(0, len(levels), (outputs, inner))]
    sx = rng.integers(125, 130, (rows, inner // 32), dtype=np.uint8)
    sw = rng.integers(125, 130, (outputs if packed else (outputs + 31) // 32, inner // 32), dtype=np.uint8)
    got = run(device, x, sx, weight, sw, packed, 32, "wave4-192x256")
    want = oracle.mx_matmul_f64(x, sx, weight, sw, 32, packed)
    assert np.abs(want).max() < 2.0 ** 24 and (want * 64 == np.round(want * 64)).all()
    assert np.array_equal(got, oracle.bf16_to_f32(oracle.f32_to_bf16(want.astype(np.float32))))


@pytest.mark.parametrize("shift", [1, 2, 3])
def test_four_wavefront_tile_block_scales_at_any_address(device, shift):
    # the block scales of E4M3 weights need no alignment: the slab is copied from the aligned address below
    # them with a ninth word per block row; exact products over three slabs show a byte taken from the wrong place
    rows, outputs, inner = 100, 424, 24 * 128
    rng = np.random.default_rng(78 + shift)
    levels = np.array([0x00, 0x30, 0x38, 0x40, 0xB0, 0xB8, 0xC0], np.uint8)
    x = levels[rng.integers(0, len(levels), (rows, inner))]
    weight = levels[rng.integers(0, len(levels), (outputs, inner))]
    sx = rng.integers(125, 130, (rows, inner // 32), dtype=np.uint8)
    sw = rng.integers(125, 130, ((outputs + 31) // 32, inner // 32), dtype=np.uint8)
    got = run(device, x, sx, weight, sw, False, 32, "wave4-192x256", shifts=(0, shift))
    want = oracle.mx_matmul_f64(x, sx, weight, sw, 32, False)
    assert np.array_equal(got, oracle.bf16_to_f32(oracle.f32_to_bf16(want.astype(np.float32))))


def test_four_wavefront_tile_refuses_what_it_cannot_run(device):
    # a scale per 128 inputs, an inner dimension that is not whole slabs of eight groups
    for packed, block, inner in ((True, 128, 2048), (False, 32, 1152), (True, 32, 1152)):
        x, sx, weight, sw = operands(5, 64, 256, inner, packed, block)
        with pytest.raises(RuntimeError):
            run(device, x, sx, weight, sw, packed, block, "wave4-192x256")


@pytest.mark.parametrize("kernel,packed,block", [f for f in FORMATS if f[0] != "auto"])
@pytest.mark.parametrize("shares,shifts", [(2, (0, 0)), (4, (1, 3)), (9, (2, 1))])
def test_exact_products_with_k_divided_over_workgroups(device, kernel, packed, block, shares, shifts):
    # Nine steps of 128 inputs over 2 (5 + 4), 3 (asked for 4: 3 + 3 + 3) and 9 workgroups per tile, whose
    # FP32 planes a second kernel adds in share order. Operands as in the test above, so that every
    # plane and their sum are exact: the result must again be the BF16 rounding of the exact product,
    # which pins the step at which each share starts in the operands and in both scale arrays.
    rows, outputs, inner = 150, 328, 1152
    rng = np.random.default_rng(57 + shares)
    levels = np.array([0x00, 0x30, 0x38, 0x40, 0xB0, 0xB8, 0xC0], np.uint8)
    x = levels[rng.integers(0, len(levels), (rows, inner))]
    if packed:
        nibbles = np.array([0, 1, 2, 3, 4, 9, 10, 11, 12], np.uint8)
        pairs = nibbles[rng.integers(0, len(nibbles), (outputs, inner // 2, 2))]
        weight = (pairs[..., 0] | (pairs[..., 1] << 4)).astype(np.uint8)
    else:
        weight = levels[rng.integers(0, len(levels), (outputs, inner))]
    sx = rng.integers(125, 130, (rows, inner // block), dtype=np.uint8)
    sw = rng.integers(125, 130, (outputs if packed else (outputs + 31) // 32, inner // 32), dtype=np.uint8)
    got = run(device, x, sx, weight, sw, packed, block, kernel, shifts, shares)
    want = oracle.mx_matmul_f64(x, sx, weight, sw, block, packed)
    assert np.abs(want).max() < 2.0 ** 24 and (want * 64 == np.round(want * 64)).all()
    want = oracle.bf16_to_f32(oracle.f32_to_bf16(want.astype(np.float32)))
    assert np.array_equal(got, want)


def test_planned_product_with_k_divided(device):
    # a narrow projection with a long K at 96 rows: the planner divides K (56 tiles of 128 x 128 on 256
    # compute units otherwise); random operands against the FP64 decoder
    for packed in (False, True):
        x, sx, weight, sw = operands(5, 96, 1024, 4096, packed, 32)
        close(run(device, x, sx, weight, sw, packed, 32), x, sx, weight, sw, packed, 32)


@pytest.mark.parametrize("packed", [False, True])
def test_rows_17_to_32_with_a_long_k_take_the_tiles(device, packed):
    # 24 rows x K = 18432: the scale bytes of 32 tokens (18 KB) exceed the streaming kernel's LDS table,
    # so the product runs on the tiled kernel (with K divided: 3 tiles otherwise); the streaming
    # kernel, forced, must agree with it
    x, sx, weight, sw = operands(11, 24, 264, 18432, packed, 32)
    planned = run(device, x, sx, weight, sw, packed, 32)
    close(planned, x, sx, weight, sw, packed, 32)
    streamed = run(device, x, sx, weight, sw, packed, 32, "stream")
    close(streamed, x, sx, weight, sw, packed, 32)


@pytest.mark.parametrize("packed", [False, True])
def test_tiled_and_streaming_kernels_agree(device, packed):
    x, sx, weight, sw = operands(77, 200, 520, 512, packed, 32)
    tiled = run(device, x, sx, weight, sw, packed, 32, "tile256x256")
    streamed = run(device, x, sx, weight, sw, packed, 32, "stream")
    magnitude = np.abs(oracle.mx_dequantise(x, sx, 32)) @ np.abs(oracle.mx_dequantise(weight, sw, 32, packed, True)).T
    assert (np.abs(tiled - streamed) <= 0.008 * np.abs(streamed) + magnitude * 2.0 ** -13).all()


@pytest.mark.parametrize("kernel", ["tile256x256", "tile256x128", "tile128x128"])
@pytest.mark.parametrize("packed", [False, True])
def test_scale_extremes_and_nan(device, kernel, packed):
    # ones times ones with unit weight scales: exact for input scales 2^-127, 1, 2^127 and NaN for
    # the scale byte 255; a NaN input or weight byte poisons exactly its row / column
    # (ref: tests/test_quantized.py:243-280)
    rows, outputs, inner = 130, 296, 128
    x = np.full((rows, inner), 0x38, np.uint8)
    weight = np.full((outputs, inner // 2), 0x22, np.uint8) if packed else np.full((outputs, inner), 0x38, np.uint8)
    sw = np.full((outputs if packed else (outputs + 31) // 32, inner // 32), 127, np.uint8)
    for exponent in (0, 127, 254, 255):
        sx = np.full((rows, inner // 32), exponent, np.uint8)
        got = run(device, x, sx, weight, sw, packed, 32, kernel)
        with np.errstate(over="ignore"):
            want = oracle.bf16_to_f32(oracle.f32_to_bf16(
                oracle.mx_matmul_f64(x, sx, weight, sw, 32, packed).astype(np.float32)))
        assert np.array_equal(got, want, equal_nan=True), exponent
    sx = np.full((rows, inner // 32), 127, np.uint8)
    one_bad_scale = sx.copy()
    one_bad_scale[77, 2] = 255
    got = run(device, x, one_bad_scale, weight, sw, packed, 32, kernel)
    assert np.isnan(got[77]).all() and (np.delete(got, 77, axis=0) == inner).all()
    poisoned = x.copy()
    poisoned[rows - 1, 5] = 0x7F
    got = run(device, poisoned, sx, weight, sw, packed, 32, kernel)
    assert np.isnan(got[rows - 1]).all() and (got[: rows - 1] == inner).all()
    if not packed:
        bad = weight.copy()
        bad[263, 100] = 0xFF
        got = run(device, x, sx, bad, sw, packed, 32, kernel)
        assert np.isnan(got[:, 263]).all() and (np.delete(got, 263, axis=1) == inner).all()


@pytest.mark.parametrize("kernel", ["auto", "tile256x256", "tile256x128", "tile128x128"])
@pytest.mark.parametrize("packed,block", [(False, 32), (True, 32), (True, 128)])
def test_grouped_products(device, kernel, packed, block):
    check_grouped_products(device, kernel, packed, block, inner=256, input_shift=1)


def test_grouped_products_on_the_four_wavefront_tile(device):
    # E4M3 weights only (the per-row scales of packed weights would have to be 16-byte aligned, which the
    # host cannot see in a device table); each group's block scales at another alignment
    check_grouped_products(device, "wave4-192x256", False, 32, inner=2048, input_shift=0)
    with pytest.raises(RuntimeError):
        check_grouped_products(device, "wave4-192x256", True, 32, inner=2048, input_shift=0)
    with pytest.raises(RuntimeError):  # input scales that are not 16-byte aligned
        check_grouped_products(device, "wave4-192x256", False, 32, inner=2048, input_shift=1)


def check_grouped_products(device, kernel, packed, block, inner, input_shift):
    # ref: include/camblas_cuda.h:156-167 — weights chosen per group through a device table, an
    # invalid index gives zeros, counts clip the rows, padding rows are zero even where the
    # padding's scale bytes say NaN
    groups, weight_groups, rows, outputs = 6, 3, 300, 264
    rng = np.random.default_rng(19)
    x = oracle.f32_to_e4m3((rng.standard_normal((groups, rows, inner)) * 8).astype(np.float32))
    sx = rng.integers(122, 129, (groups, rows, inner // block), dtype=np.uint8)
    counts_host = [300, 5, 300, 999, 130, 257]
    for g, count in enumerate(counts_host):
        sx[g, min(count, rows):] = 255
    weights, scales = [], []
    for g in range(weight_groups):
        _, _, w, sw = operands(800 + g, 1, outputs, inner, packed, 32)
        weights.append(torch.from_numpy(w).to(device))
        scales.append(shifted(device, sw, g))  # each group's scales at another alignment
    metadata = torch.tensor([[w.data_ptr(), s.data_ptr()] for w, s in zip(weights, scales)],
                            dtype=torch.int64, device=device)
    active = torch.tensor([2, 0, 7, 1, -1, 1], dtype=torch.int32, device=device)
    counts = torch.tensor(counts_host, dtype=torch.int32, device=device)
    native = _native.context(device)
    native.call("hip_set_plan_override", KERNELS[kernel], 0)
    try:
        out = _kernels.grouped_quantized_matmul(
            torch.from_numpy(x).to(device).view(torch.float8_e4m3fn), shifted(device, sx, input_shift),
            metadata, active, counts, outputs=outputs, packed=packed, activation_block=block)
        torch.cuda.synchronize()
    finally:
        native.call("hip_set_plan_override", -1, 0)
    got = bf16_values(out)
    for g, (index, count) in enumerate(zip(active.tolist(), counts_host)):
        if not 0 <= index < weight_groups:
            assert not got[g].any()
            continue
        count = min(max(count, 0), rows)
        close(got[g, :count], x[g, :count], sx[g, :count], weights[index].cpu().numpy(),
              scales[index].cpu().numpy(), packed, block)
        assert not got[g, count:].any()


@pytest.mark.parametrize("kernel", ["tile256x128", "tile128x128"])
@pytest.mark.parametrize("packed", [False, True])
def test_grouped_products_many_groups_skewed_counts(device, kernel, packed):
    check_many_groups_skewed_counts(device, kernel, packed, inner=128, compared=40)


def test_many_groups_skewed_counts_on_the_four_wavefront_tile(device):
    check_many_groups_skewed_counts(device, "wave4-192x256", False, inner=2048, compared=6)


def check_many_groups_skewed_counts(device, kernel, packed, inner, compared):
    """150 groups (three 64-lane chunks of the tile numbering) with a capacity of several token tiles
    and counts from none to all of it, negative and oversized included: every tile with work is
    computed for the right group, every other tile of the capacity is zero."""
    groups, weight_groups, rows, outputs = 150, 5, 300, 136
    rng = np.random.default_rng(23)
    x = oracle.f32_to_e4m3((rng.standard_normal((groups, rows, inner)) * 8).astype(np.float32))
    sx = rng.integers(124, 129, (groups, rows, inner // 32), dtype=np.uint8)
    counts_host = rng.choice([-3, 0, 1, 40, 127, 128, 129, 255, 256, 257, 300, 4000], size=groups).tolist()
    active_host = rng.integers(-1, weight_groups + 1, size=groups).tolist()
    weights, scales = [], []
    for g in range(weight_groups):
        _, _, w, sw = operands(900 + g, 1, outputs, inner, packed, 32)
        weights.append(torch.from_numpy(w).to(device))
        scales.append(torch.from_numpy(sw).to(device))
    metadata = torch.tensor([[w.data_ptr(), s.data_ptr()] for w, s in zip(weights, scales)],
                            dtype=torch.int64, device=device)
    active = torch.tensor(active_host, dtype=torch.int32, device=device)
    counts = torch.tensor(counts_host, dtype=torch.int32, device=device)
    native = _native.context(device)
    native.call("hip_set_plan_override", KERNELS[kernel], 0)
    try:
        out = _kernels.grouped_quantized_matmul(
            torch.from_numpy(x).to(device).view(torch.float8_e4m3fn), torch.from_numpy(sx).to(device),
            metadata, active, counts, outputs=outputs, packed=packed, activation_block=32)
        torch.cuda.synchronize()
    finally:
        native.call("hip_set_plan_override", -1, 0)
    got = bf16_values(out)
    checked = 0
    for g, (index, count) in enumerate(zip(active_host, counts_host)):
        count = min(max(count, 0), rows) if 0 <= index < weight_groups else 0
        assert not got[g, count:].any(), g
        if count and checked < compared:  # the CPU product of every group would take minutes
            close(got[g, :count], x[g, :count], sx[g, :count], weights[index].cpu().numpy(),
                  scales[index].cpu().numpy(), packed, 32)
            checked += 1
        elif count:
            assert got[g, :count].any(), g
    assert checked == compared


def test_forced_tile_kernel_refuses_what_it_cannot_run(device):
    # K that is not a multiple of 128 belongs to the streaming kernel; forcing the tiled one fails
    x, sx, weight, sw = operands(5, 70, 40, 160, False, 32)
    with pytest.raises(RuntimeError, match="quantized matrix multiplication"):
        run(device, x, sx, weight, sw, False, 32, "tile256x256")
    close(run(device, x, sx, weight, sw, False, 32, "auto"), x, sx, weight, sw, False, 32)
