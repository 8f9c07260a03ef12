"""FP8 E4M3fn block-scaled linear (1x128 activation groups, 128x128 weight blocks) against the
CPU oracle.

Bars: scale/block indexing bit-exact (exact-arithmetic cases with a distinct power-of-two scale per
block must reproduce the oracle's BF16 bits), outputs within relative Frobenius 1e-2 of the FP64
accumulation of the dequantised operands; the ordered-FMA restatement (camblas/_hopper.py:168-182)
is matched to within one BF16 unit in the last place on random data. Known-answer bytes follow
tests/test_quantized.py:160-216 (0x38 = 1.0, 0x40 = 2.0, 0x30 = 0.5, 0x7f = NaN).
"""

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import (bf16_ulp_distance, bf16_values, from_device_bf16, from_device_fp8, rel_frobenius,
                     to_device_bf16, to_device_fp8)

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-2


def run(device, a, a_scale, w, w_scale, override=None):
    native = _native.context(device)
    if override is not None:
        native.call("hip_set_plan_override", override[0], override[1])
    try:
        out = _kernels.fp8_block_matmul(
            to_device_fp8(a, device), torch.from_numpy(a_scale).to(device),
            to_device_fp8(w, device), torch.from_numpy(w_scale).to(device))
        torch.cuda.synchronize()
    finally:
        native.call("hip_set_plan_override", -1, 0)
    return out


@pytest.mark.parametrize("variant", range(4))
@pytest.mark.parametrize("split", [1, 2])
@pytest.mark.parametrize("rows", [1, 16, 70])
def test_random_blocks_every_variant(device, variant, split, rows):
    outputs, inner = 300, 512  # partial last 128-row weight block, partial tiles
    a, a_scale = oracle.fill_fp8_blocks(100 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(200, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale, override=(variant, split))
    want64 = oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), want64) <= TOLERANCE
    if split == 1:
        ordered = oracle.fp8_block_matmul(a, a_scale, w, w_scale)
        # same ordered chain; only the rounding of each group's dot product inside the matrix
        # core may differ, which can move a BF16 result by one unit (more only under cancellation)
        distance = bf16_ulp_distance(from_device_bf16(out), ordered)
        assert (distance == 0).mean() > 0.95
        wanted = oracle.bf16_to_f32(ordered)
        bound = 2.0**-7 * np.abs(wanted) + 1e-4 * np.abs(want64).max()
        assert (np.abs(bf16_values(out) - wanted) <= bound).all()


# 100 + 10*row_tiles + token_tiles: the weight-streaming decode kernel
FP8_STREAM_CODES = [100 + 10 * rows + tokens for rows in range(1, 9) for tokens in (1, 2, 3, 4)
                    if rows * tokens <= 20 and rows + tokens <= 10]


@pytest.mark.parametrize("code", FP8_STREAM_CODES)
@pytest.mark.parametrize("rows,outputs,inner", [(1, 300, 512), (20, 258, 896), (70, 131, 1280)])
def test_streaming_decode_variants(device, code, rows, outputs, inner):
    # ragged weight rows (partial 16-row tile, partial 128-row scale block, output counts that are
    # not multiples of four), token counts that underfill and span the token tiles, group counts
    # that are not multiples of the four wavefronts; the sum order differs from the oracle's single
    # chain (four interleaved chains), so results agree to the tolerance form, not bit for bit
    a, a_scale = oracle.fill_fp8_blocks(300 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(301, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale, override=(code, 1))
    want64 = oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), want64) <= TOLERANCE
    wanted = oracle.bf16_to_f32(oracle.f32_to_bf16(want64.astype(np.float32)))
    bound = 2.0**-7 * np.abs(wanted) + 1e-4 * np.abs(want64).max()
    assert (np.abs(bf16_values(out) - wanted) <= bound).all()


@pytest.mark.parametrize("rows,inner", [(16, 192 * 128), (24, 193 * 128), (5, 67 * 128)])
def test_streaming_decode_scale_table_limits(device, rows, inner):
    # the streaming kernel keeps a row of K / 128 scales per token in LDS: 192 groups is the most it
    # takes (three whole 64-float loads per row), 193 goes to another kernel, 67 leaves a load with
    # three live lanes; weight rows that straddle two 128-row scale blocks
    outputs = 200
    a, a_scale = oracle.fill_fp8_blocks(800 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(801, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale)
    want64 = oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), want64) <= TOLERANCE
    wanted = oracle.bf16_to_f32(oracle.f32_to_bf16(want64.astype(np.float32)))
    bound = 2.0**-7 * np.abs(wanted) + 1e-4 * np.abs(want64).max()
    assert (np.abs(bf16_values(out) - wanted) <= bound).all()


@pytest.mark.parametrize("code", list(range(20, 36)))
@pytest.mark.parametrize("rows,outputs,inner", [(70, 300, 512), (256, 512, 128), (513, 260, 896)])
def test_direct_lds_load_variants(device, code, rows, outputs, inner):
    # partial tiles in both directions, a partial last weight-scale block, odd and even numbers of
    # K groups; the ordered chain is the same as the oracle's, so results agree to one BF16 unit
    a, a_scale = oracle.fill_fp8_blocks(700 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(701, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale, override=(code, 1))
    want64 = oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), want64) <= TOLERANCE
    ordered = oracle.bf16_to_f32(oracle.fp8_block_matmul(a, a_scale, w, w_scale))
    bound = 2.0**-7 * np.abs(ordered) + 1e-4 * np.abs(want64).max()
    assert (np.abs(bf16_values(out) - ordered) <= bound).all()


@pytest.mark.parametrize("code,split", [(20, 2), (24, 3), (27, 2), (29, 7), (26, 64), (30, 2), (31, 3), (35, 7)])
@pytest.mark.parametrize("rows,outputs,inner", [(70, 300, 896), (129, 516, 1792)])
def test_direct_lds_loads_with_divided_k_groups(device, code, split, rows, outputs, inner):
    # the K groups of a tile shared by several workgroups (uneven shares, more shares asked for than
    # groups exist) and summed in share order: the FMA chain is cut into `split` chains, so the
    # FP64 bar applies and the ordered oracle holds to one BF16 unit plus the FP32 re-association
    a, a_scale = oracle.fill_fp8_blocks(720 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(721, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale, override=(code, split))
    want64 = oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), want64) <= TOLERANCE
    wanted = oracle.bf16_to_f32(oracle.f32_to_bf16(want64.astype(np.float32)))
    bound = 2.0**-7 * np.abs(wanted) + 1e-4 * np.abs(want64).max()
    assert (np.abs(bf16_values(out) - wanted) <= bound).all()


@pytest.mark.parametrize("rows,outputs,inner", [(70, 300, 2048), (513, 452, 3072), (256, 1156, 4096)])
def test_four_wavefront_tile(device, rows, outputs, inner):
    # code 36: 192 x 256 tiles on four wavefronts with the K loop in generated assembly; partial tiles
    # in both directions, a partial last weight-scale block, wavefronts whose 96 rows start at every
    # offset inside a 128-row scale block (0, 32, 64, 96), two to four slabs of eight K groups.
    # The chain is the ordered oracle's, so results agree to one BF16 unit.
    a, a_scale = oracle.fill_fp8_blocks(740 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(741, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale, override=(36, 1))
    want64 = oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), want64) <= TOLERANCE
    ordered = oracle.bf16_to_f32(oracle.fp8_block_matmul(a, a_scale, w, w_scale))
    bound = 2.0**-7 * np.abs(ordered) + 1e-4 * np.abs(want64).max()
    assert (np.abs(bf16_values(out) - ordered) <= bound).all()


def test_four_wavefront_tile_scale_indexing_is_bit_exact(device):
    # exact arithmetic (small-integer products, power-of-two scales, distinct per (token, group) and
    # (block, group)) over 24 K groups = three slabs: a wrong scale index, a wrong slab buffer or a
    # tile accumulated with the other block's scale changes bits
    rows, outputs, inner = 300, 836, 24 * 128
    groups, blocks = inner // 128, (outputs + 127) // 128
    rng = np.random.default_rng(8)
    small = np.array([0x00, 0x38, 0x40, 0x30, 0xB8, 0xC0], dtype=np.uint8)  # 0, 1, 2, .5, -1, -2
    a = small[rng.integers(0, len(small), size=(rows, inner))]
    w = small[rng.integers(0, len(small), size=(outputs, inner))]
    a_scale = np.exp2(rng.integers(-5, 5, size=(rows, groups))).astype(np.float32)
    w_scale = np.exp2(-((np.arange(blocks * groups).reshape(blocks, groups) * 5) % 7)).astype(np.float32)
    out = run(device, a, a_scale, w, w_scale, override=(36, 1))
    want = oracle.fp8_block_matmul(a, a_scale, w, w_scale)
    assert np.array_equal(from_device_bf16(out), want)


def test_four_wavefront_tile_matches_the_eight_wavefront_tile_bit_for_bit(device):
    # the same K positions per lane quarter and the same chain: identical bits at the benchmark's
    # inner dimension (56 groups = seven slabs), random data
    rows, outputs, inner = 520, 772, 7168
    a, a_scale = oracle.fill_fp8_blocks(750, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(751, outputs, inner, 128)
    new = from_device_bf16(run(device, a, a_scale, w, w_scale, override=(36, 1)))
    old = from_device_bf16(run(device, a, a_scale, w, w_scale, override=(34, 1)))
    assert np.array_equal(new, old)


@pytest.mark.parametrize("rows", [1, 16, 96, 256])
def test_planned_shapes(device, rows):
    outputs, inner = 1536, 1024
    a, a_scale = oracle.fill_fp8_blocks(300 + rows, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(301, outputs, inner, 128)
    out = run(device, a, a_scale, w, w_scale)
    assert rel_frobenius(bf16_values(out), oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale)) <= TOLERANCE


@pytest.mark.parametrize("override", [None, (0, 1), (1, 1), (2, 1), (3, 1), (20, 1), (21, 1), (22, 1), (23, 1), (24, 1), (25, 1), (26, 1),
                                      (24, 3), (28, 4), (111, 1), (152, 1), (134, 1)])
def test_scale_indexing_is_bit_exact(device, override):
    # every product is a small integer and every scale a distinct power of two, so the FMA chain
    # is exact: any wrong (row, group) or (block, group) scale index changes the bits
    rows, outputs, inner = 40, 384, 512
    groups, blocks = inner // 128, outputs // 128
    rng = np.random.default_rng(5)
    small = np.array([0x00, 0x38, 0x40, 0x30, 0xB8, 0xC0], dtype=np.uint8)  # 0, 1, 2, .5, -1, -2
    a = small[rng.integers(0, len(small), size=(rows, inner))]
    w = small[rng.integers(0, len(small), size=(outputs, inner))]
    a_scale = np.exp2(rng.integers(-6, 6, size=(rows, groups))).astype(np.float32)
    w_scale = np.exp2(-(np.arange(blocks * groups).reshape(blocks, groups) % 7)).astype(np.float32)
    out = run(device, a, a_scale, w, w_scale, override=override)
    want = oracle.fp8_block_matmul(a, a_scale, w, w_scale)
    assert np.array_equal(from_device_bf16(out), want)


@pytest.mark.parametrize("override", [(code, 1) for code in range(20, 36)] + [(24, 3), (27, 2), (28, 5), (20, 4), (30, 4), (33, 2)])
def test_scale_indexing_over_many_groups_is_bit_exact(device, override):
    # the same exact arithmetic over 29 K groups (an odd number: token rows of scales start at
    # every alignment; several rounds of the kernels' eight-group scale slabs, the last one partial),
    # with partial tiles of tokens and outputs and a partial last weight-scale block; every
    # (token, group) and (block, group) scale is a power of two chosen so that a wrong index changes bits
    rows, outputs, inner = 300, 452, 29 * 128
    groups, blocks = inner // 128, (outputs + 127) // 128
    rng = np.random.default_rng(6)
    small = np.array([0x00, 0x38, 0x40, 0x30, 0xB8, 0xC0], dtype=np.uint8)  # 0, 1, 2, .5, -1, -2
    a = small[rng.integers(0, len(small), size=(rows, inner))]
    w = small[rng.integers(0, len(small), size=(outputs, inner))]
    a_scale = np.exp2(rng.integers(-5, 5, size=(rows, groups))).astype(np.float32)
    w_scale = np.exp2(-((np.arange(blocks * groups).reshape(blocks, groups) * 5) % 7)).astype(np.float32)
    out = run(device, a, a_scale, w, w_scale, override=override)
    want = oracle.fp8_block_matmul(a, a_scale, w, w_scale)
    assert np.array_equal(from_device_bf16(out), want)


def test_known_answer_bytes_and_nan(device):
    rows, outputs, inner = 2, 256, 256
    a = np.full((rows, inner), 0x38, np.uint8)       # 1.0
    w = np.full((outputs, inner), 0x40, np.uint8)    # 2.0
    w[128:] = 0x30                                   # 0.5 in the second weight block
    a_scale = np.array([[1.0, 0.5], [2.0, 2.0]], np.float32)
    w_scale = np.array([[1.0, 1.0], [4.0, 8.0]], np.float32)
    out = bf16_values(run(device, a, a_scale, w, w_scale))
    # row 0: block 0 -> 128*2*(1*1) + 128*2*(0.5*1) = 384; block 1 -> 64*(1*4) + 64*(0.5*8) = 512
    assert (out[0, :128] == 384).all() and (out[0, 128:] == 512).all()
    # row 1: block 0 -> 2 * 128*2*(2*1) = 1024; block 1 -> 64*(2*4) + 64*(2*8) = 1536
    assert (out[1, :128] == 1024).all() and (out[1, 128:] == 1536).all()
    a[1, 5] = 0x7F  # NaN byte poisons its row only
    out = bf16_values(run(device, a, a_scale, w, w_scale))
    assert np.isnan(out[1]).all() and np.isfinite(out[0]).all()
    # zero activations give +0
    out = from_device_bf16(run(device, np.zeros_like(a), a_scale, w, w_scale))
    assert not out.any()


def test_weight_scale_doubling_doubles_output(device):
    rows, outputs, inner = 16, 256, 384
    a, a_scale = oracle.fill_fp8_blocks(400, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(401, outputs, inner, 128)
    base = bf16_values(run(device, a, a_scale, w, w_scale))
    doubled = bf16_values(run(device, a, a_scale, w, w_scale * np.float32(2)))
    assert np.array_equal(doubled, base * 2)


@pytest.mark.parametrize("rows,inner", [(1, 7168), (5, 256), (33, 1024)])
def test_activation_quantiser_is_bit_exact(device, rows, inner):
    x = oracle.fill_normal_bf16(500 + rows, (rows, inner))
    x[0, :128] = 0  # an all-zero group keeps amax at the 1e-10 floor
    q, scale = _kernels.fp8_quantise_1x128(to_device_bf16(x, device))
    torch.cuda.synchronize()
    want_q, want_scale = oracle.quantise_1x128(x)
    assert np.array_equal(scale.cpu().numpy(), want_scale)
    assert np.array_equal(from_device_fp8(q), want_q)
    # invariant: the group maximum maps to +-448 exactly (byte 0x7e / 0xfe)
    values = np.abs(oracle.e4m3_to_f32(from_device_fp8(q))).reshape(rows, inner // 128, 128)
    assert (values.max(axis=2)[1:] == 448).all()


def test_block_linear_with_dynamic_quantisation(device):
    rows, outputs, inner = 16, 512, 1024
    x = oracle.fill_normal_bf16(600, (rows, inner))
    w, w_scale = oracle.fill_fp8_blocks(601, outputs, inner, 128)
    out = _kernels.fp8_block_linear(to_device_bf16(x, device), to_device_fp8(w, device),
                                    torch.from_numpy(w_scale).to(device))
    q, scale = oracle.quantise_1x128(x)
    assert rel_frobenius(bf16_values(out), oracle.fp8_block_matmul_f64(q, scale, w, w_scale)) <= TOLERANCE


def test_invalid_arguments(device):
    native = _native.context(device)
    lib = _native.library()
    assert lib.camblas_cuda_fp8_block_matmul(native.handle, 1, 128, 100, None, None, None, None, None) == -1
    assert b"invalid FP8 block matrix dimensions" in lib.camblas_cuda_error(native.handle)
    assert lib.camblas_cuda_fp8_block_matmul(native.handle, 0, 128, 128, None, None, None, None, None) == 0
    assert lib.camblas_cuda_fp8_block_matmul(native.handle, 1, 128, 128, None, None, None, None, None) == -1
    assert b"invalid FP8 block matrix buffers" in lib.camblas_cuda_error(native.handle)


# ---------------------------------------------------------------- block-32 single-token decode
def block32_operands(seed, outputs, inner):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 0x7F, inner, dtype=np.uint8) | (rng.integers(0, 2, inner, dtype=np.uint8) << 7)
    w = rng.integers(0, 0x7F, (outputs, inner), dtype=np.uint8) | (rng.integers(0, 2, (outputs, inner), dtype=np.uint8) << 7)
    x[x == 0xFF] = 0x80
    w[w == 0xFF] = 0x80
    sx = rng.uniform(0.001, 0.08, inner // 32).astype(np.float32)
    sw = rng.uniform(0.002, 0.05, ((outputs + 31) // 32, inner // 32)).astype(np.float32)
    return x, sx, w, sw


def fp8_tensor(array, device):
    return torch.from_numpy(array).to(device).view(torch.float8_e4m3fn)


@pytest.mark.parametrize("outputs,inner", [(48, 96), (16, 32), (1152, 5120), (5120, 576), (18432, 7168),
                                           (80, 8192)])
def test_block32_decode_matches_ordered_oracle(device, outputs, inner):
    # ref strategy: tests/test_quantized.py:160-216 and tests/test_sglang.py:375-398; sizes cover
    # partial 128-byte steps (inner % 128 != 0), a partial last 32-row scale block and a partial
    # last workgroup. Same ordered chain as the oracle: only the rounding of a block's dot product
    # inside the matrix core may differ.
    x, sx, w, sw = block32_operands(400 + outputs, outputs, inner)
    out = _kernels.fp8_decode(fp8_tensor(x, device).view(1, -1), torch.from_numpy(sx).to(device).view(1, -1),
                              fp8_tensor(w, device), torch.from_numpy(sw).to(device))
    torch.cuda.synchronize()
    assert out.shape == (1, outputs)
    want = oracle.fp8_block32_decode(x, sx, w, sw)
    got = from_device_bf16(out)[0]
    assert (bf16_ulp_distance(got, want) == 0).mean() > 0.9
    wanted = oracle.bf16_to_f32(want)
    assert (np.abs(bf16_values(out)[0] - wanted) <= 2.0**-7 * np.abs(wanted) + 1e-4 * np.abs(wanted).max()).all()
    # padded (element stride 4) input scales and column-major weight scales give the same bits
    storage = torch.zeros((inner // 32, 4), device=device)
    storage[:, 0] = torch.from_numpy(sx).to(device)
    strided = _kernels.fp8_decode(fp8_tensor(x, device).view(1, -1), storage[:, 0].view(1, -1),
                                  fp8_tensor(w, device), torch.from_numpy(sw).to(device).T.contiguous().T)
    assert torch.equal(strided.view(torch.int16), out.view(torch.int16))
    # the forms with two and four wavefronts per workgroup (the planned one has one) give the same bits
    native = _native.context(device)
    for code in (302, 304):
        native.call("hip_set_plan_override", code, 0)
        try:
            forced = _kernels.fp8_decode(fp8_tensor(x, device).view(1, -1), torch.from_numpy(sx).to(device).view(1, -1),
                                         fp8_tensor(w, device), torch.from_numpy(sw).to(device))
        finally:
            native.call("hip_set_plan_override", -1, 0)
        assert torch.equal(forced.view(torch.int16), out.view(torch.int16)), code
    # the quantising form (BF16 token in, four wavefronts per workgroup planned) likewise
    token = torch.from_numpy(oracle.bf16_to_f32(oracle.fill_normal_bf16(77, (inner,)))).to(device).to(torch.bfloat16).view(1, -1)
    planned = _kernels.fp8_linear(token, fp8_tensor(w, device), torch.from_numpy(sw).to(device))
    for code in (301, 302):
        native.call("hip_set_plan_override", code, 0)
        try:
            forced = _kernels.fp8_linear(token, fp8_tensor(w, device), torch.from_numpy(sw).to(device))
        finally:
            native.call("hip_set_plan_override", -1, 0)
        assert torch.equal(forced.view(torch.int16), planned.view(torch.int16)), code


def test_block32_known_answers_graph_and_nan(device):
    # ref: tests/test_quantized.py:160-216 — exact expected values, a captured graph that sees later
    # in-place updates of its operands, NaN propagation
    for fused, n, k in ((False, 48, 96), (True, 48, 96), (False, 1152, 5120), (True, 1152, 5120),
                        (True, 5120, 576)):
        x = torch.zeros(1, k, device=device).to(torch.bfloat16 if fused else torch.float8_e4m3fn)
        weight = torch.ones(n, k, device=device).to(torch.float8_e4m3fn)
        sx = torch.ones(1, k // 32, device=device)
        sw = torch.ones((n + 31) // 32, k // 32, device=device)
        sw[-1].mul_(2)

        def product():
            return _kernels.fp8_linear(x, weight, sw) if fused else _kernels.fp8_decode(x, sx, weight, sw)

        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.inference_mode(), torch.cuda.stream(stream):
            before = product()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                output = product()
            if fused:
                x.fill_(0.5)
            else:
                x.view(torch.uint8).fill_(0x38)
            weight.view(torch.uint8).fill_(0x40)
            sx.mul_(0.5)
            sw.mul_(2)
            graph.replay()
        stream.synchronize()
        expected = torch.full((1, n), float(k * 2), dtype=torch.bfloat16)
        # fused: 0.5 quantises exactly (256 * 2^-9), which equals the split case's 1.0 * 0.5
        expected[:, ((n + 31) // 32 - 1) * 32:] *= 2
        assert torch.equal(output.cpu().view(torch.int16), expected.view(torch.int16)), (fused, n, k)
        assert (before == 0).all()
        weight.view(torch.uint8).fill_(0x7F)
        with torch.inference_mode():
            assert product().isnan().all()


@pytest.mark.parametrize("inner,std", [(7168, 0.75), (576, 80.0), (8192, 1e-3)])
def test_block32_fused_quantiser_is_bit_exact(device, inner, std):
    # the fused kernel quantises in LDS and then runs the same product: its output must equal the
    # product of the oracle-quantised token bit for bit, which pins bytes and power-of-two scales
    outputs = 256
    _, _, w, sw = block32_operands(500 + inner, outputs, inner)
    x_bits = oracle.fill_normal_bf16(501 + inner, (inner,), std=std)
    x_bits[:32] = 0
    q, scale = oracle.quantise_block32(x_bits)
    assert (np.log2(scale) % 1 == 0).all()
    fused = _kernels.fp8_linear(to_device_bf16(x_bits.reshape(1, -1), device), fp8_tensor(w, device),
                                torch.from_numpy(sw).to(device))
    split = _kernels.fp8_decode(fp8_tensor(q, device).view(1, -1), torch.from_numpy(scale).to(device).view(1, -1),
                                fp8_tensor(w, device), torch.from_numpy(sw).to(device))
    assert torch.equal(fused.view(torch.int16), split.view(torch.int16))


def test_block32_invalid_arguments(device):
    x, sx, w, sw = block32_operands(600, 48, 96)
    xt, wt = fp8_tensor(x, device).view(1, -1), fp8_tensor(w, device)
    sxt, swt = torch.from_numpy(sx).to(device).view(1, -1), torch.from_numpy(sw).to(device)
    assert _kernels.fp8_decode_supported(device)
    for operands in ((xt.expand(2, -1).contiguous(), sxt.expand(2, -1).contiguous(), wt, swt),
                     (xt, sxt[:, :2], wt, swt), (xt, sxt[:, :1].expand_as(sxt), wt, swt),
                     (xt, sxt, wt[:40], swt), (xt, sxt, wt, swt[:, :2])):
        with pytest.raises(RuntimeError):
            _kernels.fp8_decode(*operands)
    native, lib = _native.context(device), _native.library()
    status = lib.camblas_cuda_fp8_decode(native.handle, 40, 96, None, None, None, None, 1, 1, 1, None, 0, None)
    assert status == -1 and b"invalid FP8 decode dimensions" in lib.camblas_cuda_error(native.handle)
    status = lib.camblas_cuda_fp8_decode(native.handle, 48, 96, None, None, None, None, 1, 1, 1, None, 0, None)
    assert status == -1 and b"invalid FP8 decode buffers" in lib.camblas_cuda_error(native.handle)
    assert lib.camblas_cuda_fp8_workspace_size(0, 48, 96) == 0 == lib.camblas_cuda_fp8_workspace_size(1, 48, 96)
