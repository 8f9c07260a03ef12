"""Pins the CPU oracle (test infrastructure) before anything is compared against it.

Every oracle function is checked against evidence that does not come from the oracle itself:
the reference's own CPU library compiled from its sources (bit-exact for the scalar kernel), a
third-party codec (torch's float8_e4m3fn / bfloat16 conversions), the known-answer bytes and exact
analytic cases the reference's tests hold (tests/test_quantized.py:33-50 and :160-216,
tests/test_bfloat16.py:94-110, tests/test_mlp_packing.py:120-207, tests/test_float_gemv.py:69-90),
closed forms evaluated independently in numpy FP64, brute-force Python loops on tiny inputs, and
invariants (linearity in a scale, zero and NaN propagation, norm preservation).
"""

import math

import numpy as np
import pytest
import torch

import oracle

GOLDEN = np.load(oracle.HERE.parent / "tests" / "golden" / "linear_path.npz")


# ---------------------------------------------------------------- codecs

def test_e4m3_known_answer_bytes():
    table = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8))
    assert table[0x38] == 1.0 and table[0x40] == 2.0 and table[0x30] == 0.5
    assert table[0x7E] == 448.0 and table[0xFE] == -448.0
    assert table[0x08] == 2.0**-6 and table[0x01] == 2.0**-9 and table[0x00] == 0.0
    assert np.isnan(table[0x7F]) and np.isnan(table[0xFF]) and np.isnan(table).sum() == 2


def test_e4m3_matches_third_party_codec():
    codes = np.arange(256, dtype=np.uint8)
    mine = oracle.e4m3_to_f32(codes)
    theirs = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    finite = ~np.isnan(theirs)
    assert np.array_equal(np.isnan(mine), np.isnan(theirs)) and np.array_equal(mine[finite], theirs[finite])
    rng = np.random.default_rng(1)
    values = np.concatenate([
        (rng.standard_normal(50000) * 100).astype(np.float32),
        (rng.standard_normal(50000) * 0.02).astype(np.float32),
        mine[finite],
        np.float32([447, 448, 449, 464, 480, 1e9, -1e9, 2**-10, 2**-10 * 1.0001, 2**-9 * 1.5, 2**-9 * 2.5]),
    ])
    grid = np.sort(np.unique(np.abs(mine[finite])))
    midpoints = ((grid[:-1].astype(np.float64) + grid[1:]) / 2).astype(np.float32)  # exact ties
    values = np.concatenate([values, midpoints, -midpoints])
    encoded = oracle.f32_to_e4m3(values)
    clamped = torch.from_numpy(np.clip(values, -448, 448)).to(torch.float8_e4m3fn).view(torch.uint8)
    assert np.array_equal(encoded, clamped.numpy())  # saturating, round-to-nearest-even
    assert oracle.f32_to_e4m3(np.float32([np.nan]))[0] == 0x7F
    assert np.array_equal(oracle.f32_to_e4m3(mine[finite]), codes[finite])  # encode(decode(c)) == c


def test_bf16_rounding_matches_third_party():
    rng = np.random.default_rng(2)
    values = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10,
                             np.float32([1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf, 0.0, -0.0])])
    theirs = torch.from_numpy(values).bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(values), theirs)
    assert np.isnan(oracle.bf16_to_f32(oracle.f32_to_bf16(np.float32([np.nan]))))[0]
    assert np.array_equal(oracle.bf16_to_f32(theirs), torch.from_numpy(values).bfloat16().float().numpy())


# ---------------------------------------------------------------- FP32 GEMM

@pytest.mark.skipif(oracle.ref() is None, reason="reference CPU library not built here")
@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
def test_sgemm_bit_exact_with_reference_scalar_kernel(ta, tb):
    m, n, k = 37, 29, 53
    lda, ldb, ldc = (m if ta == "N" else k) + 3, (k if tb == "N" else n) + 2, m + 5
    a = oracle.fill_uniform(1, (lda * (k if ta == "N" else m),))
    b = oracle.fill_uniform(2, (ldb * (n if tb == "N" else k),))
    c0 = oracle.fill_uniform(3, (ldc * n,))
    for alpha, beta in ((1.25, 0.5), (1.0, 0.0), (0.0, 2.0), (2.0, 1.0)):
        mine, theirs = c0.copy(), c0.copy()
        assert oracle.sgemm(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, mine, ldc) == 0
        assert oracle.ref_sgemm_scalar(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, theirs, ldc) == 0
        assert np.array_equal(mine.view(np.uint32), theirs.view(np.uint32))


@pytest.mark.skipif(oracle.ref() is None, reason="reference CPU library not built here")
def test_reference_packed_kernel_agrees_with_fp64_product():
    size = 256
    a = oracle.fill_uniform(4, (size * size,))
    b = oracle.fill_uniform(5, (size * size,))
    c = np.zeros(size * size, np.float32)
    assert oracle.ref_sgemm_packed(4, "N", "N", size, size, size, 1.0, a, size, b, size, 0.0, c, size) == 0
    want = np.zeros(size * size, np.float32)
    want64 = oracle.sgemm_f64("N", "N", size, size, size, 1.0, a, size, b, size, 0.0, want, size, want64=True)
    assert oracle.rel_frobenius(c, want64) <= 1e-6


def test_sgemm_against_numpy_and_exact_integer_products():
    m, n, k = 33, 21, 40
    a = oracle.fill_uniform(6, (k, m))  # column-major A is the transpose of this C-order array
    b = oracle.fill_uniform(7, (n, k))
    c = np.zeros((n, m), np.float32)
    oracle.sgemm("N", "N", m, n, k, 1.0, a.ravel(), m, b.ravel(), k, 0.0, c.ravel(), m)
    want = (a.T.astype(np.float64) @ b.T.astype(np.float64)).T
    assert oracle.rel_frobenius(c, want) <= 1e-6
    c64 = np.zeros((n, m), np.float32)
    oracle.sgemm_f64("N", "N", m, n, k, 1.0, a.ravel(), m, b.ravel(), k, 0.0, c64.ravel(), m)
    assert np.array_equal(c64, want.astype(np.float32))
    # small integers: every product and sum is exact, any order gives the same bits
    # (ref: tests/test_mlp_packing.py:120-207)
    ai = (np.arange(k * m).reshape(k, m) % 7 - 3).astype(np.float32)
    bi = (np.arange(n * k).reshape(n, k) % 5 - 2).astype(np.float32)
    for ta, tb, av, lda, bv, ldb in (("N", "N", ai, m, bi, k), ("T", "T", ai.T.copy(), k, bi.T.copy(), n)):
        ci = np.full((n, m), np.nan, np.float32)
        oracle.sgemm(ta, tb, m, n, k, 2.0, av.ravel(), lda, bv.ravel(), ldb, 0.0, ci.ravel(), m)
        assert np.array_equal(ci, (2 * (ai.T @ bi.T)).T)
    assert oracle.sgemm("X", "N", 1, 1, 1, 1.0, a, 1, b, 1, 0.0, c, 1) == -1
    assert oracle.sgemm("N", "N", 4, 4, 4, 1.0, a, 3, b, 4, 0.0, c, 4) == -1


# ---------------------------------------------------------------- BF16 GEMM

def test_bgemm_exact_cases_and_numpy():
    size = 64
    eye = oracle.f32_to_bf16(np.eye(size, dtype=np.float32))
    x = oracle.f32_to_bf16((np.arange(8 * size).reshape(8, size) % 251 - 125).astype(np.float32))
    y = np.full((8, size), 0x7FC0, np.uint16)
    assert oracle.bgemm_f64("T", "N", size, 8, size, 1.0, eye.ravel(), size, x.ravel(), size, 0.0, y.ravel(), size) == 0
    assert np.array_equal(y, x)  # identity placement; beta == 0 never reads the NaN output
    w = np.zeros((size, size), np.float32)
    w[:, 0], w[:, 1], w[:, 2] = 256, 1, -256
    ones = np.zeros((2, size), np.float32)
    ones[:, :3] = 1
    y = np.zeros((2, size), np.uint16)
    oracle.bgemm_f64("T", "N", size, 2, size, 1.0, oracle.f32_to_bf16(w).ravel(), size,
                     oracle.f32_to_bf16(ones).ravel(), size, 0.0, y.ravel(), size)
    assert (oracle.bf16_to_f32(y) == 1).all()  # needs an accumulator wider than BF16
    xr = oracle.fill_normal_bf16(8, (5, 96))
    wr = oracle.fill_normal_bf16(9, (7, 96))
    c0 = oracle.fill_normal_bf16(10, (5, 7))
    y = c0.copy()
    oracle.bgemm_f64("T", "N", 7, 5, 96, 0.5, wr.ravel(), 96, xr.ravel(), 96, 2.0, y.ravel(), 7)
    want = 0.5 * oracle.linear_bf16_f64(xr, wr) + 2.0 * oracle.bf16_to_f32(c0).astype(np.float64)
    assert np.array_equal(y, oracle.f32_to_bf16(want.astype(np.float32)))
    y = c0.copy()  # alpha == 0: beta scaling only, rounded once
    oracle.bgemm_f64("T", "N", 7, 5, 96, 0.0, wr.ravel(), 96, xr.ravel(), 96, 0.5, y.ravel(), 7)
    assert np.array_equal(y, oracle.f32_to_bf16(np.float32(0.5) * oracle.bf16_to_f32(c0)))


# ---------------------------------------------------------------- FP8 block-128 rule

def brute_force_block_matmul(a, a_scale, w, w_scale):
    table = [float(v) for v in oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8))]
    rows, inner = a.shape
    out = np.zeros((rows, w.shape[0]), np.float32)
    for r in range(rows):
        for n in range(w.shape[0]):
            acc = np.float32(0)
            for g in range(inner // 128):
                dot = math.fsum(table[a[r, g * 128 + i]] * table[w[n, g * 128 + i]] for i in range(128))
                scale = np.float32(a_scale[r, g]) * np.float32(w_scale[n // 128, g])
                # fma(dot, scale, acc) evaluated exactly in FP64 (24+24-bit product fits) and rounded once
                acc = np.float32(np.float64(np.float32(dot)) * np.float64(scale) + np.float64(acc))
            out[r, n] = acc
    return out


def test_fp8_block_rule_brute_force_and_invariants():
    rows, outputs, inner = 2, 130, 256
    a, a_scale = oracle.fill_fp8_blocks(11, rows, inner, 1)
    w, w_scale = oracle.fill_fp8_blocks(12, outputs, inner, 128)
    assert w_scale.shape == (2, 2)
    bits, acc32 = oracle.fp8_block_matmul(a, a_scale, w, w_scale, want32=True)
    assert np.array_equal(acc32, brute_force_block_matmul(a, a_scale, w, w_scale))
    assert np.array_equal(bits, oracle.f32_to_bf16(acc32))
    # doubling every weight scale doubles every output exactly; zero activations give +0
    doubled = oracle.fp8_block_matmul(a, a_scale, w, w_scale * np.float32(2))
    assert np.array_equal(oracle.bf16_to_f32(doubled), 2 * oracle.bf16_to_f32(bits))
    assert not oracle.fp8_block_matmul(np.zeros_like(a), a_scale, w, w_scale).any()
    poisoned = a.copy()
    poisoned[1, 3] = 0x7F
    values = oracle.bf16_to_f32(oracle.fp8_block_matmul(poisoned, a_scale, w, w_scale))
    assert np.isnan(values[1]).all() and np.isfinite(values[0]).all()
    # FP64 yardstick agrees with dequantise-then-matmul in numpy
    dequant_a = oracle.e4m3_to_f32(a).astype(np.float64) * np.repeat(a_scale, 128, axis=1)
    dequant_w = oracle.e4m3_to_f32(w).astype(np.float64) * np.repeat(np.repeat(w_scale, 128, axis=0)[:outputs], 128, axis=1)
    assert oracle.rel_frobenius(oracle.fp8_block_matmul_f64(a, a_scale, w, w_scale), dequant_a @ dequant_w.T) <= 1e-13
    # known answers (ref: tests/test_quantized.py:160-216 restated for 128-blocks)
    ones = np.full((1, 256), 0x38, np.uint8)
    twos = np.full((256, 256), 0x40, np.uint8)
    twos[128:] = 0x30
    out = oracle.bf16_to_f32(oracle.fp8_block_matmul(ones, np.float32([[1.0, 0.5]]), twos,
                                                     np.float32([[1, 1], [4, 8]])))
    assert (out[0, :128] == 384).all() and (out[0, 128:] == 512).all()


def test_activation_quantiser_invariants():
    x = oracle.fill_normal_bf16(13, (3, 384))
    x[1, :128] = 0
    q, scale = oracle.quantise_1x128(x)
    values = oracle.bf16_to_f32(x).reshape(3, 3, 128)
    amax = np.maximum(np.abs(values).max(axis=2), np.float32(1e-10))
    assert np.array_equal(scale, amax * np.float32(1 / 448))
    decoded = oracle.e4m3_to_f32(q).reshape(3, 3, 128)
    assert (np.abs(decoded).max(axis=2)[scale > 1e-9] == 448).all()  # the group maximum maps to +-448
    assert not q.reshape(3, 3, 128)[1, 0].any()
    assert np.abs(decoded * scale[..., None] - values).max() <= np.abs(values).max() * 2.0**-4


def test_activation_quantiser_bytes_match_an_independent_codec():
    # The bytes, not just their invariants: torch's E4M3fn conversion (a third-party codec, round to
    # nearest even) applied to clamp(x * fl(448 / amax), +-448) evaluated in FP32 by torch. A
    # round-half-away encoder, a division by the scale instead of the multiplication by the
    # reciprocal, or a missing clamp each change bytes here. Constructed ties: with amax = 448 the
    # factor is exactly 1, so values halfway between two E4M3 neighbours (17 between 16 and 18,
    # 19 between 18 and 20, 0.0009765625 * 1.5 ... in the subnormal range) must go to the even code.
    rng = np.random.default_rng(77)
    x = oracle.fill_normal_bf16(78, (6, 512))
    ties = np.float32([448, 17, 19, 21, 23, -17, -19, 34, 38, 208, 240, 2.0**-9 * 1.5, 2.0**-9 * 2.5,
                       2.0**-10, -(2.0**-9) * 0.5, 416 + 16, 0.0, 1.0625, 1.1875])
    x[0, : ties.size] = oracle.f32_to_bf16(ties)
    x[0, ties.size:128] = 0
    x[1, 128:256] = oracle.f32_to_bf16(rng.uniform(-3e-5, 3e-5, 128).astype(np.float32))  # tiny group
    x[2, :128] = oracle.f32_to_bf16(np.full(128, 1e30, np.float32))                         # huge group
    q, scale = oracle.quantise_1x128(x)
    values = torch.from_numpy(oracle.bf16_to_f32(x)).reshape(6, 4, 128)
    amax = values.abs().amax(dim=2, keepdim=True).clamp_min(1e-10)
    factor = torch.tensor(448.0, dtype=torch.float32) / amax
    want = torch.clamp(values * factor, -448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    assert np.array_equal(q.reshape(6, 4, 128), want.numpy())
    assert np.array_equal(scale.reshape(6, 4, 1), (amax * torch.tensor(1 / 448, dtype=torch.float32)).numpy())
    # the constructed ties, spelled out: 17 -> 16 (0x58), 19 -> 20 (0x5a), 21 -> 20, 23 -> 24 (0x5c)
    assert list(q[0, 1:5]) == [0x58, 0x5A, 0x5A, 0x5C]


def test_block32_decode_rule_and_power_of_two_quantiser():
    # product: pure-Python chain on a small case, strided scales, the reference's known answers
    # (ref: tests/test_quantized.py:160-216: ones times twos with sx = 0.5, sw = 2, last row block
    # doubled -> 2k and 4k; NaN weights -> NaN)
    outputs, inner = 48, 96
    rng = np.random.default_rng(21)
    x = rng.integers(0, 0x7F, inner, dtype=np.uint8)
    w = rng.integers(0, 0x7F, (outputs, inner), dtype=np.uint8) | (rng.integers(0, 2, (outputs, inner), dtype=np.uint8) << 7)
    w[w == 0xFF] = 0x80
    sx_storage = rng.uniform(0.001, 0.08, (inner // 32, 4)).astype(np.float32)
    sx = sx_storage[:, 0]                                     # padded: element stride 4
    sw = np.asfortranarray(rng.uniform(0.5, 2.0, (2, inner // 32)).astype(np.float32))  # column-major
    got = oracle.fp8_block32_decode(x, sx, w, sw)
    table = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8)).astype(np.float64)
    for n in range(outputs):
        total = np.float32(0)
        for b in range(inner // 32):
            dot = np.float32(sum(table[w[n, b * 32 + i]] * table[x[b * 32 + i]] for i in range(32)))
            scaled = np.float32(dot * sw[n // 32, b])
            total = np.float32(math.fma(float(scaled), float(sx[b]), float(total))) if hasattr(math, "fma") \
                else np.float32(np.float64(scaled) * np.float64(sx[b]) + np.float64(total))
        assert oracle.f32_to_bf16(np.float32([total]))[0] == got[n], n
    k = 5120
    ones, twos = np.full(k, 0x38, np.uint8), np.full((1152, k), 0x40, np.uint8)
    sw = np.full((36, k // 32), 2, np.float32)
    sw[-1] *= 2
    out = oracle.bf16_to_f32(oracle.fp8_block32_decode(ones, np.full(k // 32, 0.5, np.float32), twos, sw))
    assert (out[:-32] == 2 * k).all() and (out[-32:] == 4 * k).all()
    twos[7, 100] = 0x7F
    out = oracle.bf16_to_f32(oracle.fp8_block32_decode(ones, np.full(k // 32, 0.5, np.float32), twos, sw))
    assert np.isnan(out[7]) and np.isfinite(np.delete(out, 7)).all()

    # quantiser: the scale is the smallest power of two not below amax / 448, the bytes are the
    # nearest E4M3 values of x / scale (ties to even), found by search rather than by the encoder
    x_bits = oracle.fill_normal_bf16(22, (256,), std=3.0)
    x_bits[32:64] = oracle.f32_to_bf16(np.float32([448.0 * 2.0**-3] * 32))     # amax/448 exactly a power of two
    x_bits[64:96] = 0
    q, scale = oracle.quantise_block32(x_bits)
    values = oracle.bf16_to_f32(x_bits).astype(np.float64).reshape(8, 32)
    amax = np.maximum(np.abs(values).max(axis=1), 1e-10)
    # the reference takes the exponent of fl32(amax * fl32(1/448)); evaluate that product exactly
    raw = (amax.astype(np.float32) * np.float32(1 / 448)).astype(np.float64)
    want_scale = 2.0 ** np.ceil(np.log2(raw))
    assert np.array_equal(scale.astype(np.float64), want_scale)
    assert scale[1] == 2.0**-3 and scale[2] == 2.0 ** math.ceil(math.log2(np.float32(1e-10) * np.float32(1 / 448)))
    finite = np.where(~np.isnan(table))[0]
    for b in range(8):
        for i in range(32):
            target = min(values[b, i] / want_scale[b], 448.0)
            target = max(target, -448.0)
            distance = np.abs(table[finite] - target)
            best = finite[distance == distance.min()]
            if len(best) > 1:                      # tie (or +-0): even mantissa wins
                best = [c for c in best if c % 2 == 0 and (target != 0 or c == (0x80 if np.signbit(values[b, i]) else 0))] or best
            assert q[b * 32 + i] in best, (b, i, target, q[b * 32 + i], best)


def test_mx_byte_decoder():
    # E2M1: (-1)^s * 2^(e-1) * (1 + m/2) for e > 0, m/2 for e == 0 (OCP microscaling formats);
    # E8M0: 2^(e-127), 255 is NaN; packed order low nibble first; E4M3 weight scales cover 32 rows
    for code in range(16):
        sign, exponent, mantissa = code >> 3, (code >> 1) & 3, code & 1
        value = (mantissa / 2 if exponent == 0 else 2.0 ** (exponent - 1) * (1 + mantissa / 2)) * (-1) ** sign
        assert oracle.E2M1_VALUES[code] == value and np.signbit(oracle.E2M1_VALUES[code]) == bool(sign)
    packed = np.array([[0x21, 0xF7]], np.uint8)                  # nibbles 1, 2, 7, 15
    scales = np.array([[126]], np.uint8)                          # 2^-1 over the one block of 32... (4 here)
    assert np.array_equal(oracle.mx_dequantise(packed, scales, 4, packed=True), [[0.25, 0.5, 3.0, -3.0]])
    bytes_ = np.array([[0x38, 0x40], [0x30, 0xB8]], np.uint8)     # 1, 2 / 0.5, -1
    assert np.array_equal(oracle.mx_dequantise(bytes_, np.array([[0], [254]], np.uint8), 2),
                          [[2.0**-127, 2.0**-126], [2.0**126, -(2.0**127)]])
    assert np.isnan(oracle.mx_dequantise(bytes_, np.array([[255], [127]], np.uint8), 2)[0]).all()
    rows = np.full((40, 32), 0x38, np.uint8)
    block_scales = np.array([[127], [128]], np.uint8)             # rows 0..31 and 32..39
    values = oracle.mx_dequantise(rows, block_scales, 32, weight=True)
    assert (values[:32] == 1).all() and (values[32:] == 2).all()
    ones = np.full((3, 64), 0x38, np.uint8)
    product = oracle.mx_matmul_f64(ones, np.full((3, 2), 128, np.uint8), rows[:, :32].repeat(2, axis=1),
                                   np.array([[127, 127], [128, 128]], np.uint8))
    assert (product[:, :32] == 128).all() and (product[:, 32:] == 256).all()


def test_routing_oracle_hand_worked_case():
    # tokens x choices = 3 x 2, groups serve local experts [1, 0, 1]: the duplicate (third group)
    # gets nothing; expert 7 has no group; -1 and 2^40 are ignored; rows = 2 discards a third row
    experts = np.array([[11, 10], [11, 17], [-1, 11]], np.int64)     # first_expert = 10
    counts, slots, reverse = oracle.route_groups(experts, [1, 0, 1], 10, 2)
    assert counts.tolist() == [3, 1, 0]
    assert slots.tolist() == [[0, 2], [1, -1], [-1, -1]]
    assert reverse.tolist() == [[0, 2], [1, -1], [-1, -1]]
    # reduce: token 0 visits experts in ascending ID order (10 then 11): rows 2 then 0
    grouped = oracle.f32_to_bf16(np.float32([[1, 2**-20], [100, 100], [2**24, 1]]))
    out = oracle.reduce_groups(grouped, experts[:1], np.array([[0, 2]], np.int32))
    assert out.tolist() == [[np.float32(2**24) + np.float32(1), np.float32(1) + np.float32(2**-20)]]
    assert out[0, 0] == 2**24       # one FP32 rounding per step
    out = oracle.reduce_groups(grouped, np.array([[10, 11]], np.int64), np.array([[0, 2]], np.int32))
    assert out[0, 0] == 2**24 and out[0, 1] == np.float32(1) + np.float32(2**-20)


# ---------------------------------------------------------------- decode epilogues

def test_rms_silu_swiglu_closed_forms():
    x = oracle.fill_normal_bf16(14, (3, 256))
    r = oracle.fill_normal_bf16(15, (3, 256))
    w = oracle.fill_normal_bf16(16, (256,), mean=1.0, std=0.1)
    added, out = oracle.rms_norm(2, 2, 1e-5, x, w, residual=r)
    summed = oracle.bf16_to_f32(oracle.f32_to_bf16(oracle.bf16_to_f32(x) + oracle.bf16_to_f32(r)))
    assert np.array_equal(oracle.bf16_to_f32(added), summed)
    scale = (1 / np.sqrt((summed.astype(np.float64) ** 2).mean(axis=1) + 1e-5)).astype(np.float32)
    normalised = oracle.bf16_to_f32(oracle.f32_to_bf16(summed * scale[:, None]))
    assert np.array_equal(out, oracle.f32_to_bf16(normalised * oracle.bf16_to_f32(w)))
    late = oracle.rms_norm(2, 2, 1e-5, x, w, round_before_weight=False)
    values = oracle.bf16_to_f32(x)
    scale = (1 / np.sqrt((values.astype(np.float64) ** 2).mean(axis=1) + 1e-5)).astype(np.float32)
    assert np.array_equal(late, oracle.f32_to_bf16((values * scale[:, None]) * oracle.bf16_to_f32(w)))
    gate = oracle.fill_normal_bf16(17, (2, 64), std=3.0)
    up = oracle.fill_normal_bf16(18, (2, 64))
    g, u = oracle.bf16_to_f32(gate).astype(np.float64), oracle.bf16_to_f32(up)
    silu = oracle.bf16_to_f32(oracle.f32_to_bf16((g / (1 + np.exp(-g))).astype(np.float32)))
    want = oracle.bf16_to_f32(oracle.f32_to_bf16(silu * u))
    got = oracle.bf16_to_f32(oracle.silu_multiply(2, gate, up))
    assert np.abs(got - want).max() <= np.abs(want).max() * 2.0**-7  # libm expf vs FP64 exp: one BF16 ulp
    routing = np.float32([0.5, 2.0])
    routed = oracle.bf16_to_f32(oracle.swiglu(2, 64, 1.0, gate, up, routing))
    gc, uc = np.minimum(g, 1.0), np.clip(u.astype(np.float64), -1.0, 1.0)
    want = (gc / (1 + np.exp(-gc)) * uc) * routing[:, None]
    assert np.abs(routed - want).max() <= np.abs(want).max() * 2.0**-7


def test_rope_and_gqa_textbook():
    x = oracle.fill_normal_bf16(19, (4, 3, 128))
    positions = np.array([0, 1, 100, 2047], np.int32)
    out = oracle.rope(x, positions, 5e5)
    assert np.array_equal(out[0], x[0])
    values, rotated = oracle.bf16_to_f32(x).astype(np.float64), oracle.bf16_to_f32(out).astype(np.float64)
    pairs = values[..., :64] + 1j * values[..., 64:]
    angle = positions[:, None, None] * 5e5 ** (-np.arange(64) / 64.0)
    want = pairs * np.exp(1j * angle)
    assert np.abs(rotated[..., :64] - want.real).max() <= 2.0**-7 * np.abs(values).max()
    assert np.abs(rotated[..., 64:] - want.imag).max() <= 2.0**-7 * np.abs(values).max()
    assert np.allclose((rotated**2).sum(-1), (values**2).sum(-1), rtol=1e-2)  # a rotation keeps the norm
    q = oracle.fill_normal_bf16(20, (2, 4, 128))
    k = oracle.fill_normal_bf16(21, (2, 50, 2, 128))
    v = oracle.fill_normal_bf16(22, (2, 50, 2, 128))
    lengths = np.array([50, 1], np.int32)
    out = oracle.bf16_to_f32(oracle.gqa_decode(q, k, v, lengths, 128**-0.5))
    qf, kf, vf = (oracle.bf16_to_f32(t).astype(np.float64) for t in (q, k, v))
    for b in range(2):
        for h in range(4):
            scores = kf[b, : lengths[b], h // 2] @ qf[b, h] * 128**-0.5
            weights = np.exp(scores - scores.max())
            want = (weights / weights.sum()) @ vf[b, : lengths[b], h // 2]
            assert np.abs(out[b, h] - want).max() <= 2.0**-7 * np.abs(want).max() + 1e-6
    assert np.array_equal(oracle.gqa_decode(q, k, v, lengths, 1.0)[1], np.repeat(v[1, 0], 2, axis=0))


def test_sgemv_exact_sparse_rows():
    w = np.zeros((6, 64), np.float32)
    w[0, 0], w[0, 63], w[0, 7] = 16777216.0, -16777216.0, 3.0
    w[5, 1] = -4.0
    y = oracle.sgemv_f64(1.0, w, np.ones(64, np.float32), 0.0, np.full(6, np.nan, np.float32))
    assert np.array_equal(y, np.float32([3, 0, 0, 0, 0, -4]))


# ---------------------------------------------------------------- committed fixtures

def test_oracle_reproduces_committed_golden_vectors():
    g = GOLDEN
    y = g["bf16_c"].copy()
    oracle.bgemm_f64("T", "N", 64, 8, 256, 0.75, g["bf16_w"], 256, g["bf16_x"], 256, -0.5, y.ravel(), 64)
    assert np.array_equal(y, g["bf16_y_alpha075_beta_m05"])
    assert np.array_equal(oracle.fp8_block_matmul(g["fp8_a"], g["fp8_a_scale"], g["fp8_w"], g["fp8_w_scale"]), g["fp8_out"])
    q, s = oracle.quantise_1x128(g["quant_x"])
    assert np.array_equal(q, g["quant_q"]) and np.array_equal(s, g["quant_scale"])
    added, out = oracle.rms_norm(2, 2, 1e-5, g["rms_x"], g["rms_weight"], residual=g["rms_residual"])
    assert np.array_equal(added, g["rms_added"]) and np.array_equal(out, g["rms_out"])
    assert np.array_equal(oracle.silu_multiply(2, g["act_gate"], g["act_up"]), g["silu_out"])
    assert np.array_equal(oracle.rope(g["rope_x"], g["rope_positions"], 5e5), g["rope_out"])
    assert np.array_equal(oracle.gqa_decode(g["attn_q"], g["attn_k"], g["attn_v"], g["attn_lengths"], 128**-0.5), g["attn_out"])
    want = g["f32_a"].astype(np.float64) @ g["f32_b"].astype(np.float64)
    assert oracle.rel_frobenius(g["f32_c"], want) <= 1e-7
