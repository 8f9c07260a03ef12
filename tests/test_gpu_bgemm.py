"""BF16 GEMM through the C ABI against the CPU oracle.

Strategy follows the reference's BF16 suite (tests/test_bfloat16.py:24-217, tests/test_linear.py):
FP64 accumulation of the exact BF16 operands rounded once to BF16, exact analytic cases that prove
FP32 accumulation and correct placement, alpha/beta and NaN semantics, padded leading dimensions,
changed-input reruns. Tolerance: relative Frobenius error <= 1e-2 against the FP64 product (the
measured error is about 2e-3, the BF16 output rounding). Every MFMA tile variant and split-K
factor is forced in turn so the whole kernel table is covered, not just the planner's choice.
"""

import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _kernels, _native
from helpers import bf16_values, from_device_bf16, ptr, rel_frobenius, to_device_bf16

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-2


def run_bgemm(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, override=None,
              algorithm="auto"):
    at, bt, ct_ = (to_device_bf16(v, device) for v in (a, b, c))
    with _native.algorithm(algorithm):
        native = _native.context(device)
        if override is not None:
            native.call("hip_set_plan_override", override[0], override[1])
        try:
            native.call("bgemm", ta.encode(), tb.encode(), m, n, k, ct.c_float(alpha), ptr(at), lda,
                        ptr(bt), ldb, ct.c_float(beta), ptr(ct_), ldc)
        finally:
            native.call("hip_set_plan_override", -1, 0)
    torch.cuda.synchronize()
    return from_device_bf16(ct_)


def reference(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    want = c.copy()
    status, want64 = oracle.bgemm_f64(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, want, ldc,
                                      want64=True)
    assert status == 0
    return want, want64


def variant_count():
    return _native.library().camblas_hip_kernel_count(2)


@pytest.mark.parametrize("variant", range(8))
@pytest.mark.parametrize("split,n_out,pad", [(1, 300, 4), (3, 300, 4), (1, 301, 4), (2, 301, 4)])
def test_tn_every_variant(device, variant, split, n_out, pad):
    assert variant < variant_count()
    # N is not a multiple of any tile (301: not of 4 either, so the scalar store path runs);
    # M=70 spans tiles; K=328 leaves a K tail
    m_rows, k = 70, 328
    lda, ldb, ldc = k + 8, k + 16, n_out + pad
    w = oracle.fill_normal_bf16(20 + variant, (n_out * lda,))
    x = oracle.fill_normal_bf16(40 + variant, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(60, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(variant, split))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (variant, split, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


# 100 + 100*log2(K blocks per step) + 10*row_tiles + token_tiles; the blocks are limited by
# row_tiles * blocks <= 8 and (row_tiles + token_tiles) * blocks <= 16
STREAM_CODES = [
    100 + 100 * depth + 10 * rows + tokens
    for depth in (0, 1, 2, 3) for rows in range(1, 9) for tokens in (1, 2, 3, 4)
    if (rows << depth) <= 8 and ((rows + tokens) << depth) <= 16
]
# five to eight token tiles (65 to 128 tokens): one K block per step; from 37 tiles on the wavefronts' partial
# tiles are combined in two passes (an odd number of tiles, 7 x 7, included)
MANY_TOKEN_CODES = [100 + 10 * rows + tokens for rows in range(1, 9) for tokens in (5, 6, 7, 8)]


@pytest.mark.parametrize("code", STREAM_CODES)
@pytest.mark.parametrize("n_out,m_rows,pad", [(300, 70, 4), (301, 9, 4), (113, 1, 7)])
@pytest.mark.parametrize("k", [328, 640, 3072])
def test_streaming_kernel_every_variant(device, code, n_out, m_rows, pad, k):
    # ragged feature count, token counts that span and underfill the token tiles, padded leading
    # dimensions; K with a tail (328 is not a multiple of the 128-deep step), and K in whole steps, which
    # takes the variant of the kernel whose loads need no masks (640: five steps of one block, a tail for
    # the deeper steps; 3072: an even number of steps of one to four blocks and three of eight), so an odd
    # number of steps, whose last pair ends with a step past the end, occurs in both
    lda, ldb, ldc = k + 8, k + 16, n_out + pad
    w = oracle.fill_normal_bf16(120 + code, (n_out * lda,))
    x = oracle.fill_normal_bf16(140 + code, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(160, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(code, 1))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (code, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


@pytest.mark.parametrize("code", MANY_TOKEN_CODES)
@pytest.mark.parametrize("n_out,m_rows,k,shares", [(300, 120, 328, 1), (301, 65, 640, 1), (264, 128, 1024, 2)])
def test_streaming_kernel_with_many_token_tiles(device, code, n_out, m_rows, k, shares):
    # ragged feature counts, token counts that fill, underfill and (120 tokens in a tile of 80) span the
    # token tiles, K with and without a tail, K divided over two workgroups
    lda, ldb, ldc = k + 8, k + 16, n_out + 4
    w = oracle.fill_normal_bf16(620 + code, (n_out * lda,))
    x = oracle.fill_normal_bf16(640 + code, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(660, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(code, shares))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (code, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


@pytest.mark.parametrize("code", range(20, 38))
@pytest.mark.parametrize("n_out,m_rows,k", [(300, 70, 320), (512, 256, 64), (260, 513, 448)])
def test_direct_lds_load_kernel(device, code, n_out, m_rows, k):
    # direct global->LDS tiles: ragged N and M (partial tiles, clamped rows), odd and even numbers
    # of 64-deep K steps, padded operand rows
    lda, ldb, ldc = k + 8, k + 16, n_out + 4
    w = oracle.fill_normal_bf16(220 + code, (n_out * lda,))
    x = oracle.fill_normal_bf16(240 + code, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(260, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(code, 1))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (code, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


@pytest.mark.parametrize("code", [38, 39])
@pytest.mark.parametrize("n_out,m_rows,k", [(300, 70, 384), (512, 256, 128), (260, 513, 512), (644, 300, 256)])
def test_four_wavefront_tiles(device, code, n_out, m_rows, k):
    # the four-wavefront 256 x 256 and 320 x 256 tiles with the K loop in assembly: an even number of
    # 64-deep K steps (two steps: the loop body never runs; more: it does), ragged N and M over one
    # and several tiles, padded operand rows
    lda, ldb, ldc = k + 8, k + 16, n_out + 4
    w = oracle.fill_normal_bf16(420 + code, (n_out * lda,))
    x = oracle.fill_normal_bf16(440 + code, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(460, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(code, 1))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (code, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


@pytest.mark.parametrize("code", [38, 39])
def test_four_wavefront_tiles_place_every_output(device, code):
    # x = one-hot rows select single weight columns: y[m, n] = W[n, hot(m)] exactly, so a fragment,
    # accumulator or tile put in the wrong place shows as a wrong value at a known position
    n_out, m_rows, k = 700, 520, 256
    rng = np.random.default_rng(code)
    w = oracle.f32_to_bf16(rng.integers(-64, 64, size=(n_out, k)).astype(np.float32))
    hot = rng.integers(0, k, size=m_rows)
    x32 = np.zeros((m_rows, k), np.float32)
    x32[np.arange(m_rows), hot] = 1.0
    x = oracle.f32_to_bf16(x32)
    c0 = np.zeros((m_rows * n_out,), np.uint16)
    got = run_bgemm(device, "T", "N", n_out, m_rows, k, 1.0, w.reshape(-1), k, x.reshape(-1), k, 0.0, c0, n_out,
                    override=(code, 1))
    want = oracle.bf16_to_f32(w)[:, hot].T
    assert np.array_equal(oracle.bf16_to_f32(got.reshape(m_rows, n_out)), want)


@pytest.mark.parametrize("code", [38, 39])
@pytest.mark.parametrize("shares", [2, 3])
def test_four_wavefront_tiles_with_k_divided_over_workgroups(device, code, shares):
    # ten steps of 64 over 2 (6 + 4) and 3 (4 + 4 + 2) workgroups per tile: shares hold an even number of steps
    n_out, m_rows, k = 260, 513, 640
    lda, ldb, ldc = k + 8, k + 16, n_out + 4
    w = oracle.fill_normal_bf16(520 + code, (n_out * lda,))
    x = oracle.fill_normal_bf16(540 + code, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(560, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(code, shares))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (code, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


@pytest.mark.parametrize("code", [22, 25, 29, 30, 32, 35, 37])
@pytest.mark.parametrize("shares", [2, 3, 7])
def test_direct_lds_load_kernel_with_k_divided_over_workgroups(device, code, shares):
    # 7 steps of 64 over 2 (4 + 3), 3 (3 + 3 + 1) and 7 workgroups per tile; FP32 planes summed in
    # share order by a second kernel, which also applies alpha, beta and the addend
    n_out, m_rows, k = 260, 513, 448
    lda, ldb, ldc = k + 8, k + 16, n_out + 4
    w = oracle.fill_normal_bf16(320 + code, (n_out * lda,))
    x = oracle.fill_normal_bf16(340 + code, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(360, (m_rows * ldc,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=(code, shares))
        want, want64 = reference("T", "N", n_out, m_rows, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(m_rows, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out))
        assert error <= TOLERANCE, (code, alpha, beta, error)
        assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])
    # one share per step: each plane is an exact product of a 64-deep slice, so the sum in share
    # order is reproducible run to run
    again = run_bgemm(device, "T", "N", n_out, m_rows, k, 0.5, w, lda, x, ldb, -1.5, c0, ldc,
                      override=(code, shares))
    assert np.array_equal(got, again)


@pytest.mark.parametrize("tokens", [1, 8, 32, 33, 64, 65, 200])
def test_planned_linear_shapes(device, tokens):
    # aligned fast path as F.linear produces it; planner picks variant and split-K
    outputs, inner = 1024 + 128, 2048
    w = oracle.fill_normal_bf16(70, (outputs, inner), std=0.02)
    x = oracle.fill_normal_bf16(71 + tokens, (tokens, inner))
    native = _native.context(device)
    native.call("reset_stats")
    y = _kernels.linear(to_device_bf16(x, device), to_device_bf16(w, device))
    torch.cuda.synchronize()
    assert _native.stats(device)["lt"] == 1
    assert rel_frobenius(bf16_values(y), oracle.linear_bf16_f64(x, w)) <= TOLERANCE
    # changed-input rerun: nothing about the previous call may be cached
    x2 = oracle.fill_normal_bf16(900 + tokens, (tokens, inner))
    y2 = _kernels.linear(to_device_bf16(x2, device), to_device_bf16(w, device))
    assert rel_frobenius(bf16_values(y2), oracle.linear_bf16_f64(x2, w)) <= TOLERANCE


@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
def test_generic_layouts_and_unaligned(device, ta, tb):
    m, n, k = 45, 38, 51  # odd sizes and leading dimensions: the layout-agnostic kernel with element loads
    lda = (m if ta == "N" else k) + 1
    ldb = (k if tb == "N" else n) + 3
    ldc = m + 2
    a = oracle.fill_normal_bf16(80, (lda * (k if ta == "N" else m),))
    b = oracle.fill_normal_bf16(81, (ldb * (n if tb == "N" else k),))
    c0 = oracle.fill_normal_bf16(82, (ldc * n,))
    got = run_bgemm(device, ta, tb, m, n, k, 1.5, a, lda, b, ldb, 0.25, c0, ldc)
    want, want64 = reference(ta, tb, m, n, k, 1.5, a, lda, b, ldb, 0.25, c0, ldc)
    got2d = got.reshape(n, ldc)
    assert rel_frobenius(oracle.bf16_to_f32(got2d[:, :m]), want64.reshape(n, m)) <= TOLERANCE
    assert np.array_equal(got2d[:, m:], c0.reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
@pytest.mark.parametrize("m,n,k,pad", [(200, 150, 72, 8), (130, 70, 33, 16), (20, 300, 64, 8), (1500, 1400, 40, 0)])
def test_every_layout_on_the_matrix_cores(device, ta, tb, m, n, k, pad):
    # leading dimensions in multiples of eight: 16-byte operand loads, with ragged edges in every
    # dimension (K = 33 ends inside a vector); 20 rows is a sliver and stays on the vector-ALU tiles
    lda = (m if ta == "N" else k) + 7 & ~7
    ldb = (k if tb == "N" else n) + 7 & ~7
    lda, ldb, ldc = lda + pad, ldb + pad, m + 4
    a = oracle.fill_normal_bf16(90, (lda * (k if ta == "N" else m),))
    b = oracle.fill_normal_bf16(91, (ldb * (n if tb == "N" else k),))
    c0 = oracle.fill_normal_bf16(92, (ldc * n,))
    got = run_bgemm(device, ta, tb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc)
    want, want64 = reference(ta, tb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc)
    got2d = got.reshape(n, ldc)
    assert rel_frobenius(oracle.bf16_to_f32(got2d[:, :m]), want64.reshape(n, m)) <= TOLERANCE
    assert np.array_equal(got2d[:, m:], c0.reshape(n, ldc)[:, m:])
    if (ta, tb) != ("T", "N") and m >= 32:
        code = _native.plan_describe(2, ta, tb, m, n, k, lda, ldb, ldc)[0]
        assert code // 1000 == 9


@pytest.mark.parametrize("tokens", [1, 7, 32, 33, 64, 100, 129, 300, 513])
@pytest.mark.parametrize("shares", [None, 2, 7])
def test_outputs_contiguous_weights_with_few_tokens(device, tokens, shares):
    # x @ W with W stored [K, N] ('N','N'): the kernel that streams W as it lies. 264 outputs (two
    # tiles of 128, the second one ragged), 7 steps of 64, padded leading dimensions; up to 512 tokens
    # (513 goes to the layout-agnostic kernel). With K divided over 2 (4 + 3 steps) and 7 workgroups.
    outputs, k = 264, 448
    lda, ldb, ldc = outputs + 8, k + 8, outputs + 4
    w = oracle.fill_normal_bf16(501, (lda * k,))
    x = oracle.fill_normal_bf16(502 + tokens, (ldb * tokens,))
    c0 = oracle.fill_normal_bf16(503, (ldc * tokens,))
    text = _native.plan_describe(2, "N", "N", outputs, tokens, k, lda, ldb, ldc)[1]
    assert ("outputs-contiguous" in text) == (tokens <= 512)
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "N", "N", outputs, tokens, k, alpha, w, lda, x, ldb, beta, c0, ldc,
                        override=None if shares is None else (62, shares))
        want, want64 = reference("N", "N", outputs, tokens, k, alpha, w, lda, x, ldb, beta, c0, ldc)
        got2d = got.reshape(tokens, ldc)
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, :outputs]), want64.reshape(tokens, outputs))
        assert error <= TOLERANCE, (alpha, beta, error)
        assert np.array_equal(got2d[:, outputs:], c0.reshape(tokens, ldc)[:, outputs:])


def test_outputs_contiguous_weights_keep_nan_where_it_belongs(device):
    # a NaN in one token reaches that token's outputs only, a NaN in one column of W that output
    # only; what lies in the padding of W's rows (here NaN) reaches nothing
    outputs, tokens, k = 260, 40, 128
    lda, ldb, ldc = outputs + 12, k, outputs
    nan = np.uint16(0x7FC0)
    w = oracle.fill_normal_bf16(511, (k, lda))
    w[:, outputs:] = nan
    x = oracle.fill_normal_bf16(512, (tokens, ldb))
    clean = run_bgemm(device, "N", "N", outputs, tokens, k, 1.0, w.ravel(), lda, x.ravel(), ldb, 0.0,
                      np.zeros(ldc * tokens, np.uint16), ldc).reshape(tokens, ldc)
    assert not np.isnan(oracle.bf16_to_f32(clean)).any()
    x[5, 77] = nan
    w[100, 9] = nan
    got = oracle.bf16_to_f32(run_bgemm(device, "N", "N", outputs, tokens, k, 1.0, w.ravel(), lda, x.ravel(), ldb,
                                       0.0, np.zeros(ldc * tokens, np.uint16), ldc).reshape(tokens, ldc))
    expected = np.zeros((tokens, outputs), bool)
    expected[5, :] = True
    expected[:, 9] = True
    assert np.array_equal(np.isnan(got), expected)
    assert np.array_equal(got[~expected], oracle.bf16_to_f32(clean)[~expected])


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "T")])
@pytest.mark.parametrize("m,n,k,pad", [(200, 150, 72, 8), (130, 70, 33, 1), (300, 260, 320, 0)])
def test_operands_transposed_into_the_linear_shape(device, ta, tb, m, n, k, pad):
    # the route large products of these layouts take, forced at sizes the oracle finishes quickly:
    # the operands that are not K-contiguous are copied transposed (odd leading dimensions take the
    # element-wise copy, ragged edges in both directions) and the product runs as 'T','N'
    lda = (m if ta == "N" else k) + pad
    ldb = (k if tb == "N" else n) + pad
    ldc = m + 4
    a = oracle.fill_normal_bf16(95, (lda * (k if ta == "N" else m),))
    b = oracle.fill_normal_bf16(96, (ldb * (n if tb == "N" else k),))
    c0 = oracle.fill_normal_bf16(97, (ldc * n,))
    got = run_bgemm(device, ta, tb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc, override=(61, 0))
    want, want64 = reference(ta, tb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc)
    got2d = got.reshape(n, ldc)
    assert rel_frobenius(oracle.bf16_to_f32(got2d[:, :m]), want64.reshape(n, m)) <= TOLERANCE
    assert np.array_equal(got2d[:, m:], c0.reshape(n, ldc)[:, m:])


def test_large_product_of_another_layout_agrees_with_the_layout_agnostic_kernel(device):
    # 1664 x 1600 x 1600 is well past the size from which the planner transposes; the layout-agnostic
    # kernel (forced) is the check, both within the BF16 bar of each other
    m, n, k = 1664, 1600, 1600
    a = oracle.fill_normal_bf16(98, (m * k,))
    b = oracle.fill_normal_bf16(99, (k * n,))
    c0 = np.zeros(m * n, np.uint16)
    native = _native.context(device)
    native.call("reset_stats")
    routed = run_bgemm(device, "N", "N", m, n, k, 1.0, a, m, b, k, 0.0, c0, m)
    assert _native.stats(device)["lt"] == 1
    direct = run_bgemm(device, "N", "N", m, n, k, 1.0, a, m, b, k, 0.0, c0, m, override=(60, 0))
    assert rel_frobenius(oracle.bf16_to_f32(routed), oracle.bf16_to_f32(direct).astype(np.float64)) <= 4e-3
    rows = np.arange(0, m, 97)  # sampled rows of C against FP64
    a2, b2 = oracle.bf16_to_f32(a).reshape(k, m).astype(np.float64), oracle.bf16_to_f32(b).reshape(n, k).astype(np.float64)
    want = (b2 @ a2[:, rows]).astype(np.float64)  # [n, rows]
    assert rel_frobenius(oracle.bf16_to_f32(routed).reshape(n, m)[:, rows], want) <= TOLERANCE


@pytest.mark.parametrize("m,n,k,pad", [(4096, 4096, 256, 0), (3976, 3850, 640, 8)])
def test_weights_as_they_lie_on_the_four_wavefront_tile(device, m, n, k, pad):
    # x @ W with a row-major W and enough tokens that 256 x 256 tiles fill the chip: the planner sends it
    # to the four-wavefront tile that copies W into LDS as it lies and gathers K through transposing LDS
    # reads. Ragged edges in both directions, padded leading dimensions, alpha and beta; checked against
    # the transposing route (a transposed copy of W, then the linear-layer tiles: the same products in
    # the same K order, so the same bits) and, on sampled outputs, against FP64.
    lda, ldb, ldc = m + pad, k + pad, m + (pad and 4)
    text = _native.plan_describe(2, "N", "N", m, n, k, lda, ldb, ldc)[1]
    assert "weights-as-they-lie" in text, text
    a = oracle.fill_normal_bf16(111, (lda * k,))
    b = oracle.fill_normal_bf16(112, (ldb * n,))
    c0 = oracle.fill_normal_bf16(113, (ldc * n,))
    for alpha, beta in ((1.0, 0.0), (0.75, -0.5)):
        got = run_bgemm(device, "N", "N", m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
        routed = run_bgemm(device, "N", "N", m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, override=(61, 0))
        assert np.array_equal(got, routed)
        got2d = got.reshape(n, ldc)
        assert np.array_equal(got2d[:, m:], c0.reshape(n, ldc)[:, m:])
        rows = np.concatenate([np.arange(0, m, 211), [m - 1]])
        a2 = oracle.bf16_to_f32(a).reshape(k, lda)[:, rows].astype(np.float64)
        b2 = oracle.bf16_to_f32(b).reshape(n, ldb)[:, :k].astype(np.float64)
        want = alpha * (b2 @ a2) + beta * oracle.bf16_to_f32(c0).reshape(n, ldc)[:, rows].astype(np.float64)
        assert rel_frobenius(oracle.bf16_to_f32(got2d[:, rows]), want) <= TOLERANCE


@pytest.mark.parametrize("m,n,k,pad", [(296, 260, 256, 8), (264, 70, 384, 0), (1000, 513, 128 * 5, 16)])
def test_weights_as_they_lie_against_the_oracle(device, m, n, k, pad):
    # the same tile forced (code 40) at sizes the oracle finishes: partial tiles in both directions, one to
    # eight workgroups, two to five pairs of K steps, padded leading dimensions, alpha and beta
    lda, ldb, ldc = m + pad, k + pad, m + (pad and 4)
    a = oracle.fill_normal_bf16(121, (lda * k,))
    b = oracle.fill_normal_bf16(122, (ldb * n,))
    c0 = oracle.fill_normal_bf16(123, (ldc * n,))
    for alpha, beta in ((1.0, 0.0), (0.5, -1.5)):
        got = run_bgemm(device, "N", "N", m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, override=(40, 1))
        want, want64 = reference("N", "N", m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
        got2d = got.reshape(n, ldc)
        assert rel_frobenius(oracle.bf16_to_f32(got2d[:, :m]), want64.reshape(n, m)) <= TOLERANCE
        assert np.array_equal(got2d[:, m:], c0.reshape(n, ldc)[:, m:])
    with pytest.raises(RuntimeError):  # the tile is for 'N','N' operands only
        run_bgemm(device, "T", "N", m, n, k, 1.0, a, k + pad, b, ldb, 0.0, c0, ldc, override=(40, 1))


def test_layout_agnostic_kernel_counts_as_a_library_product(device):
    # row-major torch.mm(x, w) with a contiguous [in, out] weight arrives as 'N','N'
    native = _native.context(device)
    native.call("reset_stats")
    x = oracle.fill_normal_bf16(93, (96, 256))
    w = oracle.fill_normal_bf16(94, (256, 160))
    y = _kernels.matmul(to_device_bf16(x, device), to_device_bf16(w, device))
    torch.cuda.synchronize()
    counts = _native.stats(device)
    assert counts["lt"] == 1 and counts["classical"] == 0
    want = oracle.bf16_to_f32(x).astype(np.float64) @ oracle.bf16_to_f32(w).astype(np.float64)
    assert rel_frobenius(bf16_values(y), want) <= TOLERANCE


def test_classical_algorithm_uses_generic_kernel(device):
    outputs, tokens, inner = 256, 16, 256
    w = oracle.fill_normal_bf16(83, (outputs, inner))
    x = oracle.fill_normal_bf16(84, (tokens, inner))
    c = np.zeros(tokens * outputs, np.uint16)
    native = _native.context(device)
    native.call("reset_stats")
    got = run_bgemm(device, "T", "N", outputs, tokens, inner, 1.0, w.ravel(), inner, x.ravel(),
                    inner, 0.0, c, outputs, algorithm="classical")
    counts = _native.stats(device)
    assert counts["classical"] == 1 and counts["lt"] == 0
    assert rel_frobenius(oracle.bf16_to_f32(got).reshape(tokens, outputs),
                         oracle.linear_bf16_f64(x, w)) <= TOLERANCE


@pytest.mark.parametrize("override", [None, (0, 1), (4, 2), (172, 1), (20, 1), (22, 1), (32, 1), (37, 1)])
def test_exact_identity_and_fp32_accumulation(device, override):
    # identity placement (ref: tests/test_bfloat16.py:94-110): W = I gives y = x exactly
    size = 256
    eye = oracle.f32_to_bf16(np.eye(size, dtype=np.float32))
    x = oracle.f32_to_bf16(np.arange(32 * size, dtype=np.float32).reshape(32, size) % 251 - 125)
    got = run_bgemm(device, "T", "N", size, 32, size, 1.0, eye.ravel(), size, x.ravel(), size, 0.0,
                    np.full(32 * size, 0x7FC0, np.uint16), size, override=override)
    assert np.array_equal(got.reshape(32, size), x)
    # [256, 1, -256] . [1, 1, 1] = 1 only when the accumulator is wider than BF16
    w = np.zeros((size, size), np.float32)
    w[:, 0], w[:, 1], w[:, 2] = 256.0, 1.0, -256.0
    ones = np.zeros((8, size), np.float32)
    ones[:, :3] = 1.0
    got = run_bgemm(device, "T", "N", size, 8, size, 1.0, oracle.f32_to_bf16(w).ravel(), size,
                    oracle.f32_to_bf16(ones).ravel(), size, 0.0, np.zeros(8 * size, np.uint16),
                    size, override=override)
    assert np.array_equal(oracle.bf16_to_f32(got), np.ones(8 * size, np.float32))


def test_alpha_zero_beta_and_nan_semantics(device):
    outputs, tokens, inner = 128, 8, 128
    w = oracle.fill_normal_bf16(85, (outputs * inner,))
    x = oracle.fill_normal_bf16(86, (tokens * inner,))
    nan_c = np.full(tokens * outputs, 0x7FC0, np.uint16)
    # beta == 0 never reads C
    got = run_bgemm(device, "T", "N", outputs, tokens, inner, 1.0, w, inner, x, inner, 0.0, nan_c,
                    outputs)
    assert np.isfinite(oracle.bf16_to_f32(got)).all()
    # alpha == 0, beta == 0 writes +0 without reading; beta == 1 is a no-op
    got = run_bgemm(device, "T", "N", outputs, tokens, inner, 0.0, w, inner, x, inner, 0.0, nan_c,
                    outputs)
    assert not got.any()
    c = oracle.fill_normal_bf16(87, (tokens * outputs,))
    got = run_bgemm(device, "T", "N", outputs, tokens, inner, 0.0, w, inner, x, inner, 1.0, c,
                    outputs)
    assert np.array_equal(got, c)
    got = run_bgemm(device, "T", "N", outputs, tokens, inner, 0.0, w, inner, x, inner, 0.5, c,
                    outputs)
    assert np.array_equal(got, oracle.f32_to_bf16(np.float32(0.5) * oracle.bf16_to_f32(c)))
    # NaN in an operand propagates to its output row only (ref: tests/test_bfloat16.py:132-139)
    x_nan = x.copy().reshape(tokens, inner)
    x_nan[3, 17] = 0x7FC0
    got = run_bgemm(device, "T", "N", outputs, tokens, inner, 1.0, w, inner, x_nan.ravel(), inner,
                    0.0, nan_c, outputs).reshape(tokens, outputs)
    values = oracle.bf16_to_f32(got)
    assert np.isnan(values[3]).all() and np.isfinite(np.delete(values, 3, axis=0)).all()


def test_addmm_beta_one_and_errors(device):
    tokens, outputs, inner = 96, 384, 512
    x = oracle.fill_normal_bf16(88, (tokens, inner))
    w = oracle.fill_normal_bf16(89, (outputs, inner), std=0.02)
    c = oracle.fill_normal_bf16(90, (tokens, outputs))
    y = _kernels.addmm(to_device_bf16(c, device), to_device_bf16(x, device),
                       to_device_bf16(w, device).t(), beta=1.0)
    want = oracle.linear_bf16_f64(x, w) + oracle.bf16_to_f32(c).astype(np.float64)
    assert rel_frobenius(bf16_values(y), want) <= TOLERANCE
    native = _native.context(device)
    lib = _native.library()
    buffer = to_device_bf16(c, device)
    status = lib.camblas_cuda_bgemm(native.handle, b"T", b"N", 8, 8, 8, 1.0, ptr(buffer), 8,
                                    ptr(buffer), 8, 0.0, ptr(buffer), 8)
    assert status == -1 and b"aliased BF16 GEMM operand" in lib.camblas_cuda_error(native.handle)
    status = lib.camblas_cuda_bgemm(native.handle, b"T", b"N", 8, 8, 8, 1.0, ptr(buffer), 4,
                                    ptr(buffer), 8, 0.0, ptr(buffer), 8)
    assert status == -1 and b"leading dimension" in lib.camblas_cuda_error(native.handle)


@pytest.mark.parametrize("form", ["row", "row matrix", "pitched", "column", "fp32"])
def test_addmm_bias_forms(device, form):
    tokens, outputs, inner = 40, 264, 320
    x = oracle.fill_normal_bf16(92, (tokens, inner))
    w = oracle.fill_normal_bf16(93, (outputs, inner), std=0.05)
    wide = to_device_bf16(oracle.fill_normal_bf16(94, (tokens, 2 * outputs)), device)
    xt, wt = to_device_bf16(x, device), to_device_bf16(w, device)
    if form == "fp32":  # FP32 operands never take the BF16 epilogue route
        xt, wt, wide = xt.float(), wt.float(), wide.float()
    bias = {"row": wide[0, :outputs], "row matrix": wide[1:2, :outputs], "pitched": wide[:, outputs:],
            "column": wide[:, :1], "fp32": wide[0, :outputs]}[form]
    y = _kernels.addmm(bias, xt, wt.t(), beta=-0.5, alpha=1.25)
    torch.cuda.synchronize()
    want = 1.25 * oracle.linear_bf16_f64(x, w) - 0.5 * bias.double().cpu().numpy()
    assert rel_frobenius(y.double().cpu().numpy(), want) <= (1e-5 if form == "fp32" else TOLERANCE)


def test_long_k_llama_dims(device):
    # down-projection depth (ref: tests/test_bfloat16.py:207-217): K = 28672
    tokens, outputs, inner = 32, 512, 28672
    x = oracle.fill_normal_bf16(91, (tokens, inner))
    w = oracle.fill_normal_bf16(92, (outputs, inner), std=0.02)
    y = _kernels.linear(to_device_bf16(x, device), to_device_bf16(w, device))
    assert rel_frobenius(bf16_values(y), oracle.linear_bf16_f64(x, w)) <= TOLERANCE


def run_bgemm_add(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, z, ldz, c, ldc, override=None,
                  z_offset=0):
    at, bt, ct_ = (to_device_bf16(v, device) for v in (a, b, c))
    zt = to_device_bf16(np.concatenate([np.zeros(z_offset, dtype=np.uint16), z]), device)
    native = _native.context(device)
    if override is not None:
        native.call("hip_set_plan_override", override[0], override[1])
    try:
        native.call("bgemm_add", ta.encode(), tb.encode(), m, n, k, ct.c_float(alpha), ptr(at), lda, ptr(bt), ldb,
                    ct.c_float(beta), ct.c_void_p(zt.data_ptr() + 2 * z_offset), ldz, ptr(ct_), ldc)
    finally:
        native.call("hip_set_plan_override", -1, 0)
    torch.cuda.synchronize()
    return from_device_bf16(ct_)


def spread(z, ldz, m, n, c, ldc):
    """The addend laid over a copy of C: what the reference's addmm does before its beta product."""
    start = c.copy()
    for j in range(n):
        start[j * ldc:j * ldc + m] = z[j * ldz:j * ldz + m]
    return start


@pytest.mark.parametrize("ta,tb,m,n,k,override", [
    ("T", "N", 300, 70, 328, (3, 1)),      # register-staged tiles
    ("T", "N", 300, 70, 328, (1, 3)),      # ... with a split K and the ordered reduction
    ("T", "N", 301, 9, 328, (121, 1)),     # streaming kernel, scalar stores
    ("T", "N", 512, 256, 320, (21, 1)),    # direct-to-LDS tiles
    ("T", "N", 512, 256, 320, (25, 2)),    # ... with K divided and the planes summed by a second kernel
    ("T", "N", 512, 256, 320, (33, 1)),    # direct-to-LDS tiles on the 16 x 16 x 32 instruction
    ("T", "N", 1024, 40, 512, None),       # the planner's choice for a decode batch
    ("N", "N", 200, 150, 72, None),        # any-layout matrix-core kernel: addend spread first
    ("N", "T", 9, 7, 5, None),             # generic kernel: addend spread first
])
@pytest.mark.parametrize("ldz_kind", ["row", "matrix"])
def test_addend_apart_from_the_output(device, ta, tb, m, n, k, override, ldz_kind):
    # C = alpha A B + beta Z equals, bit for bit, the beta form run on a C that holds Z: the same
    # kernel computes both, only the address its epilogue reads differs. And both hold the FP64 bar.
    rng = np.random.default_rng(m + n + k)
    lda = (k if ta == "T" else m) + 8
    ldb = (n if tb == "T" else k) + 8
    ldc = m + 4
    a = oracle.fill_normal_bf16(41, (lda * (m if ta == "T" else k),))
    b = oracle.fill_normal_bf16(42, (ldb * (k if tb == "T" else n),))
    c = oracle.fill_normal_bf16(43, (ldc * n,))
    ldz = 0 if ldz_kind == "row" else m + 12
    z = oracle.fill_normal_bf16(44, (max(ldz, m) * n,))
    alpha, beta = 0.75, -1.5
    got = run_bgemm_add(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, z, ldz, c, ldc, override)
    start = spread(z, ldz, m, n, c, ldc)
    composed = run_bgemm(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, start, ldc, override)
    assert np.array_equal(got, composed)
    want, want64 = reference(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, start, ldc)
    got2d = got.reshape(n, ldc)
    assert rel_frobenius(oracle.bf16_to_f32(got2d[:, :m]), want64.reshape(n, m)) <= TOLERANCE
    assert np.array_equal(got2d[:, m:], c.reshape(n, ldc)[:, m:])  # the padding of C is left alone


@pytest.mark.parametrize("ldz_kind", [None, "row", "matrix"])
def test_plan_that_ends_with_a_second_launch(device, ldz_kind):
    # 28672 outputs x 1024 tokens is 1.4 rounds of 320 x 256 tiles: the planner covers the first
    # 20480 outputs with one whole round and the last 8192 with a second launch of smaller tiles.
    # Weights, output and addend of that launch start at an offset, with padded pitches.
    m, n, k = 28672, 1024, 1024
    lda, ldb, ldc = k + 8, k + 16, m + 4
    assert ", last 8192 outputs " in _native.plan_describe(2, "T", "N", m, n, k, lda, ldb, ldc)[1]
    a = oracle.fill_normal_bf16(51, (lda * m,), std=0.05)
    b = oracle.fill_normal_bf16(52, (ldb * n,))
    c = oracle.fill_normal_bf16(53, (ldc * n,))
    alpha, beta = 0.75, -1.5
    if ldz_kind is None:
        start = c
        got = run_bgemm(device, "T", "N", m, n, k, alpha, a, lda, b, ldb, beta, c, ldc)
    else:
        ldz = 0 if ldz_kind == "row" else m + 12
        z = oracle.fill_normal_bf16(54, (max(ldz, m) * n,))
        start = spread(z, ldz, m, n, c, ldc)
        got = run_bgemm_add(device, "T", "N", m, n, k, alpha, a, lda, b, ldb, beta, z, ldz, c, ldc)
    want, want64 = reference("T", "N", m, n, k, alpha, a, lda, b, ldb, beta, start, ldc)
    got2d = got.reshape(n, ldc)
    for first, last in ((0, 20480), (20480, m)):  # each launch's share holds the bar by itself
        error = rel_frobenius(oracle.bf16_to_f32(got2d[:, first:last]), want64.reshape(n, m)[:, first:last])
        assert error <= TOLERANCE, (first, error)
    assert np.array_equal(got2d[:, m:], c.reshape(n, ldc)[:, m:])


def test_addend_that_is_not_eight_byte_aligned(device):
    # the direct-to-LDS family reads the addend eight bytes at a time; an odd element offset sends
    # the product to the register-staged family, which must still give the FP64-bar answer
    m, n, k = 512, 256, 320
    a = oracle.fill_normal_bf16(51, (k * m,))
    b = oracle.fill_normal_bf16(52, (k * n,))
    z = oracle.fill_normal_bf16(53, (m,))
    c = np.zeros(m * n, dtype=np.uint16)
    got = run_bgemm_add(device, "T", "N", m, n, k, 1.0, a, k, b, k, 1.0, z, 0, c, m, z_offset=1)
    want, want64 = reference("T", "N", m, n, k, 1.0, a, k, b, k, 1.0, spread(z, 0, m, n, c, m), m)
    assert rel_frobenius(oracle.bf16_to_f32(got).reshape(n, m), want64.reshape(n, m)) <= TOLERANCE


def test_addend_argument_checks(device):
    native, lib = _native.context(device), _native.library()
    m, n, k = 64, 8, 32
    a = torch.zeros(m * k, dtype=torch.bfloat16, device=device)
    b = torch.zeros(n * k, dtype=torch.bfloat16, device=device)
    c = torch.ones(m * n + m, dtype=torch.bfloat16, device=device)
    z = torch.full((m * n,), 2.0, dtype=torch.bfloat16, device=device)
    call = lambda *args: lib.camblas_cuda_bgemm_add(native.handle, b"T", b"N", m, n, k, *args)
    one = ct.c_float(1.0)
    assert call(one, ptr(a), k, ptr(b), k, one, ptr(z), m - 1, ptr(c), m) == -1          # ldz below m
    assert call(one, ptr(a), k, ptr(b), k, one, None, 0, ptr(c), m) == -1                # missing addend
    assert call(one, ptr(a), k, ptr(b), k, one, ct.c_void_p(c.data_ptr() + 2 * m), m, ptr(c), m) == -1  # overlaps C
    assert b"aliased" in lib.camblas_cuda_error(native.handle)
    assert call(one, ptr(a), k, ptr(b), k, ct.c_float(0.0), None, 0, ptr(c), m) == 0     # beta 0: never read
    torch.cuda.synchronize()
    assert float(c[:m * n].float().abs().max()) == 0.0
    assert call(ct.c_float(0.0), None, k, None, k, ct.c_float(0.5), ptr(z), 0, ptr(c), m) == 0  # only beta acts
    torch.cuda.synchronize()
    assert torch.equal(c[:m * n].float(), torch.ones(m * n, device=device))


@pytest.mark.parametrize("n_out,m_rows,k,code,shares", [
    (300, 32, 2048, 142, 2),    # 64-row tiles, two shares, ragged rows
    (301, 9, 1664, 121, 3),     # odd N: element-wise partial planes and stores; 13 K steps in three shares
    (512, 32, 4096, 182, 4),    # 128-row tiles
    (256, 64, 1024, 234, 64),   # more shares asked for than K steps exist (k_step 256: four steps)
    (113, 1, 1280, 111, 5),
])
def test_streaming_kernel_with_k_divided_over_workgroups(device, n_out, m_rows, k, code, shares):
    # each share parks FP32 sums, the last workgroup to arrive adds the planes in index order: run
    # twice (the counters must be back at zero) with alpha and beta, against the FP64 product; the
    # second run must reproduce the first bit for bit whatever the arrival order was
    lda, ldb, ldc = k + 8, k + 16, n_out + 4
    w = oracle.fill_normal_bf16(60, (n_out * lda,))
    x = oracle.fill_normal_bf16(61, (m_rows * ldb,))
    c0 = oracle.fill_normal_bf16(62, (m_rows * ldc,))
    first = run_bgemm(device, "T", "N", n_out, m_rows, k, 0.5, w, lda, x, ldb, 2.0, c0, ldc, override=(code, shares))
    again = run_bgemm(device, "T", "N", n_out, m_rows, k, 0.5, w, lda, x, ldb, 2.0, c0, ldc, override=(code, shares))
    assert np.array_equal(first, again)
    want, want64 = reference("T", "N", n_out, m_rows, k, 0.5, w, lda, x, ldb, 2.0, c0, ldc)
    got2d = first.reshape(m_rows, ldc)
    assert rel_frobenius(oracle.bf16_to_f32(got2d[:, :n_out]), want64.reshape(m_rows, n_out)) <= TOLERANCE
    assert np.array_equal(got2d[:, n_out:], c0.reshape(m_rows, ldc)[:, n_out:])


def test_divided_k_linear_under_graph_capture(device):
    # a down-projection-shaped linear ([8192, 8192] weights, 32 tokens) takes the divided-K route of
    # the streaming kernel. Captured after a warm-up it must replay bit-equal to the eager result
    # (the arrival counters are back at zero after every launch); captured on a context that has
    # never run it, the planes and counters cannot be made during the capture and the undivided
    # kernel must run instead, counted as a fallback, with the same answer to the BF16 bar.
    outputs, tokens, inner = 8192, 32, 8192
    assert "k_shares=2" in _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1]
    generator = torch.Generator(device=device).manual_seed(77)
    w = (torch.randn((outputs, inner), device=device, generator=generator) * 0.02).to(torch.bfloat16)
    x = torch.randn((tokens, inner), device=device, generator=generator).to(torch.bfloat16)
    eager = _kernels.matmul(x, w.t())
    torch.cuda.synchronize()
    rows = torch.arange(0, outputs, 251, device=device)
    want = x.double() @ w[rows].double().t()
    assert float((eager[:, rows].double() - want).norm() / want.norm()) <= TOLERANCE

    warm = torch.cuda.Stream()
    warm.wait_stream(torch.cuda.current_stream())
    out = torch.empty_like(eager)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(warm):
        _kernels.matmul(x, w.t(), out=out)  # this stream's context makes its planes and counters
        warm.synchronize()
        with torch.cuda.graph(graph, stream=warm):
            _kernels.matmul(x, w.t(), out=out)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
    graph.reset()

    cold = torch.cuda.Stream()
    cold.wait_stream(torch.cuda.current_stream())
    small = torch.ones((4, 64), device=device, dtype=torch.bfloat16)
    with torch.cuda.stream(cold):
        _kernels.matmul(small, small.t())  # creates the context of this stream, nothing more
        cold.synchronize()
        before = _native.stats(device)["guard_fallback"]
        with torch.cuda.graph(graph, stream=cold):
            _kernels.matmul(x, w.t(), out=out)
        assert _native.stats(device)["guard_fallback"] == before + 1
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert float((out.double() - eager.double()).norm() / eager.double().norm()) <= 4e-3
    graph.reset()


def test_divided_k_result_does_not_depend_on_arrival_order(device):
    # the down projection of the 70B layer, two hundred launches on the same operands: whichever
    # workgroup of a tile arrives last, the planes are added in index order, so every launch must
    # reproduce the first bit for bit (and the counters must have returned to zero each time)
    outputs, tokens, inner = 8192, 32, 28672
    assert "k_shares=2" in _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1]
    generator = torch.Generator(device=device).manual_seed(78)
    w = (torch.randn((outputs, inner), device=device, generator=generator) * 0.02).to(torch.bfloat16)
    x = torch.randn((tokens, inner), device=device, generator=generator).to(torch.bfloat16)
    first = _kernels.matmul(x, w.t())
    out = torch.empty_like(first)
    mismatches = 0
    for _ in range(200):
        _kernels.matmul(x, w.t(), out=out)
        mismatches += int(not torch.equal(out, first))
    assert mismatches == 0
    rows = torch.arange(0, outputs, 257, device=device)
    want = x.double() @ w[rows].double().t()
    assert float((first[:, rows].double() - want).norm() / want.norm()) <= TOLERANCE


@pytest.mark.parametrize("outputs,tokens", [(12288, 33), (10240, 48), (16384, 64)])
def test_mid_width_projection_at_33_to_64_tokens(device, outputs, tokens):
    # the planner sends these to the streaming kernel with K divided over two workgroups per tile
    # (three token tiles up to 48 tokens, four above, 80 to 128 rows per workgroup); sampled output
    # rows against FP64
    inner = 8192
    text = _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1]
    assert "stream" in text and f"tokens={48 if tokens <= 48 else 64}" in text and "k_shares=2" in text, text
    generator = torch.Generator(device=device).manual_seed(outputs + tokens)
    w = (torch.randn((outputs, inner), device=device, generator=generator) * 0.02).to(torch.bfloat16)
    x = torch.randn((tokens, inner), device=device, generator=generator).to(torch.bfloat16)
    y = _kernels.matmul(x, w.t())
    rows = torch.cat([torch.arange(0, outputs, 509, device=device), torch.tensor([outputs - 1], device=device)])
    want = x.double() @ w[rows].double().t()
    got = y[:, rows].double()
    assert float((got - want).norm() / want.norm()) <= TOLERANCE
    bound = 2.0**-7 * want.abs() + 1e-4 * want.abs().max()
    assert bool(((got - want).abs() <= bound).all())


@pytest.mark.parametrize("outputs,inner,tokens,shares", [(8192, 8192, 33, 2), (8192, 28672, 48, 2), (4096, 14336, 64, 4),
                                                         (10240, 8192, 33, 2)])
def test_narrow_projection_at_33_to_64_tokens(device, outputs, inner, tokens, shares):
    # projections with too few rows for a workgroup per compute unit: the streaming kernel with K divided
    # over two or four workgroups of 64 to 128 rows (about one workgroup per compute unit in all); sampled
    # output rows against FP64, and the same bits on every launch (the shares are added in index order)
    text = _native.plan_describe(2, "T", "N", outputs, tokens, inner, inner, inner, outputs)[1]
    assert "stream" in text and f"tokens={48 if tokens <= 48 else 64}" in text and f"k_shares={shares}" in text, text
    generator = torch.Generator(device=device).manual_seed(outputs + tokens)
    w = (torch.randn((outputs, inner), device=device, generator=generator) * 0.02).to(torch.bfloat16)
    x = torch.randn((tokens, inner), device=device, generator=generator).to(torch.bfloat16)
    y = _kernels.matmul(x, w.t())
    for _ in range(20):
        assert torch.equal(_kernels.matmul(x, w.t()), y)
    rows = torch.cat([torch.arange(0, outputs, 509, device=device), torch.tensor([outputs - 1], device=device)])
    want = x.double() @ w[rows].double().t()
    got = y[:, rows].double()
    assert float((got - want).norm() / want.norm()) <= TOLERANCE
    bound = 2.0**-7 * want.abs() + 1e-4 * want.abs().max()
    assert bool(((got - want).abs() <= bound).all())
