"""FP32 GEMM/GEMV through the C ABI against the CPU oracle.

Mirrors the reference's strategy (tests/test_cuda.py:38-58, :285-354; tests/test_float_gemv.py):
independent FP64 product, padded leading dimensions with untouched padding, beta=0 over NaN-filled
C, alpha=0 semantics, exact analytic cases. Tolerance: relative Frobenius error <= 1e-5 against the
FP64 accumulation.
"""

import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from camblas_amd import _native
from helpers import ptr, rel_frobenius

pytestmark = pytest.mark.gpu
TOLERANCE = 1e-5


KERNEL = {"planner": -1, "vector": 0, "matrix": 1, "matrix64": 2}  # FP32 kernels (forced for the test)


def run_sgemm(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, algorithm="auto",
              kernel="planner"):
    at, bt, ct_ = (torch.from_numpy(v).to(device) for v in (a, b, c))
    with _native.algorithm(algorithm):
        native = _native.context(device)
        native.call("hip_set_plan_override", KERNEL[kernel], 0)
        try:
            native.call("sgemm", ta.encode(), tb.encode(), m, n, k, ct.c_float(alpha), ptr(at), lda,
                        ptr(bt), ldb, ct.c_float(beta), ptr(ct_), ldc)
        finally:
            native.call("hip_set_plan_override", -1, 0)
    torch.cuda.synchronize()
    return ct_.cpu().numpy()


@pytest.mark.parametrize("kernel", ["vector", "matrix", "matrix64"])
@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
@pytest.mark.parametrize("shape", [(37, 29, 53), (128, 96, 200), (65, 130, 17), (259, 140, 33)])
def test_sgemm_padded_alpha_beta(device, kernel, ta, tb, shape):
    m, n, k = shape
    lda = (m if ta == "N" else k) + 3
    ldb = (k if tb == "N" else n) + 2
    ldc = m + 5
    a = oracle.fill_uniform(1, (lda * (k if ta == "N" else m),))
    b = oracle.fill_uniform(2, (ldb * (n if tb == "N" else k),))
    c0 = oracle.fill_uniform(3, (ldc * n,))
    got = run_sgemm(device, ta, tb, m, n, k, 1.25, a, lda, b, ldb, -0.5, c0.copy(), ldc, kernel=kernel)
    want = c0.copy()
    want64 = oracle.sgemm_f64(ta, tb, m, n, k, 1.25, a, lda, b, ldb, -0.5, want, ldc, want64=True)
    got2d, c2d = got.reshape(n, ldc), c0.reshape(n, ldc)
    assert rel_frobenius(got2d[:, :m].ravel(), want64.reshape(n, m).ravel()) <= TOLERANCE
    assert np.array_equal(got2d[:, m:], c2d[:, m:]), "padding rows of C were written"
    # the reference's scalar-order result is within the same bar of the FP64 product
    scalar = c0.copy()
    oracle.sgemm(ta, tb, m, n, k, 1.25, a, lda, b, ldb, -0.5, scalar, ldc)
    assert rel_frobenius(got2d[:, :m], scalar.reshape(n, ldc)[:, :m]) <= 5 * TOLERANCE


@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
@pytest.mark.parametrize("n", [1, 5, 31, 40])
def test_sgemm_few_columns_against_a_large_matrix(device, ta, tb, n):
    # a linear layer at a handful of tokens, every layout: matrix-core tiles with K divided over four
    # workgroups per tile (k = 1024, five row tiles) and the planes summed in share order; padded
    # leading dimensions, alpha and beta, untouched padding of C
    m, k = 520, 1024
    lda = (m if ta == "N" else k) + 3
    ldb = (k if tb == "N" else n) + 2
    ldc = m + 5
    tile = "128x32x32" if n <= 32 else "128x64x32"
    assert _native.plan_describe(0, ta, tb, m, n, k, lda, ldb, ldc)[1] == f"f32 mfma {tile} split_k=4" or (
        n == 1 and ta == "T" and tb == "N")
    a = oracle.fill_uniform(11, (lda * (k if ta == "N" else m),))
    b = oracle.fill_uniform(12, (ldb * (n if tb == "N" else k),))
    c0 = oracle.fill_uniform(13, (ldc * n,))
    got = run_sgemm(device, ta, tb, m, n, k, 1.25, a, lda, b, ldb, -0.5, c0.copy(), ldc, algorithm="lt")
    want64 = oracle.sgemm_f64(ta, tb, m, n, k, 1.25, a, lda, b, ldb, -0.5, c0.copy(), ldc, want64=True)
    got2d, c2d = got.reshape(n, ldc), c0.reshape(n, ldc)
    assert rel_frobenius(got2d[:, :m].ravel(), want64.reshape(n, m).ravel()) <= TOLERANCE
    assert np.array_equal(got2d[:, m:], c2d[:, m:]), "padding rows of C were written"
    # beta = 0 over a NaN-filled C
    nan_c = np.full(ldc * n, np.nan, np.float32)
    got = run_sgemm(device, ta, tb, m, n, k, 1.0, a, lda, b, ldb, 0.0, nan_c, ldc, algorithm="lt").reshape(n, ldc)
    want64 = oracle.sgemm_f64(ta, tb, m, n, k, 1.0, a, lda, b, ldb, 0.0, np.zeros(ldc * n, np.float32), ldc,
                              want64=True)
    assert rel_frobenius(got[:, :m].ravel(), want64.reshape(n, m).ravel()) <= TOLERANCE


def test_sgemm_beta_zero_ignores_nan_and_alpha_zero(device):
    m, n, k = 70, 33, 40
    a = oracle.fill_uniform(4, (m * k,))
    b = oracle.fill_uniform(5, (k * n,))
    want = np.zeros(m * n, np.float32)
    want64 = oracle.sgemm_f64("N", "N", m, n, k, 1.0, a, m, b, k, 0.0, want, m, want64=True)
    for kernel in ("vector", "matrix", "matrix64"):
        c = np.full(m * n, np.nan, dtype=np.float32)
        got = run_sgemm(device, "N", "N", m, n, k, 1.0, a, m, b, k, 0.0, c, m, kernel=kernel)
        assert np.isfinite(got).all() and rel_frobenius(got, want64) <= TOLERANCE
    # alpha == 0: beta scaling only; beta == 0 writes zeros over NaN; beta == 1 leaves C alone
    c = np.full(m * n, np.nan, dtype=np.float32)
    assert not run_sgemm(device, "N", "N", m, n, k, 0.0, a, m, b, k, 0.0, c, m).any()
    c = oracle.fill_uniform(6, (m * n,))
    assert np.array_equal(run_sgemm(device, "N", "N", m, n, k, 0.0, a, m, b, k, 1.0, c.copy(), m), c)
    assert np.array_equal(
        run_sgemm(device, "N", "N", m, n, k, 0.0, a, m, b, k, 2.0, c.copy(), m), np.float32(2.0) * c
    )


@pytest.mark.parametrize("kernel", ["vector", "matrix", "matrix64"])
def test_sgemm_full_precision_not_reduced(device, kernel):
    # (1 + 2^-12)^2 needs more than a 10-bit mantissa: a reduced-precision matrix path would
    # return exactly 1 (ref: tests/test_cuda.py:245-270)
    m = n = k = 64
    value = np.float32(1.0 + 2.0**-12)
    a = np.zeros((m, k), np.float32)
    a[np.arange(m), np.arange(m)] = value
    b = a.copy()
    got = run_sgemm(device, "N", "N", m, n, k, 1.0, a.ravel(), m, b.ravel(), k, 0.0,
                    np.zeros(m * n, np.float32), m, kernel=kernel).reshape(n, m)
    assert got[5, 5] == np.float32(value * value)
    # and a sum that needs all 24 bits: 2^12 + 1 + 2^-11 terms in one dot product
    a = np.zeros((m, k), np.float32)
    b = np.zeros((k, n), np.float32)
    a[3, :3] = (4096.0, 1.0, 1.0)
    b[:3, 7] = (1.0, 1.0, 2.0**-11)
    got = run_sgemm(device, "T", "T", m, n, k, 1.0, a.ravel(), k, b.ravel(), n, 0.0,
                    np.zeros(m * n, np.float32), m, kernel=kernel).reshape(n, m)
    assert got[7, 3] == np.float32(4097.0 + 2.0**-11)


def test_sgemm_config1_row_major_2048(device):
    # row-major C = A.B arrives as the swapped column-major call (ref: src/cblas_shim.c:184-199)
    size = 2048
    a = oracle.fill_uniform(101, (size, size))
    b = oracle.fill_uniform(102, (size, size))
    got = run_sgemm(device, "N", "N", size, size, size, 1.0, b.ravel(), size, a.ravel(), size, 0.0,
                    np.zeros(size * size, np.float32), size).reshape(size, size)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert rel_frobenius(got, want) <= TOLERANCE


@pytest.mark.parametrize("rows,inner,pad", [(1024, 4096, 0), (1536, 4100, 8), (1027, 8192, 4)])
def test_sgemv_shortcut(device, rows, inner, pad):
    ld = inner + pad
    w = oracle.fill_uniform(7, (rows, ld))
    x = oracle.fill_uniform(8, (inner,))
    y0 = oracle.fill_uniform(9, (rows,))
    native = _native.context(device)
    native.call("reset_stats")
    got = run_sgemm(device, "T", "N", rows, 1, inner, 0.75, w.ravel(), ld, x, inner, 0.5, y0.copy(),
                    rows)
    want = oracle.sgemv_f64(0.75, w[:, :inner], x, 0.5, y0.copy())
    assert rel_frobenius(got, want) <= TOLERANCE
    assert _native.stats(device)["classical"] >= 1


def test_sgemv_exact_sparse_and_cancellation(device):
    # ref: tests/test_float_gemv.py:69-90: one-hot rows select single inputs exactly, and
    # 256 + 1 - 256 = 1 in full FP32 in any summation order
    rows, inner = 1024, 8192
    w = np.zeros((rows, inner), np.float32)
    w[np.arange(rows), np.arange(rows) * 7] = 1
    x = np.arange(inner, dtype=np.float32)
    got = run_sgemm(device, "T", "N", rows, 1, inner, 1.0, w.ravel(), inner, x, inner, 0.0,
                    np.full(rows, np.nan, np.float32), rows)
    assert np.array_equal(got, x[np.arange(rows) * 7])
    w[:] = 0
    w[:, 0], w[:, 8], w[:, 16] = 256, 1, -256
    got = run_sgemm(device, "T", "N", rows, 1, inner, 1.0, w.ravel(), inner,
                    np.ones(inner, np.float32), inner, 0.0, np.full(rows, np.nan, np.float32), rows)
    assert np.array_equal(got, np.ones(rows, np.float32))


def test_invalid_arguments_report_errors(device):
    native = _native.context(device)
    lib = _native.library()
    status = lib.camblas_cuda_sgemm(native.handle, b"X", b"N", 1, 1, 1, 1.0, None, 1, None, 1, 0.0,
                                    None, 1)
    assert status == -1 and b"invalid GEMM arguments" in lib.camblas_cuda_error(native.handle)
    status = lib.camblas_cuda_sgemm(native.handle, b"N", b"N", 4, 4, 4, 1.0, None, 4, None, 4, 0.0,
                                    None, 4)
    assert status == -1
    assert b"invalid device pointer or leading dimension" in lib.camblas_cuda_error(native.handle)
    assert lib.camblas_cuda_sgemm(native.handle, b"N", b"N", 0, 4, 4, 1.0, None, 1, None, 4, 0.0,
                                  None, 1) == 0
    assert lib.camblas_cuda_dgemm(native.handle, b"N", b"N", 1, 1, 1, 1.0, None, 1, None, 1, 0.0,
                                  None, 1) == -1
    assert b"invalid device pointer" in lib.camblas_cuda_error(native.handle)
    assert lib.camblas_cuda_affine(native.handle, 0, 1, 1, 1, None, None, None, 0, None) == -1
    assert b"missing affine operand" in lib.camblas_cuda_error(native.handle)


def run_dgemm(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, kernel="planner"):
    at, bt, ct_ = (torch.from_numpy(v).to(device) for v in (a, b, c))
    native = _native.context(device)
    native.call("hip_set_plan_override", KERNEL[kernel], 0)
    try:
        native.call("dgemm", ta.encode(), tb.encode(), m, n, k, ct.c_double(alpha), ptr(at), lda,
                    ptr(bt), ldb, ct.c_double(beta), ptr(ct_), ldc)
    finally:
        native.call("hip_set_plan_override", -1, 0)
    torch.cuda.synchronize()
    return ct_.cpu().numpy()


@pytest.mark.parametrize("kernel", ["planner", "vector", "matrix"])
@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
@pytest.mark.parametrize("shape", [(67, 45, 130), (16, 16, 4), (129, 257, 19), (300, 140, 64)])
def test_dgemm_matches_float64_product(device, kernel, ta, tb, shape):
    # FP64 storage and accumulation: the only difference from numpy's product is summation order
    # (vector: LDS-tiled FMA kernel; matrix: v_mfma_f64_16x16x4 tiles; the planner picks by size)
    m, n, k = shape
    lda, ldb, ldc = (m if ta == "N" else k) + 1, (k if tb == "N" else n) + 2, m + 3
    a = oracle.fill_uniform(31, (lda * (k if ta == "N" else m),)).astype(np.float64)
    b = oracle.fill_uniform(32, (ldb * (n if tb == "N" else k),)).astype(np.float64)
    c0 = oracle.fill_uniform(33, (ldc * n,)).astype(np.float64)
    got = run_dgemm(device, ta, tb, m, n, k, 0.75, a, lda, b, ldb, -2.0, c0.copy(), ldc, kernel).reshape(n, ldc)
    left = a.reshape(-1, lda)[:, : (m if ta == "N" else k)]   # column-major storage, rows = columns
    left = left.T if ta == "N" else left                       # -> [m, k]
    right = b.reshape(-1, ldb)[:, : (k if tb == "N" else n)]
    right = right.T if tb == "N" else right                    # -> [k, n]
    want = 0.75 * (left @ right) - 2.0 * c0.reshape(n, ldc)[:, :m].T
    assert rel_frobenius(got[:, :m].T, want) <= 1e-13
    assert np.array_equal(got[:, m:], c0.reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("ta", "NT")
@pytest.mark.parametrize("tb", "NT")
@pytest.mark.parametrize("n", [1, 5, 20, 33, 130])
def test_dgemm_few_columns_against_a_large_matrix(device, ta, tb, n):
    # five (ten at n = 130) row tiles of 128 x 128 against 256 compute units, or of 128 x 16 up to 32
    # columns (n = 20: two column tiles, the second ragged): the planner divides K = 1024 over four
    # workgroups per tile and sums the FP64 planes in share order. Small integers
    # make every order of summation exact; random values are held to the tolerance of the test above.
    m, k = 520, 1024
    lda, ldb, ldc = (m if ta == "N" else k) + 1, (k if tb == "N" else n) + 2, m + 3
    rng = np.random.default_rng(n)
    for exact in (True, False):
        if exact:
            a = rng.integers(-8, 9, lda * (k if ta == "N" else m)).astype(np.float64)
            b = rng.integers(-8, 9, ldb * (n if tb == "N" else k)).astype(np.float64)
            c0 = rng.integers(-8, 9, ldc * n).astype(np.float64)
        else:
            a = oracle.fill_uniform(41, (lda * (k if ta == "N" else m),)).astype(np.float64)
            b = oracle.fill_uniform(42, (ldb * (n if tb == "N" else k),)).astype(np.float64)
            c0 = oracle.fill_uniform(43, (ldc * n,)).astype(np.float64)
        got = run_dgemm(device, ta, tb, m, n, k, 0.5, a, lda, b, ldb, -2.0, c0.copy(), ldc).reshape(n, ldc)
        left = a.reshape(-1, lda)[:, : (m if ta == "N" else k)]
        left = left.T if ta == "N" else left
        right = b.reshape(-1, ldb)[:, : (k if tb == "N" else n)]
        right = right.T if tb == "N" else right
        want = 0.5 * (left @ right) - 2.0 * c0.reshape(n, ldc)[:, :m].T
        if exact:
            assert np.array_equal(got[:, :m].T, want)
        else:
            assert rel_frobenius(got[:, :m].T, want) <= 1e-13
        assert np.array_equal(got[:, m:], c0.reshape(n, ldc)[:, m:]), "padding rows of C were written"
    nan_c = np.full(ldc * n, np.nan)
    got = run_dgemm(device, ta, tb, m, n, k, 1.0, a, lda, b, ldb, 0.0, nan_c, ldc).reshape(n, ldc)
    assert rel_frobenius(got[:, :m].T, left @ right) <= 1e-13


@pytest.mark.parametrize("kernel", ["vector", "matrix"])
def test_dgemm_beta_zero_ignores_nan_and_keeps_full_precision(device, kernel):
    # beta = 0 must not read C; 1 + 2^-40 squared keeps its 2^-39 term only in full FP64 arithmetic
    m, n, k = 48, 33, 20
    a = np.full(m * k, 1.0 + 2.0 ** -40)
    b = np.full(k * n, 1.0 + 2.0 ** -40)
    c = np.full(m * n, np.nan)
    got = run_dgemm(device, "N", "N", m, n, k, 1.0, a, m, b, k, 0.0, c, m, kernel)
    assert np.array_equal(got, np.full(m * n, k * (1.0 + 2.0 ** -39 + 2.0 ** -80)))


@pytest.mark.parametrize("kernel", ["vector", "matrix", "matrix64"])
@pytest.mark.parametrize("shape", [(67, 45, 130), (200, 131, 257), (129, 64, 1024)])
def test_sgemm_exact_rank_two_integer_identity(device, kernel, shape):
    # ref: tests/test_mlp_packing.py:120-207 — A = u v^T + p q^T and B = r s^T + t w^T make A B four
    # outer products of small integers: every product and every partial sum is exact in FP32, so
    # any summation order must give the same bits, and a wrong index shows up exactly
    m, n, k = shape
    i, j, depth = np.arange(m), np.arange(n), np.arange(k)
    v, q, r, t = depth % 5 - 2, depth % 11 - 5, depth % 13 - 6, depth % 3 - 1
    products = [int(np.sum(x * y)) for x, y in ((v, r), (v, t), (q, r), (q, t))]
    for ta in "NT":
        for tb in "NT":
            for change, (alpha, beta) in enumerate([(1.0, 0.0), (0.5, -0.25), (-1.0, 1.0)]):
                u, p = i % 7 - 3 + change, i % 3 - 1 - change
                s, w = j % 5 - 2 - change, j % 7 - 3 + change
                left = (u[:, None] * v + p[:, None] * q).astype(np.float32)       # [m, k]
                right = (r[:, None] * s + t[:, None] * w).astype(np.float32)      # [k, n]
                lda, ldb, ldc = (m if ta == "N" else k) + 3, (k if tb == "N" else n) + 5, m + 7
                a = np.full(lda * (k if ta == "N" else m), -73.0, np.float32)
                b = np.full(ldb * (n if tb == "N" else k), -73.0, np.float32)
                # column-major storage: element (x, y) of the stored matrix at x + y * ld
                stored_a = left if ta == "N" else left.T
                stored_b = right if tb == "N" else right.T
                a.reshape(-1, lda)[:, : stored_a.shape[0]] = stored_a.T
                b.reshape(-1, ldb)[:, : stored_b.shape[0]] = stored_b.T
                c = np.full(ldc * n, np.nan if beta == 0 else 2.0, np.float32)
                c.reshape(n, ldc)[:, m:] = -73.0
                got = run_sgemm(device, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, kernel=kernel)
                expected = alpha * (products[0] * u[:, None] * s + products[1] * u[:, None] * w
                                    + products[2] * p[:, None] * s + products[3] * p[:, None] * w) + beta * 2.0
                assert np.array_equal(got.reshape(n, ldc)[:, :m].T, expected.astype(np.float32)), (ta, tb, change)
                assert (got.reshape(n, ldc)[:, m:] == -73.0).all()


@pytest.mark.parametrize("kernel", ["matrix64", "vector"])
def test_more_column_tiles_than_one_grid_dimension_holds(device, kernel):
    # a grid dimension holds 65535 tiles: 64-column tiles cover 4,194,240 columns. A product with
    # more columns (row-major: a tall left operand times a small matrix) is launched panel by
    # panel; columns on both sides of the seam and at the far end are compared with FP64 products.
    m, k = 40, 16
    n = 65535 * 64 + 70
    rng = np.random.default_rng(11)
    a = torch.from_numpy(rng.uniform(-1, 1, (k, m)).astype(np.float32)).to(device)      # column-major [m, k]
    b = (torch.rand((n, k), device=device, dtype=torch.float32) * 2 - 1)                 # column-major [k, n]
    c = torch.full((n, m), float("nan"), device=device, dtype=torch.float32)
    native = _native.context(device)
    native.call("hip_set_plan_override", KERNEL[kernel], 0)
    try:
        native.call("sgemm", b"N", b"N", m, n, k, ct.c_float(1.0), ptr(a), m, ptr(b), k, ct.c_float(0.0),
                    ptr(c), m)
    finally:
        native.call("hip_set_plan_override", -1, 0)
    torch.cuda.synchronize()
    seam = 65535 * 64
    columns = np.r_[0:64, seam - 64:seam + 70, n - 64:n]
    got = c[columns].cpu().numpy().astype(np.float64)
    want = b[columns].cpu().numpy().astype(np.float64) @ a.cpu().numpy().astype(np.float64)
    assert rel_frobenius(got.ravel(), want.ravel()) <= TOLERANCE
    assert bool(torch.isfinite(c).all())
