"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU checker.

`oracle/camblas_oracle.c` restates the arithmetic rules of the reference's GPU linear path on the
CPU; `oracle/_ref/libcamblas_ref.so` is the reference's own CPU library compiled from its sources.
Only tests, the smoke run and the benchmark's cpu_baseline leg import this package; the product
package (`camblas_amd`) never does.
"""

import ctypes as ct
import subprocess
from functools import lru_cache
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
_ORACLE = HERE / "_build" / "libcamblas_oracle.so"
_REF = HERE / "_ref" / "libcamblas_ref.so"


def build(reference=True):
    """Compile the restatement (always) and the reference CPU library (when its sources exist)."""
    subprocess.run(["make", "-C", str(HERE), "-B", "oracle"], check=True)
    if reference:
        subprocess.run(["make", "-C", str(HERE), "ref"], check=True)


def _ptr(array):
    return None if array is None else array.ctypes.data_as(ct.c_void_p)


@lru_cache(maxsize=1)
def lib():
    if not _ORACLE.is_file():
        build(reference=False)
    return ct.CDLL(str(_ORACLE))


@lru_cache(maxsize=1)
def ref():
    """The reference CPU library, or None when it was never built (its sources do not travel)."""
    return ct.CDLL(str(_REF)) if _REF.is_file() else None


# ------------------------------------------------------------------ codecs


def bf16_to_f32(bits):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16(ct.c_size_t(values.size), _ptr(values), _ptr(out))
    return out


def e4m3_to_f32(bytes_):
    bytes_ = np.ascontiguousarray(bytes_, dtype=np.uint8)
    out = np.empty(bytes_.shape, dtype=np.float32)
    lib().oracle_e4m3_to_f32(ct.c_size_t(bytes_.size), _ptr(bytes_), _ptr(out))
    return out


def f32_to_e4m3(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, dtype=np.uint8)
    lib().oracle_f32_to_e4m3(ct.c_size_t(values.size), _ptr(values), _ptr(out))
    return out


# ------------------------------------------------------------------ GEMM


def _gemm_args(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    return (
        ct.c_char(ta.encode()),
        ct.c_char(tb.encode()),
        m,
        n,
        k,
        ct.c_float(alpha),
        _ptr(a),
        lda,
        _ptr(b),
        ldb,
        ct.c_float(beta),
        _ptr(c),
        ldc,
    )


def sgemm(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    """Column-major FP32 GEMM in the reference scalar kernel's arithmetic order (in place on c)."""
    return lib().oracle_sgemm(*_gemm_args(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc))


def sgemm_f64(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, want64=False):
    out64 = np.empty(m * n, dtype=np.float64) if want64 else None
    lib().oracle_sgemm_f64(
        *_gemm_args(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc), _ptr(out64)
    )
    return out64


def bgemm_f64(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, want64=False):
    """BF16 (uint16 bit patterns) GEMM with FP64 accumulation, one RN rounding (in place on c)."""
    out64 = np.empty(m * n, dtype=np.float64) if want64 else None
    status = lib().oracle_bgemm_f64(
        *_gemm_args(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc), _ptr(out64)
    )
    return (status, out64) if want64 else status


def ref_sgemm_scalar(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    return ref().ref_sgemm_scalar(*_gemm_args(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc))


def ref_sgemm_packed(threads, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    return ref().ref_sgemm_packed(
        threads, *_gemm_args(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc)
    )


def ref_threads_available():
    return ref().ref_threads_available()


def linear_bf16_f64(x_bits, w_bits):
    """y = x W^T for BF16 bit patterns x [M,K], W [N,K]; FP64 result [M,N] via BLAS dgemm.

    The operands are exact in FP64 and every product is exact, so only the FP64 summation order
    differs from `bgemm_f64` (relative 1e-16): this is the fast form used at larger sizes.
    """
    return bf16_to_f32(x_bits).astype(np.float64) @ bf16_to_f32(w_bits).astype(np.float64).T


# ------------------------------------------------------------------ FP8 block-128


def quantise_1x128(x_bits):
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    rows, inner = x_bits.shape
    q = np.empty((rows, inner), dtype=np.uint8)
    scale = np.empty((rows, inner // 128), dtype=np.float32)
    lib().oracle_quantise_1x128(rows, inner, _ptr(x_bits), _ptr(q), _ptr(scale))
    return q, scale


def quantise_block32(x_bits):
    """Power-of-two block-32 quantiser for one BF16 token [inner]: (E4M3 bytes, FP32 scales)."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16).reshape(-1)
    q = np.empty(x_bits.size, dtype=np.uint8)
    scale = np.empty(x_bits.size // 32, dtype=np.float32)
    lib().oracle_quantise_block32(x_bits.size, _ptr(x_bits), _ptr(q), _ptr(scale))
    return q, scale


def fp8_block32_decode(x, sx, w, sw):
    """Single-token block-32 product; sx [inner/32] and sw [ceil(outputs/32), inner/32] may be
    strided views (their element strides are passed on)."""
    outputs, inner = w.shape
    assert sx.ndim == 1 and sw.ndim == 2 and sx.dtype == np.float32 and sw.dtype == np.float32
    out = np.empty(outputs, dtype=np.uint16)
    x = np.ascontiguousarray(x, dtype=np.uint8).reshape(-1)
    w = np.ascontiguousarray(w, dtype=np.uint8)
    status = lib().oracle_fp8_block32_decode(
        outputs, inner, _ptr(x), ct.c_void_p(sx.ctypes.data), sx.strides[0] // 4, _ptr(w),
        ct.c_void_p(sw.ctypes.data), sw.strides[0] // 4, sw.strides[1] // 4, _ptr(out))
    assert status == 0
    return out


E2M1_VALUES = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.0, -0.5, -1, -1.5, -2, -3, -4, -6], np.float64)


def mx_dequantise(data, scales, block, packed=False, weight=False):
    """FP64 values of E8M0 block-scaled storage (byte decoder of the reference's
    tests/test_quantized.py:12-50, restated in numpy): `data` holds E4M3 bytes [r, k] or, when
    packed, E2M1 nibbles [r, k/2] in low/high order; a scale byte e stands for 2^(e-127) and 255
    for NaN; scales are [r, k/block], or [ceil(r/32), k/32] for E4M3 weights (weight=True)."""
    raw = np.ascontiguousarray(data, dtype=np.uint8)
    if packed:
        values = E2M1_VALUES[np.stack((raw & 15, raw >> 4), -1).reshape(raw.shape[0], -1)]
    else:
        values = e4m3_to_f32(raw).astype(np.float64)
    exponents = np.ascontiguousarray(scales, dtype=np.uint8).astype(np.int64)
    powers = np.ldexp(1.0, exponents - 127)
    powers[exponents == 255] = np.nan
    if weight and not packed:
        powers = np.repeat(powers, 32, axis=0)[: values.shape[0]]
    return values * np.repeat(powers, block, axis=-1)


def mx_matmul_f64(x, sx, w, sw, activation_block=32, packed=False):
    """FP64 product of the dequantised operands: the yardstick for the E8M0 block-scaled linear."""
    with np.errstate(invalid="ignore"):
        return mx_dequantise(x, sx, activation_block) @ mx_dequantise(w, sw, 32, packed, True).T


def route_groups(experts, active, first_expert, rows):
    """Expert routing of include/camblas_cuda.h:168-176 in the reference (kernel:
    src/cuda/routing.cuh:2-24), with a group's rows assigned in ascending slot order:
    returns (counts [groups], slots [groups, rows], reverse [tokens, choices])."""
    experts = np.asarray(experts, dtype=np.int64)
    active = np.asarray(active, dtype=np.int32)
    groups = active.size
    counts = np.zeros(groups, np.int32)
    slots = np.full((groups, rows), -1, np.int32)
    reverse = np.full(experts.shape, -1, np.int32)
    flat_reverse = reverse.reshape(-1)
    for slot, expert in enumerate(experts.reshape(-1)):
        if expert < first_expert or expert >= 2**31 - 1:
            continue
        local = int(expert) - first_expert
        matches = np.nonzero(active == local)[0]
        if matches.size == 0:
            continue
        group = int(matches[0])             # duplicate active IDs select their first group
        row = int(counts[group])
        counts[group] += 1
        if row < rows:
            slots[group, row] = slot
            flat_reverse[slot] = group * rows + row
    return counts, slots, reverse


def reduce_groups(grouped_bits, experts, reverse):
    """FP32 sums of BF16 grouped rows per token in ascending (expert ID, choice) order
    (ref: include/camblas_cuda.h:177-185, src/cuda/routing.cuh:26-56); float32 [tokens, width]."""
    experts = np.asarray(experts, dtype=np.int64)
    reverse = np.asarray(reverse, dtype=np.int32)
    values = bf16_to_f32(np.asarray(grouped_bits, dtype=np.uint16))
    tokens, choices = experts.shape
    out = np.zeros((tokens, values.shape[1]), np.float32)
    for token in range(tokens):
        order = sorted((int(experts[token, c]), c) for c in range(choices)
                       if 0 <= experts[token, c] < 2**31 - 1)
        for _, choice in order:
            row = int(reverse[token, choice])
            if 0 <= row < values.shape[0]:
                out[token] = out[token] + values[row]      # float32 add, one rounding per step
    return out


def fp8_block_matmul(a, a_scale, w, w_scale, want32=False):
    rows, inner = a.shape
    outputs = w.shape[0]
    out = np.empty((rows, outputs), dtype=np.uint16)
    out32 = np.empty((rows, outputs), dtype=np.float32) if want32 else None
    status = lib().oracle_fp8_block_matmul(
        rows, outputs, inner, _ptr(a), _ptr(a_scale), _ptr(w), _ptr(w_scale), _ptr(out), _ptr(out32)
    )
    assert status == 0
    return (out, out32) if want32 else out


def fp8_block_matmul_f64(a, a_scale, w, w_scale):
    rows, inner = a.shape
    outputs = w.shape[0]
    out = np.empty((rows, outputs), dtype=np.float64)
    lib().oracle_fp8_block_matmul_f64(
        rows, outputs, inner, _ptr(a), _ptr(a_scale), _ptr(w), _ptr(w_scale), _ptr(out)
    )
    return out


def fp8_moe_decode_f64(x_bits, w1, s1, w2, s2, ids, routing, factor, limit=10.0):
    """One BF16 token through the reference's FP8 mixture-of-experts step with FP64 dot products
    and the reference's rounding points (camblas/_hopper.py:329-401 `fused`: dynamic 1x128
    quantiser :82-98, ordered scaled products :118-126 and :168-182, clipped SiLU-multiply rounded
    to BF16 :65-80, routing, BF16 rounding and ordered expert sum :305-326). Returns FP64
    [hidden_out], before the final BF16 rounding. Built from the pinned `quantise_1x128` and
    `fp8_block_matmul_f64`; the steps added here are pinned by tests/test_cpu_fp8_moe.py."""
    width = w1.shape[1] // 2
    q, scale = quantise_1x128(np.asarray(x_bits, dtype=np.uint16).reshape(1, -1))
    total = np.zeros(w2.shape[1], dtype=np.float32)
    for choice, expert in enumerate(np.asarray(ids).reshape(-1)):
        up = fp8_block_matmul_f64(q, scale, w1[expert], s1[expert])[0]
        up = bf16_to_f32(f32_to_bf16(up.astype(np.float32))).astype(np.float64)
        gate, value = np.minimum(up[:width], limit), np.clip(up[width:], -limit, limit)
        act = f32_to_bf16((gate / (1.0 + np.exp(-gate)) * value).astype(np.float32))
        q2, scale2 = quantise_1x128(act.reshape(1, -1))
        down = fp8_block_matmul_f64(q2, scale2, w2[expert], s2[expert])[0]
        routed = (down * np.float64(np.float32(routing.reshape(-1)[choice]))).astype(np.float32)
        total = total + bf16_to_f32(f32_to_bf16(routed))  # FP32 sum of BF16 values, choice order
    return total.astype(np.float64) * float(factor)


# ------------------------------------------------------------------ decode epilogues


def sgemv_f64(alpha, w, x, beta, y):
    rows, inner = w.shape
    lib().oracle_sgemv_f64(
        rows, inner, ct.c_float(alpha), _ptr(w), w.strides[0] // 4, _ptr(x), ct.c_float(beta), _ptr(y)
    )
    return y


def silu_multiply(dtype, gate, up):
    out = np.empty_like(gate)
    lib().oracle_silu_multiply(dtype, ct.c_size_t(gate.size), _ptr(gate), _ptr(up), _ptr(out))
    return out


def swiglu(dtype, width, limit, gate, up, routing=None):
    out = np.empty_like(gate)
    lib().oracle_swiglu(
        dtype,
        ct.c_size_t(gate.size),
        width,
        ct.c_float(limit),
        _ptr(gate),
        _ptr(up),
        _ptr(routing),
        _ptr(out),
    )
    return out


def rms_norm(dtype, weight_dtype, epsilon, x, weight, residual=None, round_before_weight=True):
    rows, width = x.shape
    out = np.empty_like(x)
    added = np.empty_like(x) if residual is not None else None
    lib().oracle_rms_norm(
        dtype,
        weight_dtype,
        rows,
        width,
        ct.c_float(epsilon),
        int(round_before_weight),
        _ptr(x),
        _ptr(residual),
        _ptr(weight),
        _ptr(added),
        _ptr(out),
    )
    return (added, out) if residual is not None else out


def rope(x_bits, positions, theta):
    x = np.array(x_bits, dtype=np.uint16, order="C")
    tokens, heads, dim = x.shape
    positions = np.ascontiguousarray(positions, dtype=np.int32)
    lib().oracle_rope(tokens, heads, dim, ct.c_double(theta), _ptr(positions), _ptr(x))
    return x


def gqa_decode(q, k, v, lengths, scale):
    batch, q_heads, dim = q.shape
    _, context, kv_heads, _ = k.shape
    out = np.empty_like(q)
    lengths = None if lengths is None else np.ascontiguousarray(lengths, dtype=np.int32)
    lib().oracle_gqa_decode(
        batch, q_heads, kv_heads, dim, context, _ptr(lengths), ct.c_double(scale), _ptr(q), _ptr(k),
        _ptr(v), _ptr(out),
    )
    return out


# ------------------------------------------------------------------ synthetic inputs


def fill_uniform(seed, shape, lo=-1.0, hi=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib().oracle_fill_uniform(
        ct.c_uint64(seed), ct.c_size_t(out.size), ct.c_float(lo), ct.c_float(hi), _ptr(out)
    )
    return out


def fill_normal(seed, shape, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib().oracle_fill_normal(
        ct.c_uint64(seed), ct.c_size_t(out.size), ct.c_float(mean), ct.c_float(std), _ptr(out)
    )
    return out


def fill_normal_bf16(seed, shape, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.uint16)
    lib().oracle_fill_normal_bf16(
        ct.c_uint64(seed), ct.c_size_t(out.size), ct.c_float(mean), ct.c_float(std), _ptr(out)
    )
    return out


def fill_fp8_blocks(seed, rows, inner, block_rows):
    data = np.empty((rows, inner), dtype=np.uint8)
    scales = np.empty(((rows + block_rows - 1) // block_rows, inner // 128), dtype=np.float32)
    lib().oracle_fill_fp8_blocks(ct.c_uint64(seed), rows, inner, block_rows, _ptr(data), _ptr(scales))
    return data, scales


def rel_frobenius(value, reference):
    value = np.asarray(value, dtype=np.float64)
    reference = np.asarray(reference, dtype=np.float64)
    norm = np.linalg.norm(reference)
    return float(np.linalg.norm(value - reference) / (norm if norm else 1.0))
