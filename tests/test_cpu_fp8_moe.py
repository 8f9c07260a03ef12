"""Pins the oracle's restatement of the reference's single-token FP8 mixture-of-experts step
(oracle.fp8_moe_decode_f64; rule of camblas/_hopper.py:329-401) by evidence that does not retype
its formula: a scalar loop that decodes every byte with the OCP E4M3 closed form and walks the
steps one number at a time, an independent restatement of the clipped SiLU-multiply that the
oracle already holds (oracle.swiglu, from src/cuda/inference_fusion.cuh:30-51), and cases whose
answer is known in closed form. The reference tests this step only against SGLang's Triton kernels
on Hopper (tests/test_sglang.py:131-321), which cannot run here."""

import math

import numpy as np

import oracle


def e4m3_value(byte):
    sign = -1.0 if byte & 0x80 else 1.0
    exponent, mantissa = (byte >> 3) & 15, byte & 7
    if exponent == 15 and mantissa == 7:
        return math.nan
    if exponent == 0:
        return sign * mantissa * 2.0 ** -9
    return sign * (1 + mantissa / 8) * 2.0 ** (exponent - 7)


def bf16(value):
    return float(oracle.bf16_to_f32(oracle.f32_to_bf16(np.array([value], np.float32)))[0])


def scalar_moe(x_bits, w1, s1, w2, s2, ids, routing, factor):
    """The step written out element by element (FP64 dot products, the rule's rounding points)."""
    x = [float(v) for v in oracle.bf16_to_f32(x_bits)]
    hidden, width, outputs = len(x), w1.shape[1] // 2, w2.shape[1]

    def quantise(values):
        codes, scales = [], []
        for g in range(len(values) // 128):
            group = values[g * 128:(g + 1) * 128]
            amax = np.float32(max(max(abs(v) for v in group), 1e-10))
            scales.append(float(amax * np.float32(1.0 / 448.0)))
            inverse = np.float32(448.0) / amax
            codes += [int(oracle.f32_to_e4m3(np.array([min(max(np.float32(v) * inverse, -448.0), 448.0)],
                                                      np.float32))[0]) for v in group]
        return codes, scales

    def product(codes, scales, weight, weight_scale):
        result = []
        for n in range(weight.shape[0]):
            acc = 0.0
            for g in range(len(scales)):
                dot = sum(e4m3_value(codes[g * 128 + i]) * e4m3_value(int(weight[n, g * 128 + i])) for i in range(128))
                acc += dot * float(np.float32(scales[g]) * weight_scale[n // 128, g])
            result.append(acc)
        return result

    codes, scales = quantise(x)
    total = np.float32(0.0)
    totals = [np.float32(0.0)] * outputs
    for choice, expert in enumerate(ids):
        up = [bf16(v) for v in product(codes, scales, w1[expert], s1[expert])]
        act = []
        for i in range(width):
            gate, value = min(up[i], 10.0), min(max(up[width + i], -10.0), 10.0)
            act.append(bf16(gate / (1.0 + math.exp(-gate)) * value))
        act_codes, act_scales = quantise(act)
        down = product(act_codes, act_scales, w2[expert], s2[expert])
        for n in range(outputs):
            totals[n] = np.float32(totals[n] + np.float32(bf16(down[n] * float(routing[choice]))))
    del total
    return np.array([float(t) * factor for t in totals])


def small_case(seed, experts=3, choices=2, hidden=128, width=128, outputs=16, magnitude=1.0):
    rng = np.random.default_rng(seed)
    x = oracle.f32_to_bf16((rng.standard_normal(hidden) * magnitude).astype(np.float32))
    w1 = oracle.f32_to_e4m3((rng.standard_normal((experts, 2 * width, hidden)) * 0.6).astype(np.float32))
    w2 = oracle.f32_to_e4m3((rng.standard_normal((experts, outputs, width)) * 0.6).astype(np.float32))
    s1 = (rng.random((experts, 2 * width // 128, hidden // 128)) * 0.05 + 0.01).astype(np.float32)
    s2 = (rng.random((experts, (outputs + 127) // 128, width // 128)) * 0.05 + 0.01).astype(np.float32)
    ids = rng.permutation(experts)[:choices].astype(np.int32)
    routing = rng.random(choices).astype(np.float32) + 0.1
    return x, w1, s1, w2, s2, ids, routing


def test_matches_the_scalar_walk():
    for seed, magnitude in ((1, 1.0), (2, 40.0)):
        case = small_case(seed, magnitude=magnitude)
        got = oracle.fp8_moe_decode_f64(*case, 2.5)
        want = scalar_moe(*case, 2.5)
        # FP64 sums in another order: equal to rounding of the last place of an FP32 total
        assert np.allclose(got, want, rtol=1e-6, atol=1e-9)


def test_activation_is_the_clipped_silu_multiply_the_fusion_oracle_holds():
    # the same activation through oracle.swiglu (restated from another reference file): BF16
    # storage, limit 10; at most one BF16 ulp apart (FP32 against FP64 evaluation before rounding)
    rng = np.random.default_rng(5)
    gate = oracle.f32_to_bf16((rng.standard_normal(4096) * 8).astype(np.float32))
    up = oracle.f32_to_bf16((rng.standard_normal(4096) * 8).astype(np.float32))
    fused = oracle.bf16_to_f32(oracle.swiglu(2, 4096, 10.0, gate, up))
    g = np.minimum(oracle.bf16_to_f32(gate).astype(np.float64), 10.0)
    u = np.clip(oracle.bf16_to_f32(up).astype(np.float64), -10.0, 10.0)
    mine = oracle.bf16_to_f32(oracle.f32_to_bf16((g / (1.0 + np.exp(-g)) * u).astype(np.float32)))
    assert (np.abs(mine - fused) <= np.abs(fused) * 2.0 ** -7 + 1e-30).all()
    assert (mine == fused).mean() > 0.99


def test_closed_forms():
    # weights that pick single inputs: w1 gate row i and up row i read x[i] (code 0x38 = 1.0), w2 is
    # the identity on the first 16 intermediate values; unit block scales. Then
    # out[n] = factor * routing * bf16(silu(min(q(x[n]), 10)) * clamp(q(x[n]), +-10)) re-quantised.
    hidden = width = 128
    outputs = 16
    w1 = np.zeros((1, 2 * width, hidden), np.uint8)
    for i in range(width):
        w1[0, i, i] = w1[0, width + i, i] = 0x38
    w2 = np.zeros((1, outputs, width), np.uint8)
    for n in range(outputs):
        w2[0, n, n] = 0x38
    s1 = np.ones((1, 2, 1), np.float32)
    s2 = np.ones((1, 1, 1), np.float32)
    # powers of two survive both quantisers exactly when the group maximum is 448 * 2^k
    values = np.zeros(hidden, np.float32)
    values[:16] = [7.0, 3.5, 1.75, 0.875, -7.0, -3.5, 14.0, -14.0, 0.0, 0.4375, 28.0, 1.0, 2.0, 4.0, -1.0, -2.0]
    values[127] = 28.0
    x = oracle.f32_to_bf16(values)
    ids, routing = np.array([0], np.int32), np.array([0.5], np.float32)
    got = oracle.fp8_moe_decode_f64(x, w1, s1, w2, s2, ids, routing, 4.0)
    act = []
    for v in values[:16].astype(np.float64):
        gate, value = min(v, 10.0), min(max(v, -10.0), 10.0)
        act.append(bf16(gate / (1.0 + math.exp(-gate)) * value))
    # the intermediate group's maximum is act for 28 -> 10 * 10 / (1 + e^-10); its quantiser has
    # steps of amax / 448 * 2^(e-10): compare through the quantiser the oracle already pins
    q, scale = oracle.quantise_1x128(oracle.f32_to_bf16(np.array(act + [0.0] * 111 + [act[10]], np.float32)).reshape(1, -1))
    expected = oracle.e4m3_to_f32(q[0, :16]).astype(np.float64) * float(scale[0, 0])
    expected = np.array([bf16(v * 0.5) for v in expected]) * 4.0
    assert np.array_equal(got, expected)
    # a gate above the limit is clipped: 14 and 28 give silu(10) * 10
    assert got[6] == got[10]
    # zero routing weight removes a choice exactly; doubling the weights doubles the result
    case = small_case(9, choices=3)
    x2, w1b, s1b, w2b, s2b, ids2, routing2 = case
    dropped = routing2.copy()
    dropped[1] = 0.0
    keep = np.array([0, 2])
    assert np.array_equal(oracle.fp8_moe_decode_f64(x2, w1b, s1b, w2b, s2b, ids2, dropped, 1.5),
                          oracle.fp8_moe_decode_f64(x2, w1b, s1b, w2b, s2b, ids2[keep], routing2[keep], 1.5))
    assert np.array_equal(oracle.fp8_moe_decode_f64(x2, w1b, s1b, w2b, s2b, ids2, routing2 * 2, 1.5),
                          2 * oracle.fp8_moe_decode_f64(x2, w1b, s1b, w2b, s2b, ids2, routing2, 1.5))
