/*
 * TEST INFRASTRUCTURE ONLY. CPU restatement of the arithmetic rules of the reference's GPU linear
 * path, used as the checker by tests/, the smoke run and the benchmark's cpu_baseline leg.
 * The product library never links, loads or calls anything in this file.
 *
 * Each function cites the reference source it restates (paths relative to the reference tree).
 * Pinning of each function (what independent evidence it was checked against) is listed in
 * oracle/README.md; a function without an independent check is marked "parity unpinned" there.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- storage codecs */

/* BF16 <-> FP32, round-to-nearest-even; the rule __float2bfloat16_rn applies in
 * src/cuda/bfloat16.cuh:8 and src/cuda/inference_fusion.cuh:14-17. NaN stays NaN (quiet). */
static inline float bf16_to_f32(uint16_t v)
{
    uint32_t bits = (uint32_t)v << 16;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

static inline uint16_t f32_to_bf16(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((bits >> 16) | 0x0040u);
    uint32_t lsb = (bits >> 16) & 1u;
    bits += 0x7fffu + lsb;
    return (uint16_t)(bits >> 16);
}

void oracle_bf16_to_f32(size_t count, const uint16_t *in, float *out)
{
    for (size_t i = 0; i < count; ++i)
        out[i] = bf16_to_f32(in[i]);
}

void oracle_f32_to_bf16(size_t count, const float *in, uint16_t *out)
{
    for (size_t i = 0; i < count; ++i)
        out[i] = f32_to_bf16(in[i]);
}

/* OCP FP8 E4M3 "fn": 1 sign, 4 exponent (bias 7), 3 mantissa, no infinity, NaN = S.1111.111,
 * max finite 448. Same table as the byte decoder in tests/test_quantized.py:33-50. */
static inline float e4m3_to_f32(uint8_t byte)
{
    int sign = byte >> 7, exponent = (byte >> 3) & 15, mantissa = byte & 7;
    float value;
    if (exponent == 15 && mantissa == 7)
        return NAN;
    if (exponent == 0)
        value = ldexpf((float)mantissa, -9);
    else
        value = ldexpf((float)(8 + mantissa), exponent - 10);
    return sign ? -value : value;
}

void oracle_e4m3_to_f32(size_t count, const uint8_t *in, float *out)
{
    for (size_t i = 0; i < count; ++i)
        out[i] = e4m3_to_f32(in[i]);
}

/* FP32 -> E4M3fn, round-to-nearest-even, saturating to +-448 (the reference clamps to +-448
 * before converting: camblas/_hopper.py:94, src/cuda/fp8_decode.cuh:70-71). NaN -> 0x7f. */
static inline uint8_t f32_to_e4m3_sat(float value)
{
    if (isnan(value))
        return 0x7f;
    uint8_t sign = signbit(value) ? 0x80 : 0;
    float a = fabsf(value);
    if (a >= 448.f)
        return sign | 0x7e;
    if (a < ldexpf(1.f, -10)) /* below half of the smallest subnormal 2^-9 */
        return sign;
    int exponent;
    (void)frexpf(a, &exponent); /* a = f * 2^exponent, f in [0.5,1) */
    int e = exponent - 1;       /* a in [2^e, 2^(e+1)) */
    if (e < -6)
        e = -6;                         /* subnormal range shares the 2^-6 binade spacing */
    float step = ldexpf(1.f, e - 3);    /* spacing of representable values in this binade */
    float scaled = a / step;            /* exact: power-of-two division */
    float rounded = nearbyintf(scaled); /* ties-to-even under the default rounding mode */
    int q = (int)rounded;               /* 8..16 for normals, 0..8 for subnormals */
    int biased = e + 7;
    if (e == -6 && q < 8)
        return sign | (uint8_t)q;
    if (q == 16) {
        q = 8;
        biased += 1;
    }
    if (biased > 15 || (biased == 15 && q - 8 > 6))
        return sign | 0x7e;
    return sign | (uint8_t)(biased << 3) | (uint8_t)(q - 8);
}

void oracle_f32_to_e4m3(size_t count, const float *in, uint8_t *out)
{
    for (size_t i = 0; i < count; ++i)
        out[i] = f32_to_e4m3_sat(in[i]);
}

/* ---------------------------------------------------------------- FP32 GEMM */

/* Column-major C = alpha op(A) op(B) + beta C in the arithmetic order of the reference's scalar
 * CPU kernel (src/scalar.c:223-255): C is beta-scaled first (beta==0 stores 0 without reading),
 * then each element receives alpha * acc with acc accumulated in FP32 for l = 0..k-1 using a
 * separate multiply and add. Returns -1 for the argument errors of src/cuda/backend.cu:794-799. */
int oracle_sgemm(char ta, char tb, int m, int n, int k, float alpha, const float *a, int lda,
                 const float *b, int ldb, float beta, float *c, int ldc)
{
    int na = ta == 'N' || ta == 'n', tra = ta == 'T' || ta == 't';
    int nb = tb == 'N' || tb == 'n', trb = tb == 'T' || tb == 't';
    if ((!na && !tra) || (!nb && !trb) || m < 0 || n < 0 || k < 0 || lda < 1 || ldb < 1 || ldc < 1)
        return -1;
    if (m == 0 || n == 0)
        return 0;
    if (!c || lda < (na ? m : k) || ldb < (nb ? k : n) || ldc < m)
        return -1;
#pragma omp parallel for schedule(static)
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            float *out = c + (size_t)i + (size_t)j * ldc;
            if (beta == 0.f)
                *out = 0.f;
            else if (beta != 1.f)
                *out *= beta;
            if (alpha == 0.f || k == 0)
                continue;
            volatile float acc = 0.f; /* volatile: forbid contraction/reassociation */
            for (int l = 0; l < k; ++l) {
                float av = na ? a[(size_t)i + (size_t)l * lda] : a[(size_t)l + (size_t)i * lda];
                float bv = nb ? b[(size_t)l + (size_t)j * ldb] : b[(size_t)j + (size_t)l * ldb];
                volatile float product = av * bv;
                acc = acc + product;
            }
            *out += alpha * acc;
        }
    }
    return 0;
}

/* Same contract with FP64 accumulation and a single final rounding: the "independent CPU FP64
 * product rounded to the storage dtype" the reference's GPU tests compare against
 * (tests/test_cuda.py:38-58). out64 (optional) receives the unrounded FP64 result, dense m*n
 * column-major with leading dimension m. */
int oracle_sgemm_f64(char ta, char tb, int m, int n, int k, float alpha, const float *a, int lda,
                     const float *b, int ldb, float beta, float *c, int ldc, double *out64)
{
    int na = ta == 'N' || ta == 'n', nb = tb == 'N' || tb == 'n';
    if (m <= 0 || n <= 0)
        return 0;
#pragma omp parallel for schedule(static)
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            double acc = 0;
            if (alpha != 0.f)
                for (int l = 0; l < k; ++l) {
                    double av = na ? a[(size_t)i + (size_t)l * lda] : a[(size_t)l + (size_t)i * lda];
                    double bv = nb ? b[(size_t)l + (size_t)j * ldb] : b[(size_t)j + (size_t)l * ldb];
                    acc += av * bv;
                }
            double value = (double)alpha * acc;
            if (beta != 0.f)
                value += (double)beta * (double)c[(size_t)i + (size_t)j * ldc];
            if (out64)
                out64[(size_t)i + (size_t)j * m] = value;
            c[(size_t)i + (size_t)j * ldc] = (float)value;
        }
    }
    return 0;
}

/* ---------------------------------------------------------------- BF16 GEMM */

/* BF16 storage, float alpha/beta, wide accumulation, one RN rounding to BF16
 * (contract of src/cuda/bfloat16.cuh:11-57; beta==0 never reads C, :8). The accumulation is FP64
 * over the exact BF16 operand values, which is what tests/test_bfloat16.py:24-52 compares the
 * vendor GEMM against. out64 (optional) as above. */
int oracle_bgemm_f64(char ta, char tb, int m, int n, int k, float alpha, const uint16_t *a, int lda,
                     const uint16_t *b, int ldb, float beta, uint16_t *c, int ldc, double *out64)
{
    int na = ta == 'N' || ta == 'n', tra = ta == 'T' || ta == 't';
    int nb = tb == 'N' || tb == 'n', trb = tb == 'T' || tb == 't';
    if ((!na && !tra) || (!nb && !trb) || m < 0 || n < 0 || k < 0 || lda < 1 || ldb < 1 || ldc < 1)
        return -1;
    if (m == 0 || n == 0)
        return 0;
    if (!c || lda < (na ? m : k) || ldb < (nb ? k : n) || ldc < m)
        return -1;
#pragma omp parallel for schedule(static)
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            uint16_t *out = c + (size_t)i + (size_t)j * ldc;
            double value;
            if (alpha == 0.f || k == 0) {
                if (beta == 1.f) {
                    if (out64)
                        out64[(size_t)i + (size_t)j * m] = bf16_to_f32(*out);
                    continue;
                }
                value = beta == 0.f ? 0.0 : (double)(beta * bf16_to_f32(*out));
            } else {
                double acc = 0;
                for (int l = 0; l < k; ++l) {
                    double av = bf16_to_f32(na ? a[(size_t)i + (size_t)l * lda]
                                               : a[(size_t)l + (size_t)i * lda]);
                    double bv = bf16_to_f32(nb ? b[(size_t)l + (size_t)j * ldb]
                                               : b[(size_t)j + (size_t)l * ldb]);
                    acc += av * bv;
                }
                value = (double)alpha * acc;
                if (beta != 0.f)
                    value += (double)beta * (double)bf16_to_f32(*out);
            }
            if (out64)
                out64[(size_t)i + (size_t)j * m] = value;
            *out = f32_to_bf16((float)value);
        }
    }
    return 0;
}

/* ---------------------------------------------------------------- FP8 block-128 linear */

/* Dynamic 1x128 activation quantiser (camblas/_hopper.py:82-98): per group of 128 values,
 * amax = max(|x|, 1e-10); scale = amax * (1/448) in FP32; q = e4m3(clamp(x * inv, +-448)) with
 * inv = 448/amax. The reference computes inv with an approximate reciprocal-divide instruction;
 * this restatement uses the IEEE quotient, so FP8 bytes at exact rounding ties of that
 * reciprocal are "parity unpinned" against the reference. The bytes themselves are pinned: the
 * tests recompute x * inv in numpy and convert it with PyTorch's CPU float8_e4m3fn cast, which
 * must give the same byte for every element. */
void oracle_quantise_1x128(int rows, int inner, const uint16_t *x_bf16, uint8_t *q, float *scale)
{
    int groups = inner / 128;
    for (int r = 0; r < rows; ++r)
        for (int g = 0; g < groups; ++g) {
            const uint16_t *src = x_bf16 + (size_t)r * inner + (size_t)g * 128;
            float amax = 1e-10f;
            for (int i = 0; i < 128; ++i) {
                float v = fabsf(bf16_to_f32(src[i]));
                if (v > amax)
                    amax = v;
            }
            scale[(size_t)r * groups + g] = amax * (1.0f / 448.0f);
            float inv = 448.0f / amax;
            for (int i = 0; i < 128; ++i) {
                float v = bf16_to_f32(src[i]) * inv;
                v = fminf(fmaxf(v, -448.f), 448.f);
                q[(size_t)r * inner + (size_t)g * 128 + i] = f32_to_e4m3_sat(v);
            }
        }
}

/* Power-of-two block-32 activation quantiser of src/cuda/fp8_decode.cuh:58-72: per 32 values
 * amax = max(|x|, 1e-10); bits of fl(amax * (1/448)); exponent = biased exponent - 127, plus one
 * unless the mantissa is zero; scale = 2^exponent; q = e4m3(min(x * 2^-exponent, 448)) with a
 * saturating finite conversion (which caps the negative side). The same integer recipe is
 * restated on the CPU in the reference's tests/test_sglang.py:423-445. */
void oracle_quantise_block32(int inner, const uint16_t *x_bf16, uint8_t *q, float *scale)
{
    for (int b = 0; b < inner / 32; ++b) {
        float amax = 1e-10f;
        for (int i = 0; i < 32; ++i) {
            float v = fabsf(bf16_to_f32(x_bf16[b * 32 + i]));
            if (v > amax)
                amax = v;
        }
        float raw = amax * (1.0f / 448.0f);
        uint32_t bits;
        memcpy(&bits, &raw, 4);
        int exponent = (int)((bits >> 23) & 255u) - 127 + ((bits & 0x7fffffu) != 0);
        scale[b] = ldexpf(1.0f, exponent);
        for (int i = 0; i < 32; ++i) {
            float v = ldexpf(bf16_to_f32(x_bf16[b * 32 + i]), -exponent);
            q[b * 32 + i] = f32_to_e4m3_sat(fminf(v, 448.f));
        }
    }
}

/* Single-token block-32 product of src/cuda/fp8_decode.cuh:150-157 for every output row n:
 *     sum = 0;  for b ascending:  sum = fmaf(fl(dot_b * sw[n/32, b]), sx[b], sum)
 * then one RN rounding to BF16. dot_b (32 products of two E4M3 values) is formed exactly in
 * FP64 and rounded once to FP32. Scales are addressed with element strides as in
 * include/camblas_cuda.h:124-137. */
int oracle_fp8_block32_decode(int outputs, int inner, const uint8_t *x, const float *sx,
                              int sx_stride, const uint8_t *w, const float *sw, int sw_row,
                              int sw_col, uint16_t *out)
{
    if (outputs < 1 || inner < 32 || inner % 32)
        return -1;
    float table[256];
    for (int i = 0; i < 256; ++i)
        table[i] = e4m3_to_f32((uint8_t)i);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < outputs; ++n) {
        float sum = 0.f;
        for (int b = 0; b < inner / 32; ++b) {
            double dot = 0.0;
            for (int i = 0; i < 32; ++i)
                dot += (double)table[w[(size_t)n * inner + b * 32 + i]] * (double)table[x[b * 32 + i]];
            float scaled = (float)dot * sw[(size_t)(n / 32) * sw_row + (size_t)b * sw_col];
            sum = fmaf(scaled, sx[(size_t)b * sx_stride], sum);
        }
        out[n] = f32_to_bf16(sum);
    }
    return 0;
}

/* Block-scaled product rule of camblas/_hopper.py:118-126 (unscaled per-group dot, stored FP32)
 * and :168-182 (ordered reduction): for each output (r, n)
 *     acc = 0;  for g ascending:  acc = fmaf(dot_g, a_scale[r,g] * w_scale[n/128, g], acc)
 * with a_scale*w_scale rounded to FP32 first, then one RN rounding to BF16.
 * dot_g is computed exactly (FP64 holds a sum of 128 products of two E4M3 values exactly) and
 * rounded once to FP32; the tensor-core accumulation order inside one group is unspecified in the
 * reference, so this is the correctly rounded member of the family it allows.
 * Shapes: a [rows, inner] bytes, a_scale [rows, inner/128], w [outputs, inner] bytes,
 * w_scale [ceil(outputs/128), inner/128], out BF16 [rows, outputs]. out32 (optional) gets the
 * FP32 accumulator before the BF16 rounding. */
int oracle_fp8_block_matmul(int rows, int outputs, int inner, const uint8_t *a, const float *a_scale,
                            const uint8_t *w, const float *w_scale, uint16_t *out, float *out32)
{
    if (rows < 0 || outputs < 1 || inner < 128 || inner % 128)
        return -1;
    int groups = inner / 128;
    float table[256];
    for (int i = 0; i < 256; ++i)
        table[i] = e4m3_to_f32((uint8_t)i);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < outputs; ++n) {
        const uint8_t *wrow = w + (size_t)n * inner;
        const float *ws = w_scale + (size_t)(n / 128) * groups;
        for (int r = 0; r < rows; ++r) {
            const uint8_t *arow = a + (size_t)r * inner;
            float acc = 0.f;
            for (int g = 0; g < groups; ++g) {
                double dot = 0;
                for (int i = 0; i < 128; ++i)
                    dot += (double)table[arow[g * 128 + i]] * (double)table[wrow[g * 128 + i]];
                volatile float scale = a_scale[(size_t)r * groups + g] * ws[g];
                acc = fmaf((float)dot, scale, acc);
            }
            if (out32)
                out32[(size_t)r * outputs + n] = acc;
            out[(size_t)r * outputs + n] = f32_to_bf16(acc);
        }
    }
    return 0;
}

/* FP64 accumulation of the dequantised operands (value * block scale), the yardstick the
 * tolerance bar is stated against. out64 [rows, outputs]. */
void oracle_fp8_block_matmul_f64(int rows, int outputs, int inner, const uint8_t *a,
                                 const float *a_scale, const uint8_t *w, const float *w_scale,
                                 double *out64)
{
    int groups = inner / 128;
    float table[256];
    for (int i = 0; i < 256; ++i)
        table[i] = e4m3_to_f32((uint8_t)i);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < outputs; ++n) {
        const uint8_t *wrow = w + (size_t)n * inner;
        const float *ws = w_scale + (size_t)(n / 128) * groups;
        for (int r = 0; r < rows; ++r) {
            const uint8_t *arow = a + (size_t)r * inner;
            double acc = 0;
            for (int g = 0; g < groups; ++g) {
                double dot = 0;
                for (int i = 0; i < 128; ++i)
                    dot += (double)table[arow[g * 128 + i]] * (double)table[wrow[g * 128 + i]];
                acc += dot * (double)a_scale[(size_t)r * groups + g] * (double)ws[g];
            }
            out64[(size_t)r * outputs + n] = acc;
        }
    }
}

/* ---------------------------------------------------------------- FP32 GEMV */

/* y = alpha W x + beta y for row-major W [rows, inner] (src/cuda/decode_float.cuh:2-41). The
 * reference fixes a 128-thread-per-row reduction tree that is specific to 32-wide warps; this
 * restatement keeps the same contract with FP64 accumulation (the tolerance form used by
 * tests/test_float_gemv.py:30-60) and the same epilogue fmaf(beta, y, alpha*sum). */
void oracle_sgemv_f64(int rows, int inner, float alpha, const float *w, int ld, const float *x,
                      float beta, float *y)
{
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        double acc = 0;
        for (int l = 0; l < inner; ++l)
            acc += (double)w[(size_t)r * ld + l] * (double)x[l];
        double value = (double)alpha * acc;
        if (beta != 0.f)
            value += (double)beta * (double)y[r];
        y[r] = (float)value;
    }
}

/* ---------------------------------------------------------------- fused decode epilogues */

static inline float load_storage(int dtype, const void *p, size_t i)
{
    return dtype == 0 ? ((const float *)p)[i] : bf16_to_f32(((const uint16_t *)p)[i]);
}

static inline float round_storage(int dtype, float v)
{
    return dtype == 0 ? v : bf16_to_f32(f32_to_bf16(v));
}

static inline void store_storage(int dtype, void *p, size_t i, float v)
{
    if (dtype == 0)
        ((float *)p)[i] = v;
    else
        ((uint16_t *)p)[i] = f32_to_bf16(v);
}

/* silu_multiply (src/cuda/inference_fusion.cuh:19-28): round_T(g/(1+exp(-g))) then
 * round_T(that * u). dtype 0 FP32, 2 BF16. expf here is libm's; the GPU's differs in the last
 * ulp, so tests compare with a one-storage-ulp allowance, as tests/test_inference_fusion.py does. */
void oracle_silu_multiply(int dtype, size_t count, const void *gate, const void *up, void *out)
{
    for (size_t i = 0; i < count; ++i) {
        float g = load_storage(dtype, gate, i);
        float activated = round_storage(dtype, g / (1.f + expf(-g)));
        store_storage(dtype, out, i, activated * load_storage(dtype, up, i));
    }
}

/* swiglu (src/cuda/inference_fusion.cuh:30-51): optional clamp (g<=L, |u|<=L, comparisons keep
 * NaN), FP32 silu(g)*u, optional routing[row] factor, one final rounding. */
void oracle_swiglu(int dtype, size_t count, int width, float limit, const void *gate, const void *up,
                   const float *routing, void *out)
{
    for (size_t i = 0; i < count; ++i) {
        float g = load_storage(dtype, gate, i), u = load_storage(dtype, up, i);
        if (limit > 0) {
            if (g > limit)
                g = limit;
            if (u > limit)
                u = limit;
            if (u < -limit)
                u = -limit;
        }
        volatile float value = (g / (1.f + expf(-g))) * u;
        if (routing) {
            volatile float routed = routing[i / (size_t)width] * value;
            value = routed;
        }
        store_storage(dtype, out, i, value);
    }
}

/* RMSNorm family (src/cuda/inference_fusion.cuh:53-86, :136-191): optional residual add with the
 * sum rounded to storage first; scale = 1/sqrt(mean(v^2) + eps) with the mean taken in FP64 here
 * (the reference copies one specific FP32 reduction tree; its own tolerance-form tests are
 * tests/test_residual_rms.py:64-69); out = round_T(round_T(v*scale) * w) when round_before_weight,
 * else round_T((v*scale) * w). weight_dtype: 0 FP32, 2 BF16. added may be NULL. */
void oracle_rms_norm(int dtype, int weight_dtype, int rows, int width, float epsilon,
                     int round_before_weight, const void *input, const void *residual,
                     const void *weight, void *added, void *out)
{
    for (int r = 0; r < rows; ++r) {
        size_t base = (size_t)r * width;
        double sum = 0;
        for (int i = 0; i < width; ++i) {
            float v = load_storage(dtype, input, base + i);
            if (residual)
                v = round_storage(dtype, v + load_storage(dtype, residual, base + i));
            sum += (double)v * (double)v;
        }
        float scale = (float)(1.0 / sqrt(sum / (double)width + (double)epsilon));
        for (int i = 0; i < width; ++i) {
            float v = load_storage(dtype, input, base + i);
            if (residual) {
                v = round_storage(dtype, v + load_storage(dtype, residual, base + i));
                if (added)
                    store_storage(dtype, added, base + i, v);
            }
            volatile float normalised = v * scale;
            if (round_before_weight)
                normalised = round_storage(dtype, normalised);
            volatile float weighted = normalised * load_storage(weight_dtype, weight, i);
            store_storage(dtype, out, base + i, weighted);
        }
    }
}

/* ---------------------------------------------------------------- RoPE and GQA decode attention */

/* Rotary embedding, "rotate-half" (NeoX/Llama) pairing: for head dim d, pair (i, i + d/2),
 * angle = position * theta^(-2i/d). No reference counterpart (the reference leaves RoPE to the
 * serving engine); textbook formula in FP64, rounded once to BF16. x is [tokens, heads, d] BF16,
 * rotated in place. */
void oracle_rope(int tokens, int heads, int dim, double theta, const int32_t *positions,
                 uint16_t *x)
{
    int half = dim / 2;
    for (int t = 0; t < tokens; ++t)
        for (int h = 0; h < heads; ++h) {
            uint16_t *v = x + ((size_t)t * heads + h) * dim;
            for (int i = 0; i < half; ++i) {
                double angle = (double)positions[t] * pow(theta, -2.0 * i / dim);
                double c = cos(angle), s = sin(angle);
                double lo = bf16_to_f32(v[i]), hi = bf16_to_f32(v[i + half]);
                v[i] = f32_to_bf16((float)(lo * c - hi * s));
                v[i + half] = f32_to_bf16((float)(hi * c + lo * s));
            }
        }
}

/* Grouped-query decode attention, one query token per sequence. No reference counterpart
 * (src/cuda/fusion.cuh:95-157 is dense single-head FP32/FP64 only); textbook softmax(q k^T *
 * scale) v in FP64, one BF16 rounding.
 * q [batch, q_heads, d]; k,v cache [batch, context, kv_heads, d]; out [batch, q_heads, d];
 * lengths[batch] = number of valid cache positions (<= context). */
void oracle_gqa_decode(int batch, int q_heads, int kv_heads, int dim, int context,
                       const int32_t *lengths, double scale, const uint16_t *q, const uint16_t *k,
                       const uint16_t *v, uint16_t *out)
{
    int group = q_heads / kv_heads;
#pragma omp parallel for schedule(static) collapse(2)
    for (int b = 0; b < batch; ++b)
        for (int h = 0; h < q_heads; ++h) {
            int kvh = h / group, len = lengths ? lengths[b] : context;
            const uint16_t *qv = q + ((size_t)b * q_heads + h) * dim;
            double *score = (double *)malloc(sizeof(double) * (size_t)(len > 0 ? len : 1));
            double top = -INFINITY;
            for (int t = 0; t < len; ++t) {
                const uint16_t *kv = k + (((size_t)b * context + t) * kv_heads + kvh) * dim;
                double dot = 0;
                for (int i = 0; i < dim; ++i)
                    dot += (double)bf16_to_f32(qv[i]) * (double)bf16_to_f32(kv[i]);
                score[t] = dot * scale;
                if (score[t] > top)
                    top = score[t];
            }
            double total = 0;
            for (int t = 0; t < len; ++t) {
                score[t] = exp(score[t] - top);
                total += score[t];
            }
            for (int i = 0; i < dim; ++i) {
                double acc = 0;
                for (int t = 0; t < len; ++t)
                    acc += score[t] *
                           (double)bf16_to_f32(v[(((size_t)b * context + t) * kv_heads + kvh) * dim + i]);
                out[((size_t)b * q_heads + h) * dim + i] =
                    f32_to_bf16(len > 0 ? (float)(acc / total) : 0.f);
            }
            free(score);
        }
}

/* ---------------------------------------------------------------- repo-owned counter-based RNG */

/* SplitMix64 of (seed, index): identical streams on every host without any library RNG. Used by
 * tests and the benchmark to generate the same synthetic inputs on both machines. */
static inline uint64_t mix64(uint64_t z)
{
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

static inline double unit_open(uint64_t seed, uint64_t index)
{
    uint64_t bits = mix64(seed * 0x2545f4914f6cdd1dull + index);
    return ((double)(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

void oracle_fill_uniform(uint64_t seed, size_t count, float lo, float hi, float *out)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; ++i)
        out[i] = (float)(lo + (hi - lo) * unit_open(seed, i));
}

void oracle_fill_normal(uint64_t seed, size_t count, float mean, float stddev, float *out)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; ++i) {
        double u1 = unit_open(seed, 2 * i), u2 = unit_open(seed, 2 * i + 1);
        out[i] = (float)(mean + stddev * sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
    }
}

void oracle_fill_normal_bf16(uint64_t seed, size_t count, float mean, float stddev, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; ++i) {
        double u1 = unit_open(seed, 2 * i), u2 = unit_open(seed, 2 * i + 1);
        out[i] = f32_to_bf16(
            (float)(mean + stddev * sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2)));
    }
}

/* FP8 synthetic operand of the block-scaled configuration: N(0,1) draws, each block of
 * block_rows x 128 rescaled so its amax maps to 448, encoded to E4M3fn; scales log-uniform in
 * [1e-4, 1e-1]. block_rows is 1 for activations and 128 for weights. */
void oracle_fill_fp8_blocks(uint64_t seed, int rows, int inner, int block_rows, uint8_t *bytes,
                            float *scales)
{
    int groups = inner / 128, row_blocks = (rows + block_rows - 1) / block_rows;
#pragma omp parallel for schedule(static)
    for (int rb = 0; rb < row_blocks; ++rb)
        for (int g = 0; g < groups; ++g) {
            int r0 = rb * block_rows, r1 = r0 + block_rows > rows ? rows : r0 + block_rows;
            float amax = 0;
            for (int r = r0; r < r1; ++r)
                for (int i = 0; i < 128; ++i) {
                    size_t index = (size_t)r * inner + (size_t)g * 128 + i;
                    double u1 = unit_open(seed, 2 * index), u2 = unit_open(seed, 2 * index + 1);
                    float v = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
                    if (fabsf(v) > amax)
                        amax = fabsf(v);
                }
            float factor = amax > 0 ? 448.f / amax : 0.f;
            for (int r = r0; r < r1; ++r)
                for (int i = 0; i < 128; ++i) {
                    size_t index = (size_t)r * inner + (size_t)g * 128 + i;
                    double u1 = unit_open(seed, 2 * index), u2 = unit_open(seed, 2 * index + 1);
                    float v = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
                    bytes[index] = f32_to_e4m3_sat(v * factor);
                }
            double u = unit_open(seed ^ 0x5ca1ab1eull, (uint64_t)rb * groups + g);
            scales[(size_t)rb * groups + g] = (float)pow(10.0, -4.0 + 3.0 * u);
        }
}
