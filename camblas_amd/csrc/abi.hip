// extern "C" surface of libcamblas_hip.so: context lifetime, argument validation in the
// reference's order, planning and dispatch. No kernel lives here.
#include "common.hpp"

#include <algorithm>
#include <limits>
#include <cmath>
#include <climits>
#include <cstring>
#include <exception>
#include <new>

namespace camblas_hip
{
namespace
{
thread_local char creation_error[256] = "";
}

int fail(camblas_cuda_context *context, const char *operation, int code)
{
    char *message = context ? context->error : creation_error;
    std::snprintf(message, 256, "%s failed (status %d)", operation, code);
    return code > 0 ? -code : -1;
}

hipError_t reserve_scratch(camblas_cuda_context *context, size_t bytes)
{
    if (bytes <= context->scratch_bytes)
        return hipSuccess;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    hipStreamIsCapturing(context->stream, &capture);
    if (capture != hipStreamCaptureStatusNone)
        return hipErrorStreamCaptureUnsupported;
    size_t wanted = std::max(bytes, context->scratch_bytes * 2);
    wanted = (wanted + 255) & ~size_t(255);
    void *fresh = nullptr;
    hipError_t status = hipMalloc(&fresh, wanted);
    if (status != hipSuccess) {
        (void)hipGetLastError();
        return status;
    }
    // Earlier launches (possibly captured) may still reference the old arena.
    if (context->scratch)
        context->retired.push_back(context->scratch);
    context->scratch = fresh;
    context->scratch_bytes = wanted;
    return hipSuccess;
}

namespace
{
// Activates the context's device for one call and restores the caller's (ref: backend.cu:913-932).
class DeviceScope
{
    int previous = -1;
    bool changed = false;

  public:
    hipError_t status;
    explicit DeviceScope(int device) : status(hipGetDevice(&previous))
    {
        if (status == hipSuccess && previous != device) {
            status = hipSetDevice(device);
            changed = status == hipSuccess;
        }
    }
    ~DeviceScope()
    {
        if (changed)
            (void)hipSetDevice(previous);
    }
};

// ref: backend.cu:934-951
template <typename Function> int execute(camblas_cuda_context *context, Function function)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    DeviceScope device(context->device);
    if (device.status != hipSuccess)
        return fail(context, "activate device", device.status);
    try {
        return function();
    } catch (const std::bad_alloc &) {
        return fail(context, "host allocation", 2);
    } catch (const std::exception &error) {
        std::snprintf(context->error, sizeof(context->error), "host exception: %s", error.what());
        return -1;
    } catch (...) {
        return fail(context, "unexpected host exception", 1);
    }
}

bool is_n(char t) { return t == 'N' || t == 'n'; }
bool is_t(char t) { return t == 'T' || t == 't'; }
bool aligned(const void *p, size_t bytes) { return reinterpret_cast<uintptr_t>(p) % bytes == 0; }

// Column-major GEMM shared by FP32/FP64 (ref: backend.cu:786-866): validation order, no-op and
// beta-only cases, alias rejection, then the planner's choice.
template <typename T, typename Scale, typename Launch>
int gemm(camblas_cuda_context *context, const char *type_name, char trans_a, char trans_b, int m,
         int n, int k, T alpha, const T *a, int lda, const T *b, int ldb, T beta, T *c, int ldc,
         Scale scale, Launch launch)
{
    (void)type_name;
    bool na = is_n(trans_a), ta = is_t(trans_a), nb = is_n(trans_b), tb = is_t(trans_b);
    if ((!na && !ta) || (!nb && !tb) || m < 0 || n < 0 || k < 0 || lda < 1 || ldb < 1 || ldc < 1)
        return fail(context, "invalid GEMM arguments", 1);
    if (m == 0 || n == 0)
        return 0;
    if (!c || lda < std::max(1, na ? m : k) || ldb < std::max(1, nb ? k : n) || ldc < m)
        return fail(context, "invalid device pointer or leading dimension", 1);
    if (alpha == T(0) || k == 0) {
        if (beta == T(1))
            return 0;
        hipError_t error = scale();
        return error == hipSuccess ? 0 : fail(context, "scale output", error);
    }
    if (!a || !b || a == c || b == c)
        return fail(context, "missing or aliased GEMM operand", 1);
    return launch(ta, tb);
}
} // namespace
} // namespace camblas_hip

using namespace camblas_hip;

extern "C" int camblas_cuda_create(int device, void *stream, camblas_cuda_context **out)
{
    if (!out)
        return fail(nullptr, "missing context output", 1);
    *out = nullptr;
    DeviceScope scope(device);
    if (scope.status != hipSuccess)
        return fail(nullptr, "activate device", scope.status);
    auto *context = new (std::nothrow) camblas_cuda_context;
    if (!context)
        return fail(nullptr, "context allocation", 2);
    context->device = device;
    context->stream = static_cast<hipStream_t>(stream);
    hipDeviceProp_t properties;
    hipError_t status = hipGetDeviceProperties(&properties, device);
    if (status != hipSuccess) {
        delete context;
        return fail(nullptr, "device properties", status);
    }
    if (std::strncmp(properties.gcnArchName, "gfx950", 6) != 0) {
        delete context;
        std::snprintf(creation_error, sizeof(creation_error),
                      "libcamblas_hip is built for gfx950 only; device %d is %s", device,
                      properties.gcnArchName);
        return -1;
    }
    context->compute_units = properties.multiProcessorCount;
    // the allocation-free attention entry point's fixed array: find this device's copy now, so
    // that the entry point itself never has to ask the runtime
    void *resident = nullptr;
    status = gqa_resident_scratch(device, &resident);
    if (status != hipSuccess) {
        delete context;
        return fail(nullptr, "resident scratch address", status);
    }
    *out = context;
    return 0;
}

extern "C" int camblas_cuda_destroy(camblas_cuda_context *context)
{
    if (!context)
        return 0;
    DeviceScope scope(context->device);
    if (scope.status != hipSuccess)
        return fail(context, "activate device for destruction", scope.status);
    hipError_t error = hipStreamSynchronize(context->stream);
    if (context->scratch)
        (void)hipFree(context->scratch);
    for (void *allocation : context->retired)
        (void)hipFree(allocation);
    delete context;
    return error == hipSuccess ? 0 : fail(nullptr, "stream completion during destruction", error);
}

extern "C" const char *camblas_cuda_error(const camblas_cuda_context *context)
{
    return context ? context->error : creation_error;
}

extern "C" int camblas_cuda_set_algorithm(camblas_cuda_context *context, int algorithm)
{
    if (!context || algorithm < CAMBLAS_CUDA_AUTO || algorithm > CAMBLAS_CUDA_STRASSEN_FOUR)
        return fail(context, "invalid algorithm", 1);
    context->algorithm = algorithm;
    return 0;
}

namespace camblas_hip
{
namespace
{
// Depth of the Strassen recursion for this product under the context's policy, 0 for none: square
// untransposed products of even size from 256 under an explicit Strassen policy, from 8192 under
// the default one (ref: src/cuda/backend.cu:843-853).
int square_strassen_levels(const camblas_cuda_context *context, bool trans_a, bool trans_b, int m, int n, int k)
{
    if (trans_a || trans_b || m != n || n != k || n % 2 != 0 || n < 256)
        return 0;
    return strassen_levels(context->algorithm, n);
}

// The symmetric policy applies to a product of a matrix with its own transpose that overwrites C
// (ref: src/cuda/backend.cu:819-835): only the tiles on and below the diagonal are computed, the
// upper triangle is a copy of the lower one, so C is symmetric bit for bit.
bool symmetric_gram(const camblas_cuda_context *context, bool trans_a, bool trans_b, int m, int n,
                    const void *a, int lda, const void *b, int ldb, bool overwrite)
{
    return context->algorithm == CAMBLAS_CUDA_SYMMETRIC && a == b && trans_a != trans_b && m == n &&
           lda == ldb && overwrite;
}

// Tile width of the FP32 lower-triangle product: 128 x 128 once the tiles that reach the diagonal
// number two per compute unit, else 128 x 64 (the rule of the full product)
bool gram_prefers_wide_tiles(int n, int compute_units)
{
    const double rows = (n + 127) / 128;
    return rows * (rows + 1) / 2 >= 2.0 * compute_units;
}

// FP32 / FP64 column-major GEMM on the context's stream, without the device scope: shared by the
// public entry points and by the dense helpers below.
int dense_gemm(camblas_cuda_context *context, char ta, char tb, int m, int n, int k, float alpha,
               const float *a, int lda, const float *b, int ldb, float beta, float *c, int ldc)
{
    return gemm<float>(
        context, "FP32", ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc,
        [&] { return launch_scale_f32(context->stream, m, n, beta, c, ldc); },
        [&](bool trans_a, bool trans_b) {
            if (symmetric_gram(context, trans_a, trans_b, m, n, a, lda, b, ldb, beta == 0.f)) {
                context->counts[2]++;
                hipError_t error =
                    m >= 32 && k >= 16
                        ? launch_sgemm_mfma(context->stream, gram_prefers_wide_tiles(m, context->compute_units),
                                            trans_a, trans_b, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, 1, 0, true)
                        : launch_generic_f32(context->stream, trans_a, trans_b, m, n, k, alpha, a, lda, b, ldb,
                                             beta, c, ldc);
                if (error != hipSuccess)
                    return fail(context, "symmetric Gram", error);
                error = launch_mirror_lower(context->stream, 0, n, c, ldc);
                return error == hipSuccess ? 0 : fail(context, "Gram mirroring", error);
            }
            if (int levels = square_strassen_levels(context, trans_a, trans_b, m, n, k)) {
                const int outcome = strassen_gemm(context, levels, n, alpha, a, lda, b, ldb, beta, c, ldc);
                if (outcome != STRASSEN_FALL_BACK && outcome != STRASSEN_NOT_ELIGIBLE)
                    return outcome;
            }
            Plan plan = make_plan(0, context->algorithm, trans_a, trans_b, m, n, k, lda, ldb, ldc,
                                  aligned(a, 16) && aligned(b, 16), context->compute_units);
            context->counts[plan.counter]++;
            hipError_t error;
            if (plan.family == FAMILY_GEMV_F32) {
                error = launch_gemv_f32(context->stream, m, k, alpha, a, lda, b, beta, c);
                return error == hipSuccess ? 0 : fail(context, "FP32 native GEMV", error);
            }
            if (context->override_kernel >= 0) { // diagnostics: 0 vector-ALU tiles, 1 / 2 matrix-core tiles
                plan.family = context->override_kernel >= 1 ? FAMILY_MFMA_F32 : FAMILY_GENERIC;
                plan.kernel = context->override_kernel == 2 ? 1 : 0;
            }
            if (plan.family == FAMILY_MFMA_F32)
                error = launch_sgemm_mfma(context->stream, plan.kernel == 0, trans_a, trans_b, m, n, k,
                                          alpha, a, lda, b, ldb, beta, c, ldc);
            else
                error = launch_generic_f32(context->stream, trans_a, trans_b, m, n, k, alpha, a, lda,
                                           b, ldb, beta, c, ldc);
            return error == hipSuccess ? 0 : fail(context, "classical GEMM", error);
        });
}

// ref: src/cuda/backend.cu:1066-1073; products with at least one 16 x 16 x 4 matrix-core tile in
// every dimension run on the matrix cores, smaller ones on the LDS-tiled FMA kernel
int dense_gemm(camblas_cuda_context *context, char ta, char tb, int m, int n, int k, double alpha,
               const double *a, int lda, const double *b, int ldb, double beta, double *c, int ldc)
{
    return gemm<double>(
        context, "FP64", ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc,
        [&] { return launch_scale_f64(context->stream, m, n, beta, c, ldc); },
        [&](bool trans_a, bool trans_b) {
            if (symmetric_gram(context, trans_a, trans_b, m, n, a, lda, b, ldb, beta == 0.0)) {
                context->counts[2]++;
                hipError_t error =
                    m >= 16 && k >= 4
                        ? launch_dgemm_mfma(context->stream, trans_a, trans_b, m, n, k, alpha, a, lda, b, ldb, beta,
                                            c, ldc, 1, 0, true)
                        : launch_generic_f64(context->stream, trans_a, trans_b, m, n, k, alpha, a, lda, b, ldb,
                                             beta, c, ldc);
                if (error != hipSuccess)
                    return fail(context, "symmetric Gram", error);
                error = launch_mirror_lower(context->stream, 1, n, c, ldc);
                return error == hipSuccess ? 0 : fail(context, "Gram mirroring", error);
            }
            if (int levels = square_strassen_levels(context, trans_a, trans_b, m, n, k)) {
                const int outcome = strassen_gemm(context, levels, n, alpha, a, lda, b, ldb, beta, c, ldc);
                if (outcome != STRASSEN_FALL_BACK && outcome != STRASSEN_NOT_ELIGIBLE)
                    return outcome;
            }
            context->counts[0]++;
            bool matrix = m >= 16 && n >= 16 && k >= 4;
            if (context->override_kernel >= 0) // diagnostics: 0 vector-ALU tiles, else matrix-core tiles
                matrix = context->override_kernel >= 1;
            hipError_t error =
                matrix ? launch_dgemm_mfma(context->stream, trans_a, trans_b, m, n, k, alpha, a, lda, b,
                                           ldb, beta, c, ldc)
                       : launch_generic_f64(context->stream, trans_a, trans_b, m, n, k, alpha, a, lda,
                                            b, ldb, beta, c, ldc);
            return error == hipSuccess ? 0 : fail(context, "classical FP64 GEMM", error);
        });
}

// Row-major out[rows, columns] = x[rows, inner] . weight[inner, columns] + bias, optional ReLU
// (ref: src/cuda/backend.cu:871-905): as a column-major product out^T = weight^T-view . x^T-view,
// then one bias/activation pass.
template <typename T>
int affine(camblas_cuda_context *context, int rows, int inner, int columns, const T *x, const T *weight,
           const T *bias, bool relu, T *output)
{
    if (rows < 0 || inner < 0 || columns < 0)
        return fail(context, "invalid affine dimensions", 1);
    if (rows == 0 || columns == 0)
        return 0;
    if (!output || !bias || (inner > 0 && (!x || !weight)))
        return fail(context, "missing affine operand", 1);
    context->counts[3]++;
    int result = dense_gemm(context, 'N', 'N', columns, rows, inner, T(1), weight, std::max(1, columns),
                            x, std::max(1, inner), T(0), output, columns);
    if (result != 0)
        return result;
    hipError_t error = launch_bias_activation(context->stream, sizeof(T) == 4 ? 0 : 1, output, bias,
                                              size_t(rows) * columns, columns, relu);
    return error == hipSuccess ? 0 : fail(context, "bias/activation", error);
}

// softmax(scale . q k^T) v with the scores in context scratch (ref: src/cuda/fusion.cuh:95-157).
template <typename T>
int dense_attention(camblas_cuda_context *context, int queries, int keys, int depth, int values, T scale,
                    const T *q, const T *k, const T *v, T *output)
{
    if (queries < 0 || keys < 0 || depth < 0 || values < 0)
        return fail(context, "invalid attention dimensions", 1);
    if (queries == 0 || values == 0)
        return 0;
    if (!output || (depth > 0 && !q) || (keys > 0 && depth > 0 && !k) || (keys > 0 && !v))
        return fail(context, "missing attention operand", 1);
    if (keys > 0 && size_t(queries) > std::numeric_limits<size_t>::max() / sizeof(T) / size_t(keys))
        return fail(context, "attention scratch size overflow", 2);
    context->counts[6]++;
    hipError_t error = reserve_scratch(context, size_t(queries) * keys * sizeof(T));
    if (error != hipSuccess)
        return fail(context, "attention scratch", error);
    T *scores = static_cast<T *>(context->scratch);
    // scores[queries, keys] = q k^T (keys == 0: nothing to do; the product below then zeroes out)
    int result = dense_gemm(context, 'T', 'N', keys, queries, depth, T(1), k, std::max(1, depth), q,
                            std::max(1, depth), T(0), scores, std::max(1, keys));
    if (result != 0)
        return result;
    error = launch_softmax_rows(context->stream, sizeof(T) == 4 ? 0 : 1, scores, queries, keys,
                                double(scale));
    if (error != hipSuccess)
        return fail(context, "attention softmax", error);
    return dense_gemm(context, 'N', 'N', values, queries, keys, T(1), v, std::max(1, values), scores,
                      std::max(1, keys), T(0), output, std::max(1, values));
}

// Gradients of output = relu(x w1 + b1) w2 + b2 (ref: src/cuda/fusion.cuh:207-275). Null gradient
// pointers are skipped; grad_hidden is scratch of the caller, left holding the masked gradient.
template <typename T>
int mlp_backward(camblas_cuda_context *context, int rows, int inputs, int hidden, int outputs, const T *x,
                 const T *w1, const T *w2, const T *h, const T *grad, T *dh, T *dx, T *dw1, T *db1,
                 T *dw2, T *db2)
{
    if (rows < 0 || inputs < 0 || hidden < 0 || outputs < 0)
        return fail(context, "invalid backward dimensions", 1);
    const bool first_layer = dx || dw1 || db1;
    if ((rows > 0 && outputs > 0 && !grad) || (rows > 0 && hidden > 0 && first_layer && (!dh || !h)))
        return fail(context, "missing backward operand", 1);
    context->counts[7]++;
    const int dtype = sizeof(T) == 4 ? 0 : 1;
    // column sums run over chunks of 128 rows; more than one chunk goes through context scratch
    const int chunks = int(std::min<size_t>(65535, std::max<size_t>(1, (size_t(rows) + 127) / 128)));
    const int chunk_rows = std::max(1, int((int64_t(rows) + chunks - 1) / chunks));
    T *partial = nullptr;
    if (chunks > 1 && ((db2 && outputs > 0) || (db1 && hidden > 0))) {
        hipError_t error =
            reserve_scratch(context, size_t(chunks) * std::max(hidden, outputs) * sizeof(T));
        if (error != hipSuccess)
            return fail(context, "backward scratch", error);
        partial = static_cast<T *>(context->scratch);
    }
    int result = 0;
    if (dw2) { // dw2[hidden, outputs] = h^T grad
        result = dense_gemm(context, 'N', 'T', outputs, hidden, rows, T(1), grad, std::max(1, outputs), h,
                            std::max(1, hidden), T(0), dw2, std::max(1, outputs));
        if (result != 0)
            return result;
    }
    if (db2 && outputs > 0) {
        hipError_t error = launch_column_sums(context->stream, dtype, false, const_cast<T *>(grad),
                                              nullptr, rows, outputs, chunks, chunk_rows, partial, db2);
        if (error != hipSuccess)
            return fail(context, "backward bias", error);
    }
    if (!first_layer)
        return 0;
    // dh[rows, hidden] = grad w2^T, masked by the ReLU (h > 0), summed over rows for db1
    result = dense_gemm(context, 'T', 'N', hidden, rows, outputs, T(1), w2, std::max(1, outputs), grad,
                        std::max(1, outputs), T(0), dh, std::max(1, hidden));
    if (result != 0)
        return result;
    if (hidden > 0) {
        hipError_t error = launch_column_sums(context->stream, dtype, true, dh, h, rows, hidden, chunks,
                                              chunk_rows, db1 ? partial : nullptr, db1);
        if (error != hipSuccess)
            return fail(context, "backward activation", error);
    }
    if (dw1) { // dw1[inputs, hidden] = x^T dh
        result = dense_gemm(context, 'N', 'T', hidden, inputs, rows, T(1), dh, std::max(1, hidden), x,
                            std::max(1, inputs), T(0), dw1, std::max(1, hidden));
        if (result != 0)
            return result;
    }
    if (dx) // dx[rows, inputs] = dh w1^T
        result = dense_gemm(context, 'T', 'N', inputs, rows, hidden, T(1), w1, std::max(1, hidden), dh,
                            std::max(1, hidden), T(0), dx, std::max(1, inputs));
    return result;
}
} // namespace
} // namespace camblas_hip

extern "C" int camblas_cuda_sgemm(camblas_cuda_context *context, char ta, char tb, int m, int n,
                                  int k, float alpha, const float *a, int lda, const float *b,
                                  int ldb, float beta, float *c, int ldc)
{
    return execute(context, [&] {
        return dense_gemm(context, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
    });
}

extern "C" int camblas_cuda_dgemm(camblas_cuda_context *context, char ta, char tb, int m, int n,
                                  int k, double alpha, const double *a, int lda, const double *b,
                                  int ldb, double beta, double *c, int ldc)
{
    return execute(context, [&] {
        return dense_gemm(context, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
    });
}

extern "C" int camblas_cuda_bgemm(camblas_cuda_context *context, char trans_a, char trans_b, int m,
                                  int n, int k, float alpha, const void *a, int lda, const void *b,
                                  int ldb, float beta, void *c, int ldc)
{
    // ref: src/cuda/bfloat16.cuh:11-57
    return execute(context, [&] {
        bool na = is_n(trans_a), ta = is_t(trans_a), nb = is_n(trans_b), tb = is_t(trans_b);
        if ((!na && !ta) || (!nb && !tb) || m < 0 || n < 0 || k < 0 || lda < 1 || ldb < 1 ||
            ldc < 1)
            return fail(context, "invalid BF16 GEMM arguments", 1);
        if (m == 0 || n == 0)
            return 0;
        if (!c || lda < std::max(1, na ? m : k) || ldb < std::max(1, nb ? k : n) || ldc < m)
            return fail(context, "invalid BF16 pointer or leading dimension", 1);
        if (alpha == 0 || k == 0) {
            if (beta == 1)
                return 0;
            hipError_t error = launch_scale_bf16(context->stream, m, n, beta, c, ldc);
            return error == hipSuccess ? 0 : fail(context, "scale BF16 output", error);
        }
        if (!a || !b || a == c || b == c)
            return fail(context, "missing or aliased BF16 GEMM operand", 1);
        Plan plan = make_plan(2, context->algorithm, ta, tb, m, n, k, lda, ldb, ldc,
                              aligned(a, 16) && aligned(b, 16), context->compute_units);
        if (plan.family == FAMILY_DMA && !aligned(c, 8))
            plan.family = FAMILY_MFMA_TN; // same tile shapes, register-staged loads, scalar stores
        if ((plan.family == FAMILY_MFMA_TN || plan.family == FAMILY_STREAM ||
             plan.family == FAMILY_DMA) &&
            context->override_kernel >= 0) {
            // diagnostics: 0.. selects an MFMA tile variant, 100 + 10*row_tiles + token_tiles the
            // streaming kernel (+ 100*mode)
            if (context->override_kernel >= 100) {
                plan.family = FAMILY_STREAM;
                plan.kernel = context->override_kernel - 100;
                plan.split_k = 1;
            } else if (context->override_kernel >= 20 && context->override_kernel < 60) {
                plan.family = FAMILY_DMA; // 20..59: direct-to-LDS tile variants
                plan.kernel = context->override_kernel - 20;
                plan.split_k = 1;
            } else {
                plan.family = FAMILY_MFMA_TN;
                plan.kernel = context->override_kernel;
                plan.split_k = context->override_split > 0 ? context->override_split : 1;
            }
        }
        if (plan.family == FAMILY_DMA) {
            context->counts[plan.counter]++;
            hipError_t error = launch_bgemm_dma(context->stream, plan.kernel, m, n, k, alpha, a, lda,
                                                b, ldb, beta, c, ldc);
            return error == hipSuccess ? 0 : fail(context, "BF16 MFMA GEMM (direct LDS loads)", error);
        }
        if (plan.family == FAMILY_STREAM) {
            context->counts[plan.counter]++;
            hipError_t error =
                launch_bgemv_stream(context->stream, plan.kernel / 100, plan.kernel / 10 % 10,
                                    plan.kernel % 10, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
            return error == hipSuccess ? 0 : fail(context, "BF16 streaming GEMV", error);
        }
        if (plan.family == FAMILY_MFMA_TN) {
            float *partials = nullptr;
            if (plan.split_k > 1) {
                hipError_t grown =
                    reserve_scratch(context, size_t(plan.split_k) * size_t(m) * size_t(n) * 4);
                if (grown != hipSuccess) {
                    // cannot hold the partials (allocation failure or capture in progress):
                    // run unsplit, and if even that is impossible use the generic kernel
                    context->counts[5]++;
                    plan.split_k = 1;
                } else {
                    partials = static_cast<float *>(context->scratch);
                }
            }
            context->counts[plan.counter]++;
            hipError_t error = launch_bgemm_tn(context->stream, plan.kernel, plan.split_k, m, n, k,
                                               alpha, a, lda, b, ldb, beta, c, ldc, partials);
            return error == hipSuccess ? 0 : fail(context, "BF16 MFMA GEMM", error);
        }
        context->counts[0]++;
        hipError_t error = launch_generic_bf16(context->stream, ta, tb, m, n, k, alpha, a, lda, b,
                                               ldb, beta, c, ldc);
        return error == hipSuccess ? 0 : fail(context, "BF16 GEMM", error);
    });
}

extern "C" int camblas_cuda_affine(camblas_cuda_context *context, int dtype, int rows, int inner,
                                   int columns, const void *x, const void *weight, const void *bias,
                                   int relu, void *output)
{
    // ref: src/cuda/backend.cu:1086-1101
    return execute(context, [&] {
        if (dtype == 0)
            return affine(context, rows, inner, columns, static_cast<const float *>(x),
                          static_cast<const float *>(weight), static_cast<const float *>(bias),
                          relu != 0, static_cast<float *>(output));
        if (dtype == 1)
            return affine(context, rows, inner, columns, static_cast<const double *>(x),
                          static_cast<const double *>(weight), static_cast<const double *>(bias),
                          relu != 0, static_cast<double *>(output));
        return fail(context, "unsupported affine dtype", 1);
    });
}

extern "C" int camblas_cuda_mlp(camblas_cuda_context *context, int dtype, int rows, int inputs,
                                int hidden, int outputs, const void *x, const void *w1,
                                const void *b1, const void *w2, const void *b2, void *hidden_output,
                                void *output)
{
    // ref: src/cuda/backend.cu:1103-1117 — two affine layers, the first with ReLU; the hidden
    // activations are an output of their own and may not share storage with the result
    if (rows < 0 || inputs < 0 || hidden < 0 || outputs < 0 ||
        (rows > 0 && hidden > 0 && hidden_output == output))
        return fail(context, "invalid MLP dimensions or aliased outputs", 1);
    int result =
        camblas_cuda_affine(context, dtype, rows, inputs, hidden, x, w1, b1, 1, hidden_output);
    if (result != 0)
        return result;
    return camblas_cuda_affine(context, dtype, rows, hidden, outputs, hidden_output, w2, b2, 0, output);
}

extern "C" int camblas_cuda_attention(camblas_cuda_context *context, int dtype, int queries, int keys,
                                      int depth, int values, double scale, const void *q,
                                      const void *k, const void *v, void *output)
{
    // ref: src/cuda/backend.cu:1495-1510
    return execute(context, [&] {
        if (dtype == 0)
            return dense_attention(context, queries, keys, depth, values, float(scale),
                                   static_cast<const float *>(q), static_cast<const float *>(k),
                                   static_cast<const float *>(v), static_cast<float *>(output));
        if (dtype == 1)
            return dense_attention(context, queries, keys, depth, values, scale,
                                   static_cast<const double *>(q), static_cast<const double *>(k),
                                   static_cast<const double *>(v), static_cast<double *>(output));
        return fail(context, "unsupported attention dtype", 1);
    });
}

extern "C" int camblas_cuda_mlp_backward(camblas_cuda_context *context, int dtype, int rows,
                                         int inputs, int hidden, int outputs, const void *x,
                                         const void *w1, const void *w2, const void *hidden_output,
                                         const void *grad_output, void *grad_hidden, void *dx,
                                         void *dw1, void *db1, void *dw2, void *db2)
{
    // ref: src/cuda/backend.cu:1512-1535
    return execute(context, [&] {
        if (dtype == 0)
            return mlp_backward(context, rows, inputs, hidden, outputs, static_cast<const float *>(x),
                                static_cast<const float *>(w1), static_cast<const float *>(w2),
                                static_cast<const float *>(hidden_output),
                                static_cast<const float *>(grad_output),
                                static_cast<float *>(grad_hidden), static_cast<float *>(dx),
                                static_cast<float *>(dw1), static_cast<float *>(db1),
                                static_cast<float *>(dw2), static_cast<float *>(db2));
        if (dtype == 1)
            return mlp_backward(context, rows, inputs, hidden, outputs, static_cast<const double *>(x),
                                static_cast<const double *>(w1), static_cast<const double *>(w2),
                                static_cast<const double *>(hidden_output),
                                static_cast<const double *>(grad_output),
                                static_cast<double *>(grad_hidden), static_cast<double *>(dx),
                                static_cast<double *>(dw1), static_cast<double *>(db1),
                                static_cast<double *>(dw2), static_cast<double *>(db2));
        return fail(context, "unsupported backward dtype", 1);
    });
}

extern "C" int camblas_cuda_silu_multiply(camblas_cuda_context *context, int dtype, uint64_t count,
                                          const void *gate, const void *up, void *output)
{
    // ref: backend.cu:1119-1133
    return execute(context, [&] {
        if (dtype != 0 && dtype != 2)
            return fail(context, "unsupported SiLU dtype", 1);
        if (!count)
            return 0;
        if (!gate || !up || !output || count > SIZE_MAX / (dtype == 0 ? 4 : 2))
            return fail(context, "invalid SiLU operands or length", 1);
        hipError_t error = launch_silu_multiply(context->stream, dtype, count, gate, up, output);
        return error == hipSuccess ? 0 : fail(context, "SiLU multiply", error);
    });
}

extern "C" int camblas_cuda_swiglu(camblas_cuda_context *context, int dtype, uint64_t count,
                                   int width, float limit, const void *gate, const void *up,
                                   const float *routing, void *output)
{
    // ref: backend.cu:1135-1163
    return execute(context, [&] {
        if ((dtype != 0 && dtype != 2) || width <= 0 || count % unsigned(width) ||
            !std::isfinite(limit) || limit < 0 || count > SIZE_MAX / (dtype == 0 ? 4 : 2))
            return fail(context, "invalid SwiGLU dimensions or clipping limit", 1);
        if (!count)
            return 0;
        unsigned alignment = dtype == 0 ? 4 : 2;
        if (!gate || !up || !output || !aligned(gate, alignment) || !aligned(up, alignment) ||
            !aligned(output, alignment) || (routing && (!aligned(routing, 4) || output == routing)))
            return fail(context, "invalid SwiGLU buffers", 1);
        hipError_t error =
            launch_swiglu(context->stream, dtype, count, width, limit, gate, up, routing, output);
        return error == hipSuccess ? 0 : fail(context, "SwiGLU", error);
    });
}

extern "C" int camblas_cuda_rms_norm_decode(camblas_cuda_context *context, int dtype,
                                            int weight_dtype, int width, float epsilon,
                                            int round_before_weight, int descending,
                                            const void *input, const void *weight, void *output)
{
    // ref: backend.cu:1363-1396
    return execute(context, [&] {
        if ((dtype != 0 && dtype != 2) || (weight_dtype != 0 && weight_dtype != 2) ||
            (dtype == 0 && weight_dtype != 0) || width < 2048 || width > 65536 || width % 4 ||
            (round_before_weight != 0 && round_before_weight != 1) ||
            (descending != 0 && descending != 1) || !std::isfinite(epsilon) || epsilon < 0 ||
            !input || !weight || !output || output == input || output == weight ||
            !aligned(input, dtype == 0 ? 4 : 2) || !aligned(weight, weight_dtype == 0 ? 4 : 2) ||
            !aligned(output, dtype == 0 ? 4 : 2))
            return fail(context, "invalid decode RMS arguments", 1);
        hipError_t error =
            launch_rms_rows(context->stream, dtype, weight_dtype, 1, width, epsilon,
                            round_before_weight != 0, input, nullptr, weight, nullptr, output);
        return error == hipSuccess ? 0 : fail(context, "decode RMS normalisation", error);
    });
}

extern "C" int camblas_cuda_add_rms_norm(camblas_cuda_context *context, int dtype, int width,
                                         float epsilon, const void *input, const void *residual,
                                         const void *weight, void *added, void *output)
{
    // ref: backend.cu:1398-1421
    return execute(context, [&] {
        if ((dtype != 0 && dtype != 2) || width < 2048 || width > 65536 || width % 4 ||
            !std::isfinite(epsilon) || epsilon < 0 || !input || !residual || !weight || !added ||
            !output || added == output || added == input || added == residual || added == weight ||
            output == input || output == residual || output == weight)
            return fail(context, "invalid residual RMS arguments", 1);
        hipError_t error = launch_rms_rows(context->stream, dtype, dtype, 1, width, epsilon, true,
                                           input, residual, weight, added, output);
        return error == hipSuccess ? 0 : fail(context, "residual RMS normalisation", error);
    });
}

extern "C" int camblas_cuda_add_rms_norm_rows(camblas_cuda_context *context, int dtype,
                                              int weight_dtype, int rows, int width, float epsilon,
                                              int round_before_weight, const void *input,
                                              const void *residual, const void *weight, void *added,
                                              void *output)
{
    return execute(context, [&] {
        if ((dtype != 0 && dtype != 2) || (weight_dtype != 0 && weight_dtype != 2) ||
            (dtype == 0 && weight_dtype != 0) || rows < 0 || width < 0 ||
            (round_before_weight != 0 && round_before_weight != 1) || !std::isfinite(epsilon) ||
            epsilon < 0)
            return fail(context, "invalid residual RMS rows arguments", 1);
        if (!rows || !width)
            return 0;
        if (!input || !weight || !output || output == weight || output == input ||
            (residual && (!added || added == output || added == input || added == residual ||
                          added == weight || output == residual)))
            return fail(context, "invalid residual RMS rows operands", 1);
        hipError_t error =
            launch_rms_rows(context->stream, dtype, weight_dtype, rows, width, epsilon,
                            round_before_weight != 0, input, residual, weight, added, output);
        return error == hipSuccess ? 0 : fail(context, "residual RMS normalisation", error);
    });
}

extern "C" int camblas_cuda_rms_norm(camblas_cuda_context *context, int dtype, int rows, int width,
                                     float epsilon, const void *input, const void *weight,
                                     void *output)
{
    // ref: backend.cu:1423-1439. In-place output==input is allowed there; each element is read
    // before it is written by the same thread here as well.
    return execute(context, [&] {
        if ((dtype != 0 && dtype != 2) || rows < 0 || width < 0 || !std::isfinite(epsilon) ||
            epsilon < 0)
            return fail(context, "invalid RMS normalisation dimensions, dtype or epsilon", 1);
        if (!rows || !width)
            return 0;
        if (!input || !weight || !output || output == weight)
            return fail(context, "invalid RMS normalisation operands", 1);
        hipError_t error = launch_rms_rows(context->stream, dtype, dtype, rows, width, epsilon, true,
                                           input, nullptr, weight, nullptr, output);
        return error == hipSuccess ? 0 : fail(context, "RMS normalisation", error);
    });
}

extern "C" int camblas_cuda_bfloat16_square(camblas_cuda_context *context, uint64_t count,
                                            const void *input, float *output)
{
    return execute(context, [&] {
        if (!count)
            return 0;
        if (!input || !output || count > SIZE_MAX / sizeof(float))
            return fail(context, "invalid BF16 square operands", 1);
        hipError_t error = launch_bf16_square(context->stream, count, input, output);
        return error == hipSuccess ? 0 : fail(context, "BF16 squares", error);
    });
}

extern "C" int camblas_cuda_rms_scale(camblas_cuda_context *context, int dtype, uint64_t count,
                                      int width, float epsilon, const void *input,
                                      const void *weight, const float *means, void *output)
{
    // ref: backend.cu:1457-1475
    return execute(context, [&] {
        if ((dtype != 0 && dtype != 2) || width < 0 || !std::isfinite(epsilon) || epsilon < 0)
            return fail(context, "invalid RMS scale dimensions, dtype or epsilon", 1);
        if (!count)
            return 0;
        if (!width || count % width || count > SIZE_MAX / sizeof(float) || !input || !weight ||
            !means || !output || output == weight)
            return fail(context, "invalid RMS scale operands", 1);
        hipError_t error = launch_rms_scale(context->stream, dtype, count, width, epsilon, input,
                                            weight, means, output);
        return error == hipSuccess ? 0 : fail(context, "RMS scaling", error);
    });
}

extern "C" int camblas_cuda_stats(const camblas_cuda_context *context, uint64_t *counts, int length)
{
    if (!context || !counts || (length != 6 && length != 8))
        return fail(nullptr, "invalid stats output", 1);
    for (int i = 0; i < length; ++i)
        counts[i] = context->counts[i].load(std::memory_order_relaxed);
    return 0;
}

extern "C" int camblas_cuda_reset_stats(camblas_cuda_context *context)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    for (auto &count : context->counts)
        count.store(0, std::memory_order_relaxed);
    return 0;
}

// ------------------------------------------------------------------ extensions

extern "C" int camblas_cuda_fp8_block_matmul(camblas_cuda_context *context, int rows, int outputs,
                                             int inner, const void *a, const float *a_scale,
                                             const void *w, const float *w_scale, void *out)
{
    return execute(context, [&] {
        if (rows < 0 || rows > 65535 || outputs < 1 || inner < 128 || inner % 128)
            return fail(context, "invalid FP8 block matrix dimensions", 1);
        if (!rows)
            return 0;
        if (!a || !a_scale || !w || !w_scale || !out || !aligned(a, 16) || !aligned(w, 16) ||
            !aligned(a_scale, 4) || !aligned(w_scale, 4) || !aligned(out, 2) || out == a ||
            out == w || out == (const void *)a_scale || out == (const void *)w_scale)
            return fail(context, "invalid FP8 block matrix buffers", 1);
        Plan plan = make_plan(3, context->algorithm, true, false, outputs, rows, inner, inner, inner,
                              outputs, true, context->compute_units);
        if (plan.family == FAMILY_FP8_DMA && !aligned(out, 8))
            plan = Plan{FAMILY_FP8_BLOCK, 0, 1, 4};
        if (context->override_kernel >= 0) {
            // diagnostics: 0.. register-staged variants (with split-K), 20.. direct-to-LDS variants,
            // 100 + 10*row_tiles + token_tiles the streaming kernel
            if (context->override_kernel >= 100) {
                plan.family = FAMILY_FP8_STREAM;
                plan.kernel = context->override_kernel - 100;
                plan.split_k = 1;
            } else if (context->override_kernel >= 20) {
                plan.family = FAMILY_FP8_DMA;
                plan.kernel = context->override_kernel - 20;
                plan.split_k = 1;
            } else {
                plan.family = FAMILY_FP8_BLOCK;
                plan.kernel = context->override_kernel;
                plan.split_k = context->override_split > 0 ? context->override_split : 1;
            }
        }
        if (plan.family == FAMILY_FP8_STREAM) {
            context->counts[plan.counter]++;
            hipError_t error = launch_fp8_stream(context->stream, plan.kernel / 10, plan.kernel % 10,
                                                 rows, outputs, inner, a, a_scale, w, w_scale, out);
            return error == hipSuccess ? 0 : fail(context, "FP8 block-scaled streaming GEMV", error);
        }
        if (plan.family == FAMILY_FP8_DMA) {
            context->counts[plan.counter]++;
            hipError_t error = launch_fp8_dma(context->stream, plan.kernel, rows, outputs, inner, a,
                                              a_scale, w, w_scale, out);
            return error == hipSuccess ? 0
                                       : fail(context, "FP8 block-scaled GEMM (direct LDS loads)", error);
        }
        float *partials = nullptr;
        if (plan.split_k > 1) {
            hipError_t grown = reserve_scratch(
                context, size_t(plan.split_k) * size_t(rows) * size_t(outputs) * 4);
            if (grown != hipSuccess) {
                context->counts[5]++;
                plan.split_k = 1;
            } else {
                partials = static_cast<float *>(context->scratch);
            }
        }
        context->counts[plan.counter]++;
        hipError_t error = launch_fp8_block(context->stream, plan.kernel, plan.split_k, rows,
                                            outputs, inner, a, a_scale, w, w_scale, out, partials);
        return error == hipSuccess ? 0 : fail(context, "FP8 block-scaled GEMM", error);
    });
}

// ref: src/cuda/backend.cu:1165-1191
extern "C" int camblas_cuda_quantized_matmul(camblas_cuda_context *context, int packed, int rows,
                                             int outputs, int inner, int activation_block,
                                             const void *input, const void *input_scale,
                                             const void *weight, const void *weight_scale,
                                             void *output)
{
    return execute(context, [&] {
        if ((packed != 0 && packed != 1) || rows < 0 || rows > 65535 || outputs < 8 ||
            outputs % 8 || inner < 32 || inner % 32 ||
            (activation_block != 32 && activation_block != 128) || inner % activation_block ||
            (!packed && activation_block != 32))
            return fail(context, "invalid quantized matrix dimensions", 1);
        if (!rows)
            return 0;
        if (!input || !input_scale || !weight || !weight_scale || !output || !aligned(input, 16) ||
            !aligned(weight, 16) || !aligned(output, 2) || output == input ||
            output == input_scale || output == weight || output == weight_scale)
            return fail(context, "invalid quantized matrix buffers", 1);
        context->counts[4]++;
        hipError_t error = launch_mx_matmul(context->stream, context->override_kernel,
                                            context->compute_units, packed != 0, 0, 0, rows,
                                            outputs, inner, activation_block, input, input_scale,
                                            weight, weight_scale, nullptr, nullptr, nullptr, output);
        return error == hipSuccess ? 0 : fail(context, "quantized matrix multiplication", error);
    });
}

// ref: src/cuda/backend.cu:1258-1303. The kernel writes the zeros of inactive groups and padding
// rows itself, so no memset node is needed (the call can be captured in a graph).
extern "C" int camblas_cuda_grouped_quantized_matmul(camblas_cuda_context *context, int packed,
                                                     int groups, int weight_groups, int rows,
                                                     int outputs, int inner, int activation_block,
                                                     const void *input, const void *input_scale,
                                                     const void *metadata, const void *active,
                                                     const void *counts, void *output)
{
    return execute(context, [&] {
        if ((packed != 0 && packed != 1) || groups < 0 || groups > 65535 || weight_groups < 1 ||
            weight_groups > 65535 || rows < 0 || rows > 65535 || outputs < 8 || outputs % 8 ||
            inner < 32 || inner % 32 ||
            (activation_block != 32 && !(packed && activation_block == 128)) ||
            inner % activation_block ||
            uint64_t(groups) * uint64_t(rows) > SIZE_MAX / (uint64_t(outputs) * 2))
            return fail(context, "invalid grouped matrix dimensions", 1);
        if (!groups || !rows)
            return 0;
        if (!input || !input_scale || !metadata || !active || !counts || !output ||
            !aligned(input, 16) || !aligned(metadata, 8) || !aligned(active, 4) ||
            !aligned(counts, 4) || !aligned(output, 2) || output == input ||
            output == input_scale || output == metadata || output == active || output == counts)
            return fail(context, "invalid grouped matrix buffers", 1);
        context->counts[4]++;
        hipError_t error = launch_mx_matmul(context->stream, context->override_kernel,
                                            context->compute_units, packed != 0, groups,
                                            weight_groups, rows, outputs, inner, activation_block,
                                            input, input_scale, nullptr, nullptr, metadata, active,
                                            counts, output);
        return error == hipSuccess ? 0 : fail(context, "grouped multiplication", error);
    });
}

// ref: src/cuda/backend.cu:1306-1337
extern "C" int camblas_cuda_route_groups(camblas_cuda_context *context, int tokens, int choices,
                                         int first_expert, int groups, int rows,
                                         const void *experts, const void *active, void *counts,
                                         void *slots, void *reverse)
{
    return execute(context, [&] {
        if (tokens < 0 || choices < 1 || choices > 64 || first_expert < 0 || groups < 1 ||
            groups > 65535 || rows < 1 || rows > 65535 || int64_t(tokens) * choices > INT_MAX ||
            int64_t(groups) * rows > INT_MAX || !counts || !slots ||
            (tokens && (!experts || !reverse)) || !active || !aligned(experts, 8) ||
            !aligned(active, 4) || !aligned(counts, 4) || !aligned(slots, 4) ||
            !aligned(reverse, 4) || counts == active || slots == active || reverse == active ||
            counts == experts || slots == experts || (reverse && reverse == experts) ||
            counts == slots || counts == reverse || slots == reverse)
            return fail(context, "invalid routing dimensions or buffers", 1);
        hipError_t error = launch_route_groups(context->stream, tokens, choices, first_expert, groups,
                                               rows, experts, active, counts, slots, reverse);
        return error == hipSuccess ? 0 : fail(context, "expert routing", error);
    });
}

// ref: src/cuda/backend.cu:1339-1361
extern "C" int camblas_cuda_reduce_groups(camblas_cuda_context *context, int tokens, int choices,
                                          int width, int grouped_rows, const void *experts,
                                          const void *reverse, const void *input, void *output)
{
    return execute(context, [&] {
        if (tokens < 0 || choices < 1 || choices > 64 || width < 1 || grouped_rows < 0 ||
            int64_t(tokens) * choices > INT_MAX || (grouped_rows && !input) ||
            (tokens && (!experts || !reverse || !output)) || !aligned(experts, 8) ||
            !aligned(reverse, 4) || !aligned(input, 2) || !aligned(output, 4) ||
            (tokens && (output == experts || output == reverse || output == input)))
            return fail(context, "invalid grouped reduction arguments", 1);
        if (!tokens)
            return 0;
        hipError_t error = launch_reduce_groups(context->stream, tokens, choices, width, grouped_rows,
                                                experts, reverse, input, output);
        return error == hipSuccess ? 0 : fail(context, "grouped reduction", error);
    });
}

// ref: src/cuda/backend.cu:1193-1256 (validation order and messages of the block-32 decode pair)
extern "C" int camblas_cuda_fp8_decode_supported(const camblas_cuda_context *context)
{
    return context ? 1 : 0;
}

extern "C" size_t camblas_cuda_fp8_workspace_size(int quantise, int outputs, int inner)
{
    (void)quantise, (void)outputs, (void)inner;
    return 0; // both operations are single kernels that stage the token in LDS
}

extern "C" int camblas_cuda_fp8_decode(camblas_cuda_context *context, int outputs, int inner,
                                       const void *input, const float *input_scale,
                                       const void *weight, const float *weight_scale,
                                       int input_scale_stride, int weight_scale_row_stride,
                                       int weight_scale_column_stride, void *workspace,
                                       size_t workspace_bytes, void *output)
{
    (void)workspace, (void)workspace_bytes;
    return execute(context, [&] {
        if (outputs < 16 || outputs % 16 || inner < 32 || inner > 8192 || inner % 32 ||
            input_scale_stride < 1 || weight_scale_row_stride < 1 || weight_scale_column_stride < 1)
            return fail(context, "invalid FP8 decode dimensions or scale strides", 1);
        if (!input || !input_scale || !weight || !weight_scale || !output || !aligned(input, 4) ||
            !aligned(weight, 16) || !aligned(input_scale, 4) || !aligned(weight_scale, 4) ||
            !aligned(output, 2) || output == input || output == weight ||
            output == (const void *)input_scale || output == (const void *)weight_scale)
            return fail(context, "invalid FP8 decode buffers", 1);
        context->counts[4]++;
        hipError_t error = launch_fp8_block32_decode(
            context->stream, outputs, inner, input, input_scale, input_scale_stride, weight,
            weight_scale, weight_scale_row_stride, weight_scale_column_stride, output);
        return error == hipSuccess ? 0 : fail(context, "FP8 block-32 decode", error);
    });
}

extern "C" int camblas_cuda_fp8_linear(camblas_cuda_context *context, int outputs, int inner,
                                       const void *input, const void *weight,
                                       const float *weight_scale, int weight_scale_row_stride,
                                       int weight_scale_column_stride, void *workspace,
                                       size_t workspace_bytes, void *output)
{
    (void)workspace, (void)workspace_bytes;
    return execute(context, [&] {
        if (outputs < 16 || outputs % 16 || inner < 32 || inner > 8192 || inner % 32 ||
            weight_scale_row_stride < 1 || weight_scale_column_stride < 1)
            return fail(context, "invalid FP8 decode dimensions or scale strides", 1);
        if (!input || !weight || !weight_scale || !output || !aligned(input, 4) ||
            !aligned(weight, 16) || !aligned(weight_scale, 4) || !aligned(output, 2) ||
            output == input || output == weight || output == (const void *)weight_scale)
            return fail(context, "invalid FP8 decode buffers", 1);
        context->counts[4]++;
        hipError_t error = launch_fp8_block32_decode(
            context->stream, outputs, inner, input, nullptr, 1, weight, weight_scale,
            weight_scale_row_stride, weight_scale_column_stride, output);
        return error == hipSuccess ? 0 : fail(context, "FP8 block-32 linear", error);
    });
}

extern "C" int camblas_cuda_fp8_quantise_1x128(camblas_cuda_context *context, int rows, int inner,
                                               const void *x, void *q, float *scale)
{
    return execute(context, [&] {
        if (rows < 0 || inner < 128 || inner % 128)
            return fail(context, "invalid FP8 quantiser dimensions", 1);
        if (!rows)
            return 0;
        if (!x || !q || !scale || !aligned(x, 16) || !aligned(q, 16) || !aligned(scale, 4) ||
            q == x)
            return fail(context, "invalid FP8 quantiser buffers", 1);
        hipError_t error = launch_fp8_quantise(context->stream, rows, inner, x, q, scale);
        return error == hipSuccess ? 0 : fail(context, "FP8 activation quantisation", error);
    });
}

extern "C" size_t camblas_cuda_fp8_block_workspace_size(int rows, int inner)
{
    if (rows <= 0 || inner < 128 || inner % 128)
        return 0;
    size_t bytes = (size_t(rows) * inner + 15) & ~size_t(15);
    return bytes + size_t(rows) * (inner / 128) * sizeof(float);
}

extern "C" int camblas_cuda_fp8_block_linear(camblas_cuda_context *context, int rows, int outputs,
                                             int inner, const void *x, const void *w,
                                             const float *w_scale, void *workspace,
                                             size_t workspace_bytes, void *out)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    if (rows < 0 || rows > 65535 || outputs < 1 || inner < 128 || inner % 128)
        return fail(context, "invalid FP8 block matrix dimensions", 1);
    if (!rows)
        return 0;
    size_t required = camblas_cuda_fp8_block_workspace_size(rows, inner);
    if (!workspace || workspace_bytes < required || !aligned(workspace, 16) || workspace == x ||
        workspace == w || workspace == out)
        return fail(context, "invalid FP8 block linear workspace", 1);
    unsigned char *q = static_cast<unsigned char *>(workspace);
    float *scale = reinterpret_cast<float *>(q + ((size_t(rows) * inner + 15) & ~size_t(15)));
    int status = camblas_cuda_fp8_quantise_1x128(context, rows, inner, x, q, scale);
    if (status != 0)
        return status;
    return camblas_cuda_fp8_block_matmul(context, rows, outputs, inner, q, scale, w, w_scale, out);
}

// One token through a block-scaled FP8 mixture-of-experts layer (rule of camblas/_hopper.py:329-401,
// which the reference reaches from Python only; here it is an entry point like the other products).
extern "C" int camblas_cuda_fp8_moe_decode(camblas_cuda_context *context, int experts, int choices,
                                           int hidden, int width, int hidden_out, const void *x,
                                           const void *w1, const float *w1_scale, const void *w2,
                                           const float *w2_scale, const int32_t *expert_ids,
                                           const float *routing, float factor, void *output)
{
    return execute(context, [&] {
        if (experts < 1 || choices < 1 || choices > 16 || hidden < 128 || hidden % 128 ||
            width < 128 || width % 128 || hidden_out < 16 || hidden_out % 16 ||
            choices * (width / 128) > 512 || !std::isfinite(factor)) // (LDS of the second launch)
            return fail(context, "invalid FP8 expert dimensions", 1);
        if (!x || !w1 || !w1_scale || !w2 || !w2_scale || !expert_ids || !routing || !output ||
            !aligned(x, 16) || !aligned(w1, 16) || !aligned(w2, 16) || !aligned(w1_scale, 4) ||
            !aligned(w2_scale, 4) || !aligned(expert_ids, 4) || !aligned(routing, 4) ||
            !aligned(output, 2) || output == w1 || output == w2)
            return fail(context, "invalid FP8 expert buffers", 1);
        hipError_t grown = reserve_scratch(context, fp8_moe_decode_scratch_bytes(choices, width));
        if (grown != hipSuccess)
            return fail(context, "FP8 expert scratch", grown);
        context->counts[4]++;
        hipError_t error = launch_fp8_moe_decode(context->stream, experts, choices, hidden, width,
                                                 hidden_out, x, w1, w1_scale, w2, w2_scale, expert_ids,
                                                 routing, factor, context->scratch, output);
        return error == hipSuccess ? 0 : fail(context, "FP8 expert step", error);
    });
}

extern "C" int camblas_cuda_rope(camblas_cuda_context *context, int tokens, int heads, int dim,
                                 int token_stride, float theta, const int32_t *positions, void *x)
{
    return execute(context, [&] {
        if (tokens < 0 || heads < 1 || dim < 2 || dim % 2 || token_stride < heads * dim ||
            !std::isfinite(theta) || theta <= 0)
            return fail(context, "invalid rotary embedding arguments", 1);
        if (!tokens)
            return 0;
        if (!positions || !x || !aligned(x, 2) || !aligned(positions, 4))
            return fail(context, "invalid rotary embedding buffers", 1);
        hipError_t error =
            launch_rope(context->stream, tokens, heads, dim, token_stride, theta, positions, x);
        return error == hipSuccess ? 0 : fail(context, "rotary embedding", error);
    });
}

extern "C" int camblas_cuda_kv_append(camblas_cuda_context *context, int batch, int kv_heads, int dim,
                                      int context_length, const int32_t *positions,
                                      const void *k_new, const void *v_new, int token_stride,
                                      void *k_cache, void *v_cache)
{
    return execute(context, [&] {
        if (batch < 0 || kv_heads < 1 || dim < 8 || dim % 8 || context_length < 1 ||
            token_stride < kv_heads * dim || token_stride % 8)
            return fail(context, "invalid cache append arguments", 1);
        if (!batch)
            return 0;
        if (!positions || !k_new || !v_new || !k_cache || !v_cache || !aligned(k_new, 16) ||
            !aligned(v_new, 16) || !aligned(k_cache, 16) || !aligned(v_cache, 16) ||
            k_cache == v_cache)
            return fail(context, "invalid cache append buffers", 1);
        hipError_t error = launch_kv_append(context->stream, batch, kv_heads, dim, context_length,
                                            positions, k_new, v_new, token_stride, k_cache, v_cache);
        return error == hipSuccess ? 0 : fail(context, "cache append", error);
    });
}

extern "C" int camblas_cuda_rope_kv_append(camblas_cuda_context *context, int batch, int q_heads,
                                           int kv_heads, int dim, int token_stride, float theta,
                                           const int32_t *positions, void *qkv, int context_length,
                                           void *k_cache, void *v_cache)
{
    return execute(context, [&] {
        if (batch < 0 || q_heads < 1 || kv_heads < 1 || dim < 2 || dim % 2 || context_length < 1 ||
            token_stride < (q_heads + 2 * kv_heads) * dim || !std::isfinite(theta) || theta <= 0)
            return fail(context, "invalid rotary cache append arguments", 1);
        if (!batch)
            return 0;
        if (!positions || !qkv || !k_cache || !v_cache || k_cache == v_cache || !aligned(qkv, 2) ||
            !aligned(k_cache, 2) || !aligned(v_cache, 2) || !aligned(positions, 4))
            return fail(context, "invalid rotary cache append buffers", 1);
        hipError_t error =
            launch_rope_kv_append(context->stream, batch, q_heads, kv_heads, dim, token_stride,
                                  theta, positions, qkv, context_length, k_cache, v_cache);
        return error == hipSuccess ? 0 : fail(context, "rotary cache append", error);
    });
}

namespace camblas_hip
{
namespace
{
// Shared by the two decode-attention entry points: argument checks, then the launch with the
// partials wherever `partials_for(bytes, &where)` puts them.
template <typename Partials>
int gqa_decode(camblas_cuda_context *context, int batch, int q_heads, int kv_heads, int dim,
               int context_length, const int32_t *lengths, float scale, const void *q, int q_stride,
               const void *k_cache, const void *v_cache, void *output, Partials partials_for)
{
    if (batch < 0 || q_heads < 1 || kv_heads < 1 || q_heads % kv_heads || q_heads / kv_heads > 16 ||
        dim != 128 || context_length < 1 || q_stride < q_heads * dim || !std::isfinite(scale))
        return fail(context, "invalid decode attention arguments", 1);
    if (!batch)
        return 0;
    if (!q || !k_cache || !v_cache || !output || !aligned(q, 16) || !aligned(k_cache, 16) ||
        !aligned(v_cache, 16) || !aligned(output, 16) || q_stride % 8 || output == q ||
        output == k_cache || output == v_cache)
        return fail(context, "invalid decode attention buffers", 1);
    int splits = 1;
    const size_t bytes = gqa_decode_scratch_bytes(batch, q_heads, dim, context_length, &splits);
    void *partials = nullptr;
    if (int refused = partials_for(bytes, &partials))
        return refused;
    context->counts[6]++;
    hipError_t error =
        launch_gqa_decode(context->stream, batch, q_heads, kv_heads, dim, context_length, lengths,
                          scale, q, q_stride, k_cache, v_cache, output, partials, splits);
    return error == hipSuccess ? 0 : fail(context, "decode attention", error);
}
} // namespace
} // namespace camblas_hip

extern "C" int camblas_cuda_gqa_decode_attention(camblas_cuda_context *context, int batch,
                                                 int q_heads, int kv_heads, int dim,
                                                 int context_length, const int32_t *lengths,
                                                 float scale, const void *q, int q_stride,
                                                 const void *k_cache, const void *v_cache,
                                                 void *output)
{
    return execute(context, [&] {
        return gqa_decode(context, batch, q_heads, kv_heads, dim, context_length, lengths, scale, q,
                          q_stride, k_cache, v_cache, output, [&](size_t bytes, void **where) {
                              hipError_t grown = reserve_scratch(context, bytes);
                              if (grown != hipSuccess)
                                  return fail(context, "decode attention scratch", grown);
                              *where = context->scratch;
                              return 0;
                          });
    });
}

extern "C" size_t camblas_cuda_gqa_decode_attention_noalloc_limit(void)
{
    return gqa_resident_scratch_bytes();
}

// The same kernels with the partials in the library's fixed device array: no hipMalloc, no
// hipFree, no context scratch. Calls that overlap on one GPU share that array and race.
extern "C" int camblas_cuda_gqa_decode_attention_noalloc(camblas_cuda_context *context, int batch,
                                                         int q_heads, int kv_heads, int dim,
                                                         int context_length, const int32_t *lengths,
                                                         float scale, const void *q, int q_stride,
                                                         const void *k_cache, const void *v_cache,
                                                         void *output)
{
    return execute(context, [&] {
        return gqa_decode(context, batch, q_heads, kv_heads, dim, context_length, lengths, scale, q,
                          q_stride, k_cache, v_cache, output, [&](size_t bytes, void **where) {
                              if (bytes > gqa_resident_scratch_bytes()) {
                                  std::snprintf(context->error, sizeof(context->error),
                                                "decode attention needs %zu bytes of partials; the "
                                                "allocation-free entry point holds %zu",
                                                bytes, gqa_resident_scratch_bytes());
                                  return -1;
                              }
                              hipError_t found = gqa_resident_scratch(context->device, where);
                              return found == hipSuccess
                                         ? 0
                                         : fail(context, "resident decode attention partials", found);
                          });
    });
}

extern "C" int camblas_hip_plan_describe(int dtype, int algorithm, char trans_a, char trans_b, int m,
                                         int n, int k, int lda, int ldb, int ldc, int aligned16,
                                         char *text, size_t text_bytes)
{
    if ((dtype != 0 && dtype != 2 && dtype != 3) || (!is_n(trans_a) && !is_t(trans_a)) ||
        (!is_n(trans_b) && !is_t(trans_b)) || m < 1 || n < 1 || k < 1)
        return -1;
    Plan plan = make_plan(dtype, algorithm, is_t(trans_a), is_t(trans_b), m, n, k, lda, ldb, ldc,
                          aligned16 != 0, 256);
    describe_plan(plan, dtype, text, text_bytes);
    return plan.family * 1000 + plan.kernel;
}

extern "C" int camblas_hip_set_plan_override(camblas_cuda_context *context, int kernel, int split_k)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    context->override_kernel = kernel;
    context->override_split = split_k;
    return 0;
}

extern "C" int camblas_hip_copy_probe(camblas_cuda_context *context, size_t bytes, const void *source,
                                      void *destination)
{
    return execute(context, [&] {
        if (bytes % 16 || !source || !destination || !aligned(source, 16) ||
            !aligned(destination, 16))
            return fail(context, "invalid copy probe arguments", 1);
        if (!bytes)
            return 0;
        hipError_t error = launch_copy_probe(context->stream, bytes, source, destination);
        return error == hipSuccess ? 0 : fail(context, "copy probe", error);
    });
}

extern "C" int camblas_hip_matrix_probe(camblas_cuda_context *context, int kind, int rounds,
                                        int constant_operands, void *sink, size_t sink_bytes,
                                        double *flops)
{
    return execute(context, [&] {
        const size_t needed = size_t(context->compute_units) * 512 * sizeof(float);
        if (kind < 0 || kind > 3 || rounds < 1 || !sink || !flops || !aligned(sink, 4) ||
            sink_bytes < needed)
            return fail(context, "invalid matrix probe arguments", 1);
        hipError_t error = launch_matrix_probe(context->stream, kind, context->compute_units, rounds,
                                               constant_operands != 0, static_cast<float *>(sink), flops);
        return error == hipSuccess ? 0 : fail(context, "matrix probe", error);
    });
}

extern "C" int camblas_hip_kernel_count(int dtype)
{
    return dtype == 2 ? tn_variant_count() : dtype == 3 ? fp8_variant_count() : 1;
}
