// Guarded Strassen policies for square FP32 / FP64 'N','N' products (ref: src/cuda/backend.cu:107-165
// for the quadrant sums and their order, :442-551 for the driver, :836-853 for the gate).
//
// One level replaces an n x n product by seven of size n/2:
//   P1 = (A11 + A22)(B11 + B22)   P2 = (A21 + A22) B11     P3 = A11 (B12 - B22)
//   P4 = A22 (B21 - B11)          P5 = (A11 + A12) B22     P6 = (A21 - A11)(B11 + B12)
//   P7 = (A12 - A22)(B21 + B22)
//   C11 = ((P1 + P4) - P5) + P7   C12 = P3 + P5   C21 = P2 + P4   C22 = ((P1 - P2) + P3) + P6
// Deeper policies apply the same step to the seven operands again: level l holds 7^l matrices of
// size n / 2^l, child t of parent p at index 7 p + t, every level contiguous in the context scratch.
// All 7^L products run as one batched launch of the matrix-core kernel (one grid z-slice each), so
// small sub-products still fill the compute units. Splitting and recombination are one pass over
// memory per level, ping-ponged between two buffers per operand:
//
//   scratch: [guard flag, 256 B][A_L][B_L][P_L][spare: level L-1]
//
// Level l of an operand lives in its own buffer when L - l is even and in the spare otherwise; the
// products come back the same way (level L in P_L, L-1 in the spare, L-2 in P_L, ... level 0 in C).
// The guard: sums of quadrants and of products must not overflow, so the first split raises a flag
// when an input is not finite or exceeds sqrt(max / (factor n max(1, |alpha|))); the host reads
// the flag (one stream synchronisation, as in the reference) and the caller then runs the
// ordinary kernel. That is also why these policies never run under stream capture.
#include "common.hpp"

#include <algorithm>
#include <cmath>
#include <limits>

namespace camblas_hip
{
namespace
{
constexpr int SPLIT_THREADS = 256;
constexpr size_t FLAG_BYTES = 256;

// Quadrants of a 2h x 2h column-major matrix with leading dimension ld, at (row, column) of each.
template <typename T> struct Quadrants {
    T q11, q12, q21, q22;
    __device__ Quadrants(const T *matrix, size_t ld, int h, int row, int column)
        : q11(matrix[row + column * ld]), q12(matrix[row + (column + h) * ld]),
          q21(matrix[row + h + column * ld]), q22(matrix[row + h + (column + h) * ld])
    {
    }
};

// parents x (2h x 2h, leading dimension ld, parent_stride apart) -> 7 parents x (h x h, packed)
template <typename T, bool RIGHT>
__global__ __launch_bounds__(SPLIT_THREADS) void strassen_split_kernel(const T *input, size_t ld,
                                                                      size_t parent_stride, int h,
                                                                      T *children, T limit,
                                                                      unsigned *unsafe)
{
    const size_t area = size_t(h) * h;
    const size_t index = size_t(blockIdx.x) * SPLIT_THREADS + threadIdx.x;
    if (index >= area)
        return;
    const int row = int(index % h), column = int(index / h);
    const Quadrants<T> q(input + blockIdx.y * parent_stride, ld, h, row, column);
    if (unsafe) {
        const bool safe = fabs(q.q11) <= limit && fabs(q.q12) <= limit && fabs(q.q21) <= limit &&
                          fabs(q.q22) <= limit; // false for NaN
        if (__any(!safe) && threadIdx.x % 64 == 0)
            atomicOr(unsafe, 1u);
    }
    T *out = children + size_t(blockIdx.y) * 7 * area + index;
    if (RIGHT) {
        out[0 * area] = q.q11 + q.q22;
        out[1 * area] = q.q11;
        out[2 * area] = q.q12 - q.q22;
        out[3 * area] = q.q21 - q.q11;
        out[4 * area] = q.q22;
        out[5 * area] = q.q11 + q.q12;
        out[6 * area] = q.q21 + q.q22;
    } else {
        out[0 * area] = q.q11 + q.q22;
        out[1 * area] = q.q21 + q.q22;
        out[2 * area] = q.q11;
        out[3 * area] = q.q22;
        out[4 * area] = q.q11 + q.q12;
        out[5 * area] = q.q21 - q.q11;
        out[6 * area] = q.q12 - q.q22;
    }
}

// 7 parents x (h x h products) -> parents x (2h x 2h, leading dimension ld, parent_stride apart):
// out = alpha * C + beta * out; beta == 0 never reads out
template <typename T>
__global__ __launch_bounds__(SPLIT_THREADS) void strassen_join_kernel(const T *products, int h, T alpha,
                                                                     T beta, T *output, size_t ld,
                                                                     size_t parent_stride)
{
    const size_t area = size_t(h) * h;
    const size_t index = size_t(blockIdx.x) * SPLIT_THREADS + threadIdx.x;
    if (index >= area)
        return;
    const T *p = products + size_t(blockIdx.y) * 7 * area + index;
    const T p1 = p[0], p2 = p[area], p3 = p[2 * area], p4 = p[3 * area], p5 = p[4 * area],
            p6 = p[5 * area], p7 = p[6 * area];
    const int row = int(index % h), column = int(index / h);
    T *out = output + blockIdx.y * parent_stride + row + column * ld;
    auto store = [&](T *target, T value) {
        *target = beta == T(0) ? alpha * value : alpha * value + beta * *target;
    };
    store(out, ((p1 + p4) - p5) + p7);
    store(out + h * ld, p3 + p5);
    store(out + h, p2 + p4);
    store(out + h + h * ld, ((p1 - p2) + p3) + p6);
}

hipError_t batched_product(hipStream_t stream, int compute_units, int size, int batches, const float *a,
                           const float *b, float *c)
{
    const long long tiles = (long long)((size + 127) / 128) * ((size + 127) / 128) * batches;
    return launch_sgemm_mfma(stream, tiles >= 2LL * compute_units, false, false, size, size, size, 1.f, a,
                             size, b, size, 0.f, c, size, batches, size_t(size) * size);
}

hipError_t batched_product(hipStream_t stream, int, int size, int batches, const double *a, const double *b,
                           double *c)
{
    return launch_dgemm_mfma(stream, false, false, size, size, size, 1.0, a, size, b, size, 0.0, c, size,
                             batches, size_t(size) * size);
}

size_t power_of_seven(int level)
{
    size_t value = 1;
    for (int l = 0; l < level; ++l)
        value *= 7;
    return value;
}
} // namespace

int strassen_levels(int algorithm, int n)
{
    int levels = algorithm == CAMBLAS_CUDA_STRASSEN_FOUR    ? 4
                 : algorithm == CAMBLAS_CUDA_STRASSEN_THREE ? 3
                 : algorithm == CAMBLAS_CUDA_STRASSEN_TWO   ? 2
                 : algorithm == CAMBLAS_CUDA_STRASSEN       ? 1
                                                            : 0;
    // the default policy splits twice from 8192: measured 10.0 -> 8.8 ms (FP32) and 18.1 -> 16.3 ms
    // (FP64) there and 80 -> 66 ms at 16384, while at 4096 one level gains 5 % and two lose 4 %
    // (the reference's thresholds, 4096 for FP32 and 8192 for FP64, belong to its hardware)
    if (algorithm == CAMBLAS_CUDA_AUTO && n >= 8192)
        levels = 2;
    // every level halves n exactly, and the leaves keep at least one 32 x 32 matrix-core tile
    while (levels > 0 && (n % (1 << levels) != 0 || (n >> levels) < 32))
        --levels;
    return levels;
}

template <typename T>
int strassen_gemm(camblas_cuda_context *context, int levels, int n, T alpha, const T *a, int lda, const T *b,
                  int ldb, T beta, T *c, int ldc)
{
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    hipStreamIsCapturing(context->stream, &capture);
    auto in_scratch = [context](const void *pointer) {
        const uintptr_t address = reinterpret_cast<uintptr_t>(pointer);
        const uintptr_t base = reinterpret_cast<uintptr_t>(context->scratch);
        return address >= base && address - base < context->scratch_bytes;
    };
    // (an enclosing helper holds part of the arena: the workspace would move or overwrite it)
    if (levels < 1 || capture != hipStreamCaptureStatusNone || !std::isfinite(double(alpha)) ||
        context->held_bytes || in_scratch(a) || in_scratch(b) || in_scratch(c))
        return STRASSEN_NOT_ELIGIBLE;

    // scratch for L levels; an allocation failure drops a level (counted once as a guard fallback).
    // The default policy was not asked for by name, so it never grows the scratch beyond 16 GiB
    // (arenas kept alive for captured graphs included): it drops levels, or leaves the product to
    // the ordinary kernel, without counting anything.
    constexpr size_t DEFAULT_POLICY_LIMIT = size_t(16) << 30;
    bool counted = false;
    size_t leaves = 0, leaf_elements = 0, spare_elements = 0;
    for (;; --levels) {
        if (levels == 0) {
            if (!counted && context->algorithm == CAMBLAS_CUDA_AUTO)
                return STRASSEN_NOT_ELIGIBLE;
            if (!counted)
                context->counts[5]++;
            return STRASSEN_FALL_BACK;
        }
        const size_t leaf = size_t(n >> levels);
        leaves = power_of_seven(levels);
        leaf_elements = leaves * leaf * leaf;
        spare_elements = levels > 1 ? power_of_seven(levels - 1) * (2 * leaf) * (2 * leaf) : 0;
        const size_t bytes = FLAG_BYTES + (3 * leaf_elements + spare_elements) * sizeof(T);
        if (context->algorithm == CAMBLAS_CUDA_AUTO && bytes > context->scratch_bytes &&
            bytes + context->retired_bytes > DEFAULT_POLICY_LIMIT)
            continue;
        const hipError_t status = reserve_scratch(context, bytes);
        if (status == hipSuccess)
            break;
        if (status != hipErrorOutOfMemory)
            return fail(context, "Strassen scratch", status);
        if (!counted)
            context->counts[5]++;
        counted = true;
    }
    if (leaves > 65535)
        return fail(context, "Strassen batch count", 1);

    unsigned *flag = static_cast<unsigned *>(context->scratch);
    T *own_a = reinterpret_cast<T *>(static_cast<char *>(context->scratch) + FLAG_BYTES);
    T *own_b = own_a + leaf_elements, *products = own_b + leaf_elements, *spare = products + leaf_elements;
    const double factor = levels == 4 ? 8192.0 : 16.0 * double(1 << (2 * levels));
    const T limit = T(std::sqrt(double(std::numeric_limits<T>::max()) /
                                (factor * n * std::max(1.0, std::fabs(double(alpha))))));
    hipStream_t stream = context->stream;
    hipError_t error = hipMemsetAsync(flag, 0, sizeof(unsigned), stream);
    if (error != hipSuccess)
        return fail(context, "range-flag reset", error);

    auto split = [&](const T *matrix, int ld, T *own, bool right) {
        const T *source = matrix;
        size_t source_ld = size_t(ld), stride = 0, parents = 1;
        for (int level = 1; level <= levels; ++level) {
            const int h = n >> level;
            T *target = (levels - level) % 2 == 0 ? own : spare;
            dim3 grid(unsigned((size_t(h) * h + SPLIT_THREADS - 1) / SPLIT_THREADS), unsigned(parents));
            unsigned *guard = level == 1 ? flag : nullptr;
            if (right)
                strassen_split_kernel<T, true>
                    <<<grid, SPLIT_THREADS, 0, stream>>>(source, source_ld, stride, h, target, limit, guard);
            else
                strassen_split_kernel<T, false>
                    <<<grid, SPLIT_THREADS, 0, stream>>>(source, source_ld, stride, h, target, limit, guard);
            source = target;
            source_ld = size_t(h);
            stride = size_t(h) * h;
            parents *= 7;
        }
    };
    split(a, lda, own_a, false);
    split(b, ldb, own_b, true);
    if ((error = launch_status()) != hipSuccess)
        return fail(context, "Strassen operand sums", error);

    unsigned raised = 0;
    error = hipMemcpyAsync(&raised, flag, sizeof(unsigned), hipMemcpyDeviceToHost, stream);
    if (error == hipSuccess)
        error = hipStreamSynchronize(stream);
    if (error != hipSuccess)
        return fail(context, "packed-input range check", error);
    if (raised) {
        if (!counted)
            context->counts[5]++;
        return STRASSEN_FALL_BACK;
    }

    error = batched_product(stream, context->compute_units, n >> levels, int(leaves), own_a, own_b, products);
    if (error != hipSuccess)
        return fail(context, "packed batched GEMM", error);
    context->counts[1]++;

    for (int level = levels; level >= 1; --level) {
        const int h = n >> level;
        const size_t parents = power_of_seven(level - 1);
        const T *source = (levels - level) % 2 == 0 ? products : spare;
        dim3 grid(unsigned((size_t(h) * h + SPLIT_THREADS - 1) / SPLIT_THREADS), unsigned(parents));
        if (level == 1) {
            strassen_join_kernel<T><<<grid, SPLIT_THREADS, 0, stream>>>(source, h, alpha, beta, c, size_t(ldc), 0);
        } else {
            T *target = (levels - level + 1) % 2 == 0 ? products : spare;
            strassen_join_kernel<T><<<grid, SPLIT_THREADS, 0, stream>>>(source, h, T(1), T(0), target,
                                                                       size_t(2 * h), size_t(2 * h) * (2 * h));
        }
    }
    error = launch_status();
    return error == hipSuccess ? STRASSEN_DONE : fail(context, "Strassen recombination", error);
}

template int strassen_gemm<float>(camblas_cuda_context *, int, int, float, const float *, int, const float *,
                                  int, float, float *, int);
template int strassen_gemm<double>(camblas_cuda_context *, int, int, double, const double *, int,
                                   const double *, int, double, double *, int);
} // namespace camblas_hip
