// Elementwise and reduction kernels around the FP32/FP64 GEMM for the dense network helpers of the
// C ABI: bias + optional ReLU (affine, MLP), scaled row softmax (dense single-head attention) and
// the column sums of the MLP gradients with the ReLU mask applied in place.
// Contracts: ref include/camblas_cuda.h:71-94; semantics src/cuda/backend.cu:871-905 (affine),
// src/cuda/fusion.cuh:43-157 (softmax and attention), :159-275 (bias gradients and MLP backward).
//
// All reductions have a fixed order (a function of the shape only), so results repeat bit for bit.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int THREADS = 256;

// out[r, c] += bias[c]; ReLU keeps NaN (v < 0 is false for NaN) and sends -inf to zero.
template <typename T>
__global__ void bias_activation_kernel(T *out, const T *bias, size_t count, int columns, bool relu)
{
    const size_t index = size_t(blockIdx.x) * THREADS + threadIdx.x;
    if (index >= count)
        return;
    T value = out[index] + bias[index % size_t(columns)];
    if (relu)
        value = value < T(0) ? T(0) : value;
    out[index] = value;
}

template <typename T> __device__ __forceinline__ T shuffle_xor(T value, int mask)
{
    return __shfl_xor(value, mask, 64);
}

// Workgroup-wide maximum or sum over 256 threads: butterfly inside each wavefront (every lane ends
// with the wavefront's value), then the four wavefront values in index order through LDS.
template <typename T, bool MAXIMUM> __device__ T group_reduce(T value, T *shared)
{
#pragma unroll
    for (int mask = 32; mask > 0; mask >>= 1) {
        const T other = shuffle_xor(value, mask);
        value = MAXIMUM ? (other > value || value != value ? other : value) : value + other;
    }
    const int wave = threadIdx.x / 64;
    __syncthreads(); // the previous use of `shared` has been read by everyone
    if (threadIdx.x % 64 == 0)
        shared[wave] = value;
    __syncthreads();
    T result = shared[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) {
        const T other = shared[w];
        result = MAXIMUM ? (other > result || result != result ? other : result) : result + other;
    }
    return result;
}

template <typename T> __device__ __forceinline__ T exponential(T value);
template <> __device__ __forceinline__ float exponential<float>(float value) { return expf(value); }
template <> __device__ __forceinline__ double exponential<double>(double value) { return exp(value); }

// In-place softmax(scale * row) of one row per workgroup. ITEMS > 0: the row (at most 256*ITEMS
// columns) stays in registers between the passes; ITEMS == 0: any width, three passes over memory.
// The maximum ignores NaN, so a NaN score turns the whole row into NaN through the sum, like
// torch.softmax does.
template <typename T, int ITEMS>
__global__ __launch_bounds__(THREADS) void softmax_rows_kernel(T *scores, int columns, T scale)
{
    __shared__ T shared[THREADS / 64];
    T *row = scores + size_t(blockIdx.x) * columns;
    const T lowest = -INFINITY;
    if constexpr (ITEMS > 0) {
        T values[ITEMS];
        T maximum = lowest;
#pragma unroll
        for (int item = 0; item < ITEMS; ++item) {
            const int column = int(threadIdx.x) + item * THREADS;
            values[item] = column < columns ? row[column] * scale : lowest;
            maximum = values[item] > maximum ? values[item] : maximum;
        }
        maximum = group_reduce<T, true>(maximum, shared);
        T sum = 0;
#pragma unroll
        for (int item = 0; item < ITEMS; ++item) {
            const int column = int(threadIdx.x) + item * THREADS;
            values[item] = column < columns ? exponential(values[item] - maximum) : T(0);
            sum += values[item];
        }
        sum = group_reduce<T, false>(sum, shared);
#pragma unroll
        for (int item = 0; item < ITEMS; ++item) {
            const int column = int(threadIdx.x) + item * THREADS;
            if (column < columns)
                row[column] = values[item] / sum;
        }
    } else {
        T maximum = lowest;
        for (int column = threadIdx.x; column < columns; column += THREADS) {
            const T value = row[column] * scale;
            maximum = value > maximum ? value : maximum;
        }
        maximum = group_reduce<T, true>(maximum, shared);
        T sum = 0;
        for (int column = threadIdx.x; column < columns; column += THREADS) {
            const T value = exponential(row[column] * scale - maximum);
            row[column] = value;
            sum += value;
        }
        sum = group_reduce<T, false>(sum, shared);
        for (int column = threadIdx.x; column < columns; column += THREADS)
            row[column] /= sum;
    }
}

// Partial column sums of a row-major [rows, columns] matrix: workgroup (x, y) covers 64 columns and
// the rows of chunk y; its four wavefronts take rows r = 4i + wave of the chunk and are added in
// wavefront order. MASK: entries whose activation is not positive are first set to zero in `grad`
// itself (the ReLU derivative). partial is [chunks, columns].
template <typename T, bool MASK>
__global__ __launch_bounds__(THREADS) void column_sums_kernel(T *grad, const T *activation, int rows,
                                                              int columns, int chunk_rows,
                                                              T *partial)
{
    __shared__ T shared[THREADS / 64][64];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int64_t column = int64_t(blockIdx.x) * 64 + lane;
    const int64_t begin = int64_t(blockIdx.y) * chunk_rows;
    const int64_t end = begin + chunk_rows < rows ? begin + chunk_rows : rows;
    T sum = 0;
    if (column < columns) {
        for (int64_t row = begin + wave; row < end; row += THREADS / 64) {
            const size_t offset = size_t(row) * columns + column;
            T value = grad[offset];
            if constexpr (MASK) {
                if (!(activation[offset] > T(0)))
                    value = T(0);
                grad[offset] = value;
            }
            sum += value;
        }
    }
    shared[wave][lane] = sum;
    __syncthreads();
    if (wave == 0 && column < columns && partial) {
        T total = shared[0][lane];
#pragma unroll
        for (int w = 1; w < THREADS / 64; ++w)
            total += shared[w][lane];
        partial[size_t(blockIdx.y) * columns + column] = total;
    }
}

// sums[c] = partial[0, c] + partial[1, c] + ... in chunk order
template <typename T>
__global__ void finish_sums_kernel(const T *partial, int chunks, int columns, T *sums)
{
    const int64_t column = int64_t(blockIdx.x) * THREADS + threadIdx.x;
    if (column >= columns)
        return;
    T total = 0;
    for (int chunk = 0; chunk < chunks; ++chunk)
        total += partial[size_t(chunk) * columns + column];
    sums[column] = total;
}

template <typename T>
hipError_t bias_activation(hipStream_t stream, T *out, const T *bias, size_t count, int columns, bool relu)
{
    if (count == 0)
        return hipSuccess;
    const size_t groups = (count + THREADS - 1) / THREADS;
    if (groups > 0x7fffffffu)
        return hipErrorInvalidValue;
    bias_activation_kernel<T><<<unsigned(groups), THREADS, 0, stream>>>(out, bias, count, columns, relu);
    return launch_status();
}

template <typename T> hipError_t softmax_rows(hipStream_t stream, T *scores, int rows, int columns, T scale)
{
    if (rows == 0 || columns == 0)
        return hipSuccess;
    const unsigned grid = unsigned(rows);
    if (columns <= THREADS)
        softmax_rows_kernel<T, 1><<<grid, THREADS, 0, stream>>>(scores, columns, scale);
    else if (columns <= 2 * THREADS)
        softmax_rows_kernel<T, 2><<<grid, THREADS, 0, stream>>>(scores, columns, scale);
    else if (columns <= 4 * THREADS)
        softmax_rows_kernel<T, 4><<<grid, THREADS, 0, stream>>>(scores, columns, scale);
    else if (columns <= 8 * THREADS)
        softmax_rows_kernel<T, 8><<<grid, THREADS, 0, stream>>>(scores, columns, scale);
    else if (columns <= 16 * THREADS)
        softmax_rows_kernel<T, 16><<<grid, THREADS, 0, stream>>>(scores, columns, scale);
    else
        softmax_rows_kernel<T, 0><<<grid, THREADS, 0, stream>>>(scores, columns, scale);
    return launch_status();
}

template <typename T>
hipError_t column_sums(hipStream_t stream, bool mask, T *grad, const T *activation, int rows, int columns,
                       int chunks, int chunk_rows, T *partial, T *sums)
{
    if (columns == 0)
        return hipSuccess;
    dim3 grid(unsigned((size_t(columns) + 63) / 64), unsigned(chunks));
    // one chunk: the partial sums are the result
    T *target = chunks > 1 ? partial : sums;
    if (mask)
        column_sums_kernel<T, true><<<grid, THREADS, 0, stream>>>(grad, activation, rows, columns,
                                                                   chunk_rows, target);
    else
        column_sums_kernel<T, false><<<grid, THREADS, 0, stream>>>(grad, activation, rows, columns,
                                                                    chunk_rows, target);
    hipError_t status = launch_status();
    if (status != hipSuccess || chunks <= 1 || !sums)
        return status;
    finish_sums_kernel<T><<<unsigned((size_t(columns) + THREADS - 1) / THREADS), THREADS, 0, stream>>>(
        partial, chunks, columns, sums);
    return launch_status();
}

// Upper tile (ti, tj), ti <= tj, of a column-major matrix from the transposed lower tile (tj, ti):
// both the reads and the writes run along columns, the transposition happens in LDS.
constexpr int MIRROR_TILE = 32;
template <typename T>
__global__ __launch_bounds__(MIRROR_TILE * 8) void mirror_lower_kernel(int n, T *c, size_t ldc)
{
    __shared__ T tile[MIRROR_TILE][MIRROR_TILE + 1];
    const int ti = blockIdx.x, tj = blockIdx.y;
    if (ti > tj)
        return;
    for (int y = threadIdx.y; y < MIRROR_TILE; y += 8) {
        const int row = tj * MIRROR_TILE + threadIdx.x, column = ti * MIRROR_TILE + y; // lower source
        if (row < n && column < n)
            tile[y][threadIdx.x] = c[row + column * ldc];
    }
    __syncthreads();
    for (int y = threadIdx.y; y < MIRROR_TILE; y += 8) {
        const int row = ti * MIRROR_TILE + threadIdx.x, column = tj * MIRROR_TILE + y; // upper target
        if (row < column && column < n)
            c[row + column * ldc] = tile[threadIdx.x][y];
    }
}
} // namespace

hipError_t launch_mirror_lower(hipStream_t stream, int dtype, int n, void *c, int ldc)
{
    if (n < 2)
        return hipSuccess;
    const unsigned tiles = unsigned((n + MIRROR_TILE - 1) / MIRROR_TILE);
    if (tiles > 65535u)
        return hipErrorInvalidValue;
    dim3 grid(tiles, tiles), block(MIRROR_TILE, 8);
    if (dtype == 0)
        mirror_lower_kernel<<<grid, block, 0, stream>>>(n, static_cast<float *>(c), size_t(ldc));
    else
        mirror_lower_kernel<<<grid, block, 0, stream>>>(n, static_cast<double *>(c), size_t(ldc));
    return launch_status();
}

hipError_t launch_bias_activation(hipStream_t stream, int dtype, void *out, const void *bias,
                                  size_t count, int columns, bool relu)
{
    return dtype == 0 ? bias_activation(stream, static_cast<float *>(out),
                                        static_cast<const float *>(bias), count, columns, relu)
                      : bias_activation(stream, static_cast<double *>(out),
                                        static_cast<const double *>(bias), count, columns, relu);
}

hipError_t launch_softmax_rows(hipStream_t stream, int dtype, void *scores, int rows, int columns,
                               double scale)
{
    return dtype == 0 ? softmax_rows(stream, static_cast<float *>(scores), rows, columns, float(scale))
                      : softmax_rows(stream, static_cast<double *>(scores), rows, columns, scale);
}

hipError_t launch_column_sums(hipStream_t stream, int dtype, bool mask, void *grad,
                              const void *activation, int rows, int columns, int chunks,
                              int chunk_rows, void *partial, void *sums)
{
    return dtype == 0
               ? column_sums(stream, mask, static_cast<float *>(grad),
                             static_cast<const float *>(activation), rows, columns, chunks,
                             chunk_rows, static_cast<float *>(partial), static_cast<float *>(sums))
               : column_sums(stream, mask, static_cast<double *>(grad),
                             static_cast<const double *>(activation), rows, columns, chunks,
                             chunk_rows, static_cast<double *>(partial), static_cast<double *>(sums));
}
} // namespace camblas_hip
