// Generic column-major GEMM for any transpose, leading dimension and alignment: 64x64 output tile,
// K staged 16 deep through LDS, 256 threads with a 4x4 register micro-tile each. FP32 and FP64
// run in their own precision (plain FMA, no reduced-precision matrix path); BF16 storage
// accumulates in FP32 and rounds once. It serves FP32 SGEMM and is the fallback for every BF16
// call the MFMA path does not accept.
// Contract: ref src/cuda/backend.cu:786-866 (FP32/FP64), src/cuda/bfloat16.cuh:11-57 (BF16).
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int TILE = 64, DEPTH = 16, THREADS = 256;

// beta-only update: C <- beta*C, beta==0 stores zero without reading
// (ref: src/cuda/backend.cu:88-95, src/cuda/bfloat16.cuh:2-9).
template <typename T>
__global__ void scale_kernel(int m, int n, typename storage<T>::accumulator beta, T *c, int ldc)
{
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= size_t(m) * n)
        return;
    T *out = c + index % m + (index / m) * size_t(ldc);
    using acc_t = typename storage<T>::accumulator;
    storage<T>::store(out, beta == acc_t(0) ? acc_t(0) : beta * storage<T>::load(out));
}

// c[i + j*ldc] = z[i + j*ldz], 2-byte elements; ldz == 0 repeats one column
__global__ void spread_kernel(int m, int n, const unsigned short *z, int ldz, unsigned short *c, int ldc)
{
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= size_t(m) * n)
        return;
    c[index % m + (index / m) * size_t(ldc)] = z[index % m + (index / m) * size_t(ldz)];
}

// TA/TB: operand stored transposed. A tile element (i, l) is a[i + l*lda] (N) or a[l + i*lda] (T);
// the thread->element map makes the memory-contiguous index the fastest-varying lane index.
template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(THREADS) void generic_kernel(int m, int n, int k,
                                                          typename storage<T>::accumulator alpha,
                                                          const T *a, int lda, const T *b, int ldb,
                                                          typename storage<T>::accumulator beta,
                                                          T *c, int ldc)
{
    using acc_t = typename storage<T>::accumulator;
    __shared__ acc_t tile_a[DEPTH][TILE + 4];
    __shared__ acc_t tile_b[DEPTH][TILE + 4];
    const int thread = threadIdx.x;
    const int row0 = blockIdx.x * TILE, col0 = blockIdx.y * TILE;
    const int ti = thread % 16, tj = thread / 16;
    acc_t acc[4][4] = {};
    for (int l0 = 0; l0 < k; l0 += DEPTH) {
#pragma unroll
        for (int step = 0; step < TILE * DEPTH / THREADS; ++step) {
            int index = step * THREADS + thread;
            // A: 'N' -> i fastest; 'T' -> l fastest
            int ai = TA ? index / DEPTH : index % TILE, al = TA ? index % DEPTH : index / TILE;
            int gi = row0 + ai, gl = l0 + al;
            acc_t value = 0;
            if (gi < m && gl < k)
                value = storage<T>::load(TA ? a + gl + size_t(gi) * lda : a + gi + size_t(gl) * lda);
            tile_a[al][ai] = value;
            // B(l, j): 'N' -> b[l + j*ldb] (l fastest); 'T' -> b[j + l*ldb] (j fastest)
            int bj = TB ? index % TILE : index / DEPTH, bl = TB ? index / TILE : index % DEPTH;
            int gj = col0 + bj;
            gl = l0 + bl;
            value = 0;
            if (gj < n && gl < k)
                value = storage<T>::load(TB ? b + gj + size_t(gl) * ldb : b + gl + size_t(gj) * ldb);
            tile_b[bl][bj] = value;
        }
        __syncthreads();
#pragma unroll
        for (int l = 0; l < DEPTH; ++l) {
            acc_t av[4], bv[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                av[x] = tile_a[l][ti * 4 + x];
                bv[x] = tile_b[l][tj * 4 + x];
            }
#pragma unroll
            for (int y = 0; y < 4; ++y)
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    acc[y][x] = fma(av[x], bv[y], acc[y][x]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int y = 0; y < 4; ++y) {
        int j = col0 + tj * 4 + y;
        if (j >= n)
            continue;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            int i = row0 + ti * 4 + x;
            if (i >= m)
                continue;
            T *out = c + i + size_t(j) * ldc;
            acc_t value = alpha * acc[y][x];
            if (beta != acc_t(0))
                value = fma(beta, acc_t(storage<T>::load(out)), value);
            storage<T>::store(out, value);
        }
    }
}

template <typename T>
hipError_t launch_generic(hipStream_t stream, bool ta, bool tb, int m, int n, int k,
                          typename storage<T>::accumulator alpha, const T *a, int lda, const T *b,
                          int ldb, typename storage<T>::accumulator beta, T *c, int ldc)
{
    // column tiles travel in grid.y (at most 65535): wider products go panel by panel
    constexpr int PANEL = 65535 * TILE;
    for (int first = 0; first < n; first += PANEL) {
        const int columns = n - first < PANEL ? n - first : PANEL;
        const T *bp = b + (tb ? size_t(first) : size_t(first) * ldb);
        T *cp = c + size_t(first) * ldc;
        const dim3 grid((m + TILE - 1) / TILE, (columns + TILE - 1) / TILE);
        if (!ta && !tb)
            generic_kernel<T, false, false>
                <<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc);
        else if (!ta && tb)
            generic_kernel<T, false, true>
                <<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc);
        else if (ta && !tb)
            generic_kernel<T, true, false>
                <<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc);
        else
            generic_kernel<T, true, true>
                <<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc);
        const hipError_t status = launch_status();
        if (status != hipSuccess)
            return status;
    }
    return hipSuccess;
}
} // namespace

hipError_t launch_scale_f32(hipStream_t stream, int m, int n, float beta, float *c, int ldc)
{
    scale_kernel<float>
        <<<unsigned((size_t(m) * n + 255) / 256), 256, 0, stream>>>(m, n, beta, c, ldc);
    return launch_status();
}

hipError_t launch_scale_f64(hipStream_t stream, int m, int n, double beta, double *c, int ldc)
{
    scale_kernel<double>
        <<<unsigned((size_t(m) * n + 255) / 256), 256, 0, stream>>>(m, n, beta, c, ldc);
    return launch_status();
}

hipError_t launch_scale_bf16(hipStream_t stream, int m, int n, float beta, void *c, int ldc)
{
    scale_kernel<bf16_storage><<<unsigned((size_t(m) * n + 255) / 256), 256, 0, stream>>>(
        m, n, beta, static_cast<bf16_storage *>(c), ldc);
    return launch_status();
}

hipError_t launch_spread_bf16(hipStream_t stream, int m, int n, const void *z, int ldz, void *c, int ldc)
{
    spread_kernel<<<unsigned((size_t(m) * n + 255) / 256), 256, 0, stream>>>(
        m, n, static_cast<const unsigned short *>(z), ldz, static_cast<unsigned short *>(c), ldc);
    return launch_status();
}

hipError_t launch_generic_f32(hipStream_t stream, bool ta, bool tb, int m, int n, int k, float alpha,
                              const float *a, int lda, const float *b, int ldb, float beta, float *c,
                              int ldc)
{
    return launch_generic<float>(stream, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

hipError_t launch_generic_f64(hipStream_t stream, bool ta, bool tb, int m, int n, int k,
                              double alpha, const double *a, int lda, const double *b, int ldb,
                              double beta, double *c, int ldc)
{
    return launch_generic<double>(stream, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

hipError_t launch_generic_bf16(hipStream_t stream, bool ta, bool tb, int m, int n, int k,
                               float alpha, const void *a, int lda, const void *b, int ldb,
                               float beta, void *c, int ldc)
{
    return launch_generic<bf16_storage>(stream, ta, tb, m, n, k, alpha,
                                        static_cast<const bf16_storage *>(a), lda,
                                        static_cast<const bf16_storage *>(b), ldb, beta,
                                        static_cast<bf16_storage *>(c), ldc);
}
} // namespace camblas_hip
