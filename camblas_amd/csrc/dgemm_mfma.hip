// FP64 column-major GEMM on the matrix cores: C = alpha * op(A) op(B) + beta * C for any transpose,
// leading dimension and alignment (v_mfma_f64_16x16x4_f64: IEEE double multiply-add).
// Contract: ref src/cuda/backend.cu:1066-1073 (validation is done by the caller in abi.hip).
//
// The structure of the FP32 kernel with the shapes of the FP64 instruction: a workgroup of four
// wavefronts owns a 128 x 128 tile of C, a wavefront 64 x 64 of it as 4 x 4 tiles of 16 x 16 (64
// accumulator doubles per lane). K is walked 16 deep: the operands of a step are loaded
// element-wise with bounds checks (every layout and ragged edge), kept in registers while the
// previous step is multiplied, and laid out in LDS so that the operand reads (lane -> row lane%16,
// K index lane/16) do not collide: K-major [16][128+16] for an operand whose rows are contiguous
// in memory, row-major [128][17] for a transposed one.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
typedef double f64x4_t __attribute__((ext_vector_type(4)));

constexpr int TILE = 128, DEPTH = 16, THREADS = 256;
struct BatchStrides {
    size_t a, b, c; // elements from one product of a batch to the next, per operand
};
constexpr int K_MAJOR_PITCH = TILE + 16, ROW_MAJOR_PITCH = DEPTH + 1;
constexpr int TILE_WORDS = DEPTH * K_MAJOR_PITCH; // >= TILE * ROW_MAJOR_PITCH
static_assert(TILE * ROW_MAJOR_PITCH <= TILE_WORDS, "one buffer serves both layouts");

// LDS index of element (row r of the tile, K index l) of an operand; CONTIGUOUS_K: K is the
// contiguous index in memory (a transposed A, an untransposed B)
template <bool CONTIGUOUS_K> __device__ __forceinline__ int lds_index(int r, int l)
{
    return CONTIGUOUS_K ? r * ROW_MAJOR_PITCH + l : l * K_MAJOR_PITCH + r;
}

// COLUMNS: 128, or 64 / 16 for a product with a handful of columns (the four wavefronts then stack
// along the rows, 32 x COLUMNS each; at 16 B brings one element per thread and step)
template <bool TA, bool TB, int COLUMNS>
__global__ __launch_bounds__(THREADS, 2) void dgemm_mfma_kernel(int m, int n, int k, double alpha,
                                                             const double *a, int lda, const double *b,
                                                             int ldb, double beta, double *c, int ldc,
                                                             BatchStrides batch_strides, bool lower_only)
{
    // a symmetric product: only the tiles that reach the diagonal, the rest is the mirroring pass
    int row0 = blockIdx.x * TILE, col0 = blockIdx.y * COLUMNS;
    if (COLUMNS == TILE && lower_only && !lower_tile<TILE, TILE>(blockIdx.x, n, row0, col0))
        return;
    a += blockIdx.z * batch_strides.a; // one independent product per grid z-slice
    b += blockIdx.z * batch_strides.b;
    c += blockIdx.z * batch_strides.c;
    __shared__ double tile_a[TILE_WORDS];
    __shared__ double tile_b[TILE_WORDS];
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    constexpr int PER_THREAD = TILE * DEPTH / THREADS, PER_THREAD_B = COLUMNS * DEPTH / THREADS;
    constexpr int WAVES_DOWN = COLUMNS == TILE ? 2 : 4;           // wavefronts along the rows
    constexpr int X = TILE / WAVES_DOWN / 16, Y = COLUMNS / (4 / WAVES_DOWN) / 16;
    // A(i, l) is a[i + l*lda] ('N', rows contiguous) or a[l + i*lda] ('T', K contiguous);
    // B(l, j) is b[l + j*ldb] ('N', K contiguous) or b[j + l*ldb] ('T', columns contiguous).
    // Element e of a step goes to the thread so that consecutive threads read consecutive memory.
    double next_a[PER_THREAD], next_b[PER_THREAD_B];
    auto fetch = [&](int l0) {
#pragma unroll
        for (int s = 0; s < PER_THREAD; ++s) {
            const int e = s * THREADS + thread;
            const int ai = TA ? e / DEPTH : e % TILE, al = TA ? e % DEPTH : e / TILE;
            const int gi = row0 + ai, gl = l0 + al;
            next_a[s] = gi < m && gl < k ? (TA ? a[gl + size_t(gi) * lda] : a[gi + size_t(gl) * lda]) : 0.0;
        }
#pragma unroll
        for (int s = 0; s < PER_THREAD_B; ++s) {
            const int e = s * THREADS + thread;
            const int bj = TB ? e % COLUMNS : e / DEPTH, bl = TB ? e / COLUMNS : e % DEPTH;
            const int gj = col0 + bj, hl = l0 + bl;
            next_b[s] = gj < n && hl < k ? (TB ? b[gj + size_t(hl) * ldb] : b[hl + size_t(gj) * ldb]) : 0.0;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int s = 0; s < PER_THREAD; ++s) {
            const int e = s * THREADS + thread;
            const int ai = TA ? e / DEPTH : e % TILE, al = TA ? e % DEPTH : e / TILE;
            tile_a[lds_index<TA>(ai, al)] = next_a[s];
        }
#pragma unroll
        for (int s = 0; s < PER_THREAD_B; ++s) {
            const int e = s * THREADS + thread;
            const int bj = TB ? e % COLUMNS : e / DEPTH, bl = TB ? e / COLUMNS : e % DEPTH;
            tile_b[lds_index<!TB>(bj, bl)] = next_b[s];
        }
    };

    const int wave_i = (wave % WAVES_DOWN) * (X * 16), wave_j = (wave / WAVES_DOWN) * (Y * 16);
    const int frag_row = lane % 16, frag_k = lane / 16;
    f64x4_t acc[X][Y];
#pragma unroll
    for (int x = 0; x < X; ++x)
#pragma unroll
        for (int y = 0; y < Y; ++y)
            acc[x][y] = f64x4_t{0.0, 0.0, 0.0, 0.0};

    fetch(0);
    for (int l0 = 0; l0 < k; l0 += DEPTH) {
        stash();
        __syncthreads();
        if (l0 + DEPTH < k)
            fetch(l0 + DEPTH);
#pragma unroll
        for (int s = 0; s < DEPTH / 4; ++s) {
            double av[X], bv[Y];
#pragma unroll
            for (int x = 0; x < X; ++x)
                av[x] = tile_a[lds_index<TA>(wave_i + x * 16 + frag_row, 4 * s + frag_k)];
#pragma unroll
            for (int y = 0; y < Y; ++y)
                bv[y] = tile_b[lds_index<!TB>(wave_j + y * 16 + frag_row, 4 * s + frag_k)];
#pragma unroll
            for (int x = 0; x < X; ++x)
#pragma unroll
                for (int y = 0; y < Y; ++y)
                    acc[x][y] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[x], bv[y], acc[x][y], 0, 0, 0);
        }
        __syncthreads();
    }

    // accumulator element e of lane l: row 4*e + l/16, column l%16 of the 16 x 16 tile (found with
    // an identity product; the FP32 16 x 16 instructions use 4*(l/16) + e instead)
#pragma unroll
    for (int y = 0; y < Y; ++y) {
        const int j = col0 + wave_j + y * 16 + frag_row;
        if (j >= n)
            continue;
#pragma unroll
        for (int x = 0; x < X; ++x) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int i = row0 + wave_i + x * 16 + 4 * e + frag_k;
                if (i >= m)
                    continue;
                double *out = c + i + size_t(j) * ldc;
                const double value = alpha * acc[x][y][e];
                *out = beta != 0.0 ? fma(beta, *out, value) : value;
            }
        }
    }
}
} // namespace

namespace
{
template <int COLUMNS>
hipError_t launch_tiles(hipStream_t stream, bool ta, bool tb, int m, int n, int k, double alpha,
                        const double *a, int lda, const double *b, int ldb, double beta, double *c, int ldc,
                        int batches, BatchStrides batch_stride, bool lower_only)
{
    if (batches < 1 || batches > 65535)
        return hipErrorInvalidValue;
    // column tiles travel in grid.y (at most 65535): wider products go panel by panel; the
    // lower-triangle grid is one-dimensional
    constexpr int PANEL = 65535 * COLUMNS;
    for (int first = 0; first < n; first += lower_only ? n : PANEL) {
        const int columns = lower_only ? n : (n - first < PANEL ? n - first : PANEL);
        const double *bp = b + (tb ? size_t(first) : size_t(first) * ldb);
        double *cp = c + size_t(first) * ldc;
        dim3 grid((m + TILE - 1) / TILE, (columns + COLUMNS - 1) / COLUMNS, batches);
        if (lower_only)
            grid = dim3(lower_tile_count<TILE, TILE>(n), 1, batches);
        if (!ta && !tb)
            dgemm_mfma_kernel<false, false, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, batch_stride, lower_only);
        else if (!ta && tb)
            dgemm_mfma_kernel<false, true, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, batch_stride, lower_only);
        else if (ta && !tb)
            dgemm_mfma_kernel<true, false, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, batch_stride, lower_only);
        else
            dgemm_mfma_kernel<true, true, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, batch_stride, lower_only);
        const hipError_t status = launch_status();
        if (status != hipSuccess)
            return status;
    }
    return hipSuccess;
}

// c = alpha * (sum of the planes, in plane order) + beta * c
__global__ __launch_bounds__(256) void sum_planes_f64_kernel(int m, int n, int shares, double alpha, double beta,
                                                             const double *planes, double *c, int ldc)
{
    const size_t count = size_t(m) * n, at = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (at >= count)
        return;
    double sum = planes[at];
    for (int s = 1; s < shares; ++s)
        sum += planes[s * count + at];
    double *out = c + at % m + at / m * ldc;
    const double value = alpha * sum;
    *out = beta != 0.0 ? fma(beta, *out, value) : value;
}
} // namespace

hipError_t launch_dgemm_mfma(hipStream_t stream, bool ta, bool tb, int m, int n, int k, double alpha,
                             const double *a, int lda, const double *b, int ldb, double beta, double *c,
                             int ldc, int batches, size_t batch_stride, bool lower_only)
{
    return launch_tiles<TILE>(stream, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, batches,
                              BatchStrides{batch_stride, batch_stride, batch_stride}, lower_only);
}

// The same product with K divided over `shares` workgroups per tile (k % shares == 0): for a
// handful of columns of C against a large A, where the tiles alone would occupy a fraction of the
// compute units. tile_columns: 128, 64 or 16 columns of C per tile. planes: shares * m * n doubles.
hipError_t launch_dgemm_mfma_divided(hipStream_t stream, bool ta, bool tb, int m, int n, int k, double alpha,
                                     const double *a, int lda, const double *b, int ldb, double beta,
                                     double *c, int ldc, int shares, double *planes, int tile_columns)
{
    if (shares < 2 || shares > 65535 || k % shares || !planes ||
        (tile_columns != 16 && tile_columns != 64 && tile_columns != TILE))
        return hipErrorInvalidValue;
    const int part = k / shares;
    const BatchStrides strides = {ta ? size_t(part) : size_t(part) * lda, tb ? size_t(part) * ldb : size_t(part),
                                  size_t(m) * n};
    const hipError_t status =
        tile_columns == 16
            ? launch_tiles<16>(stream, ta, tb, m, n, part, 1.0, a, lda, b, ldb, 0.0, planes, m, shares, strides, false)
        : tile_columns == 64
            ? launch_tiles<64>(stream, ta, tb, m, n, part, 1.0, a, lda, b, ldb, 0.0, planes, m, shares, strides, false)
            : launch_tiles<TILE>(stream, ta, tb, m, n, part, 1.0, a, lda, b, ldb, 0.0, planes, m, shares, strides, false);
    if (status != hipSuccess)
        return status;
    const size_t count = size_t(m) * n;
    if ((count + 255) / 256 > 0x7fffffffu)
        return hipErrorInvalidValue;
    sum_planes_f64_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(m, n, shares, alpha, beta, planes, c, ldc);
    return launch_status();
}
} // namespace camblas_hip
