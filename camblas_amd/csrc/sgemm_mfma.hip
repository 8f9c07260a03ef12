// FP32 column-major GEMM on the matrix cores: C = alpha * op(A) op(B) + beta * C for any transpose,
// leading dimension and alignment, full FP32 arithmetic (v_mfma_f32_32x32x2_f32 multiplies and
// accumulates IEEE single precision; there is no reduced-precision path).
// Contract: ref src/cuda/backend.cu:786-866 (validation is done by the caller in abi.hip).
//
// A workgroup of four wavefronts owns a 128 x 128 tile of C, a wavefront 64 x 64 of it as 2 x 2
// MFMA tiles (64 accumulator registers). K is walked 32 deep: the operands of a step are loaded
// element-wise with bounds checks (that is what makes every layout and ragged edge work), kept in
// registers while the previous step is multiplied, and laid out in LDS so that the operand reads
// (lane -> row lane%32, K index lane/32) are conflict-free: K-major [32][128+32] for an operand
// whose rows are contiguous in memory, row-major [128][33] for a transposed one.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int TILE = 128, DEPTH = 32, THREADS = 256;
struct BatchStrides {
    size_t a, b, c; // elements from one product of a batch to the next, per operand
};
constexpr int K_MAJOR_PITCH = TILE + 32, ROW_MAJOR_PITCH = DEPTH + 1;
constexpr int TILE_WORDS = DEPTH * K_MAJOR_PITCH; // >= TILE * ROW_MAJOR_PITCH
static_assert(TILE * ROW_MAJOR_PITCH <= TILE_WORDS, "one buffer serves both layouts");

// LDS word of element (row r of the tile, K index l) of an operand; CONTIGUOUS_K: K is the
// contiguous index in memory (a transposed A, an untransposed B)
template <bool CONTIGUOUS_K> __device__ __forceinline__ int lds_word(int r, int l)
{
    return CONTIGUOUS_K ? r * ROW_MAJOR_PITCH + l : l * K_MAJOR_PITCH + r;
}

// COLUMNS: 128 or 64 columns of C per workgroup (64: twice the workgroups, for products whose
// 128 x 128 tiles would leave one workgroup per compute unit with nothing to overlap with), or 32
// for a handful of columns with K divided (the four wavefronts then stack along the rows)
template <bool TA, bool TB, int COLUMNS>
__global__ __launch_bounds__(THREADS) void sgemm_mfma_kernel(int m, int n, int k, float alpha,
                                                             const float *a, int lda, const float *b,
                                                             int ldb, float beta, float *c, int ldc,
                                                             BatchStrides strides, bool lower_only)
{
    // a symmetric product: only the tiles that reach the diagonal, the rest is the mirroring pass
    int row0 = blockIdx.x * TILE, col0 = blockIdx.y * COLUMNS;
    if (lower_only && !lower_tile<TILE, COLUMNS>(blockIdx.x, n, row0, col0))
        return;
    a += blockIdx.z * strides.a; // one independent product per grid z-slice
    b += blockIdx.z * strides.b;
    c += blockIdx.z * strides.c;
    __shared__ float tile_a[TILE_WORDS];
    __shared__ float tile_b[TILE_WORDS];
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    constexpr int A_PER_THREAD = TILE * DEPTH / THREADS, B_PER_THREAD = COLUMNS * DEPTH / THREADS;
    constexpr int WAVES_DOWN = COLUMNS >= 64 ? 2 : 4;             // wavefronts along the rows
    constexpr int WI = TILE / WAVES_DOWN / 32;                    // 32-row MFMA tiles per wavefront
    constexpr int WJ = COLUMNS / (4 / WAVES_DOWN) / 32;           // 32-column MFMA tiles per wavefront
    // A(i, l) is a[i + l*lda] ('N', rows contiguous) or a[l + i*lda] ('T', K contiguous);
    // B(l, j) is b[l + j*ldb] ('N', K contiguous) or b[j + l*ldb] ('T', columns contiguous).
    // Element e of a step goes to the thread so that consecutive threads read consecutive memory.
    float next_a[A_PER_THREAD], next_b[B_PER_THREAD];
    auto fetch = [&](int l0) {
#pragma unroll
        for (int s = 0; s < A_PER_THREAD; ++s) {
            const int e = s * THREADS + thread;
            const int ai = TA ? e / DEPTH : e % TILE, al = TA ? e % DEPTH : e / TILE;
            const int gi = row0 + ai, gl = l0 + al;
            next_a[s] = gi < m && gl < k ? (TA ? a[gl + size_t(gi) * lda] : a[gi + size_t(gl) * lda]) : 0.f;
        }
#pragma unroll
        for (int s = 0; s < B_PER_THREAD; ++s) {
            const int e = s * THREADS + thread;
            const int bj = TB ? e % COLUMNS : e / DEPTH, bl = TB ? e / COLUMNS : e % DEPTH;
            const int gj = col0 + bj, hl = l0 + bl;
            next_b[s] = gj < n && hl < k ? (TB ? b[gj + size_t(hl) * ldb] : b[hl + size_t(gj) * ldb]) : 0.f;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int s = 0; s < A_PER_THREAD; ++s) {
            const int e = s * THREADS + thread;
            const int ai = TA ? e / DEPTH : e % TILE, al = TA ? e % DEPTH : e / TILE;
            tile_a[lds_word<TA>(ai, al)] = next_a[s];
        }
#pragma unroll
        for (int s = 0; s < B_PER_THREAD; ++s) {
            const int e = s * THREADS + thread;
            const int bj = TB ? e % COLUMNS : e / DEPTH, bl = TB ? e / COLUMNS : e % DEPTH;
            tile_b[lds_word<!TB>(bj, bl)] = next_b[s];
        }
    };

    const int wave_i = (wave % WAVES_DOWN) * (32 * WI), wave_j = (wave / WAVES_DOWN) * (32 * WJ);
    const int frag_row = lane % 32, frag_k = lane / 32;
    f32x16_t acc[WI][WJ];
#pragma unroll
    for (int x = 0; x < WI; ++x)
#pragma unroll
        for (int y = 0; y < WJ; ++y)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[x][y][r] = 0.f;

    fetch(0);
    for (int l0 = 0; l0 < k; l0 += DEPTH) {
        stash();
        __syncthreads();
        if (l0 + DEPTH < k)
            fetch(l0 + DEPTH);
#pragma unroll
        for (int s = 0; s < DEPTH / 2; ++s) {
            float av[WI], bv[WJ];
#pragma unroll
            for (int x = 0; x < WI; ++x)
                av[x] = tile_a[lds_word<TA>(wave_i + x * 32 + frag_row, 2 * s + frag_k)];
#pragma unroll
            for (int y = 0; y < WJ; ++y)
                bv[y] = tile_b[lds_word<!TB>(wave_j + y * 32 + frag_row, 2 * s + frag_k)];
#pragma unroll
            for (int x = 0; x < WI; ++x)
#pragma unroll
                for (int y = 0; y < WJ; ++y)
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[x], bv[y], acc[x][y], 0, 0, 0);
        }
        __syncthreads();
    }

    // accumulator register 4q+e of lane l: row 8q + 4*(l/32) + e, column l%32 of the 32 x 32 tile;
    // the four rows of a q are contiguous in column-major C
    const bool vector = ldc % 4 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0;
#pragma unroll
    for (int y = 0; y < WJ; ++y) {
        const int j = col0 + wave_j + y * 32 + frag_row;
        if (j >= n)
            continue;
#pragma unroll
        for (int x = 0; x < WI; ++x) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int i = row0 + wave_i + x * 32 + 8 * q + 4 * frag_k;
                if (i >= m)
                    continue;
                float *out = c + i + size_t(j) * ldc;
                float value[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    value[e] = alpha * acc[x][y][4 * q + e];
                if (vector && i + 3 < m) {
                    if (beta != 0.f) {
                        const f32x4_t old = *reinterpret_cast<const f32x4_t *>(out);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            value[e] = fmaf(beta, old[e], value[e]);
                    }
                    *reinterpret_cast<f32x4_t *>(out) = f32x4_t{value[0], value[1], value[2], value[3]};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (i + e >= m)
                            break;
                        out[e] = beta != 0.f ? fmaf(beta, out[e], value[e]) : value[e];
                    }
                }
            }
        }
    }
}

template <int COLUMNS>
hipError_t launch_columns(hipStream_t stream, bool ta, bool tb, int m, int n, int k, float alpha,
                          const float *a, int lda, const float *b, int ldb, float beta, float *c, int ldc,
                          int batches, BatchStrides strides, bool lower_only)
{
    if (batches < 1 || batches > 65535)
        return hipErrorInvalidValue;
    // The column tiles travel in grid.y (at most 65535): wider products are launched as panels of
    // that many tiles, each on its own columns of B and C. The lower-triangle grid is one-dimensional.
    constexpr int PANEL = 65535 * COLUMNS;
    for (int first = 0; first < n; first += lower_only ? n : PANEL) {
        const int columns = lower_only ? n : (n - first < PANEL ? n - first : PANEL);
        const float *bp = b + (tb ? size_t(first) : size_t(first) * ldb);
        float *cp = c + size_t(first) * ldc;
        dim3 grid((m + TILE - 1) / TILE, (columns + COLUMNS - 1) / COLUMNS, batches);
        if (lower_only)
            grid = dim3(lower_tile_count<TILE, COLUMNS>(n), 1, batches);
        if (!ta && !tb)
            sgemm_mfma_kernel<false, false, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, strides, lower_only);
        else if (!ta && tb)
            sgemm_mfma_kernel<false, true, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, strides, lower_only);
        else if (ta && !tb)
            sgemm_mfma_kernel<true, false, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, strides, lower_only);
        else
            sgemm_mfma_kernel<true, true, COLUMNS><<<grid, THREADS, 0, stream>>>(m, columns, k, alpha, a, lda, bp, ldb, beta, cp, ldc, strides, lower_only);
        const hipError_t status = launch_status();
        if (status != hipSuccess)
            return status;
    }
    return hipSuccess;
}
} // namespace

// wide: 128 x 128 tiles, else 128 x 64
hipError_t launch_sgemm_mfma(hipStream_t stream, bool wide, bool ta, bool tb, int m, int n, int k,
                             float alpha, const float *a, int lda, const float *b, int ldb, float beta,
                             float *c, int ldc, int batches, size_t batch_stride, bool lower_only)
{
    const BatchStrides strides = {batch_stride, batch_stride, batch_stride};
    return wide ? launch_columns<128>(stream, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, batches,
                                      strides, lower_only)
                : launch_columns<64>(stream, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, batches,
                                     strides, lower_only);
}

namespace
{
// c = alpha * (plane 0 + plane 1 + ...) + beta * c over the shares of a divided K, planes [share][n][m]
// added in index order so that the result does not depend on scheduling.
__global__ __launch_bounds__(256) void sum_planes_f32_kernel(int m, int n, int shares, float alpha, float beta,
                                                             const float *planes, float *c, int ldc)
{
    const size_t index = size_t(blockIdx.x) * 256 + threadIdx.x, count = size_t(m) * n;
    if (index >= count)
        return;
    float sum = planes[index];
    for (int share = 1; share < shares; ++share)
        sum += planes[size_t(share) * count + index];
    float *out = c + (index / m) * size_t(ldc) + index % m;
    const float value = alpha * sum;
    *out = beta != 0.f ? fmaf(beta, *out, value) : value;
}
} // namespace

// The same product with K divided over `shares` workgroups per 128 x 64 tile (narrow: 128 x 32;
// k % shares == 0): for a handful of columns of C against a large A, where the tiles alone would
// occupy a fraction of the compute units. planes: shares * m * n floats.
hipError_t launch_sgemm_mfma_divided(hipStream_t stream, bool ta, bool tb, int m, int n, int k, float alpha,
                                     const float *a, int lda, const float *b, int ldb, float beta, float *c,
                                     int ldc, int shares, float *planes, bool narrow)
{
    if (shares < 2 || shares > 65535 || k % shares || !planes)
        return hipErrorInvalidValue;
    const int part = k / shares;
    const BatchStrides strides = {ta ? size_t(part) : size_t(part) * lda, tb ? size_t(part) * ldb : size_t(part),
                                  size_t(m) * n};
    const hipError_t status =
        narrow ? launch_columns<32>(stream, ta, tb, m, n, part, 1.f, a, lda, b, ldb, 0.f, planes, m, shares, strides, false)
               : launch_columns<64>(stream, ta, tb, m, n, part, 1.f, a, lda, b, ldb, 0.f, planes, m, shares, strides, false);
    if (status != hipSuccess)
        return status;
    const size_t count = size_t(m) * n;
    if ((count + 255) / 256 > 0x7fffffffu)
        return hipErrorInvalidValue;
    sum_planes_f32_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(m, n, shares, alpha, beta, planes, c, ldc);
    return launch_status();
}
} // namespace camblas_hip
