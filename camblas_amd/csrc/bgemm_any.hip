// BF16 column-major GEMM on the matrix cores for the layouts the K-contiguous kernels do not take:
// C = alpha * op(A) op(B) + beta * C with BF16 storage, FP32 accumulation and one rounding, for any
// transpose pair, leading dimension, alignment and ragged edge (contract: ref
// src/cuda/bfloat16.cuh:11-57; the reference sends every transpose pair to tensor-core GEMMs). These
// are the products a row-major torch.mm(x, w) with a contiguous [in, out] weight and the backward
// products dx = g W, dW = x^T g arrive as.
//
// A workgroup of four wavefronts owns 128 x COLUMNS of C, a wavefront 64 x (COLUMNS / 2) as 32 x 32
// tiles of v_mfma_f32_32x32x16_bf16. K is walked 32 deep. Both operands sit in LDS with K
// contiguous ([row][32 + 8] BF16: the 80-byte pitch makes the 16-byte operand reads of eight
// consecutive rows hit eight different bank groups), whatever their order in memory: an operand
// whose K index is contiguous in memory is copied 16 bytes at a time, one whose rows are contiguous
// is loaded 16 bytes (eight rows of one K index) at a time and scattered. Operands that are not
// 16-byte aligned, or whose leading dimension is not a multiple of eight, take element loads.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int TILE = 128, DEPTH = 32, THREADS = 256, PITCH = DEPTH + 8;

// ROWS rows of an operand for K indices l0 .. l0+31 into `tile` ([row][PITCH]); K_CONTIGUOUS: element
// (row r, K index l) is base[l + r * ld], else base[r + l * ld]. Rows >= limit and K >= k read as 0.
template <int ROWS, bool K_CONTIGUOUS, bool VECTOR> struct OperandStage {
    static constexpr int VECTORS = ROWS * DEPTH / 8 / THREADS, ELEMENTS = ROWS * DEPTH / THREADS;
    u32x4_t vectors[VECTOR ? VECTORS : 1];
    unsigned short elements[VECTOR ? 1 : ELEMENTS];

    __device__ __forceinline__ static unsigned short element(const unsigned short *base, int ld, int r, int l,
                                                             int limit, int k)
    {
        if (r >= limit || l >= k)
            return 0;
        return K_CONTIGUOUS ? base[l + size_t(r) * ld] : base[r + size_t(l) * ld];
    }

    __device__ __forceinline__ void fetch(const unsigned short *base, int ld, int row0, int limit, int l0, int k,
                                          int thread)
    {
        if constexpr (VECTOR) {
#pragma unroll
            for (int s = 0; s < VECTORS; ++s) {
                const int v = s * THREADS + thread;
                // K contiguous: vector v is K indices 8 (v % 4) .. of row v / 4; else rows 8 (v % (ROWS/8)) ..
                // of K index v / (ROWS / 8)
                const int r = K_CONTIGUOUS ? v / (DEPTH / 8) : (v % (ROWS / 8)) * 8;
                const int l = K_CONTIGUOUS ? (v % (DEPTH / 8)) * 8 : v / (ROWS / 8);
                const int gr = row0 + r, gl = l0 + l;
                const bool whole = K_CONTIGUOUS ? (gr < limit && gl + 7 < k) : (gr + 7 < limit && gl < k);
                if (whole) {
                    const unsigned short *source =
                        K_CONTIGUOUS ? base + gl + size_t(gr) * ld : base + gr + size_t(gl) * ld;
                    vectors[s] = *reinterpret_cast<const u32x4_t *>(source);
                } else {
                    unsigned short e[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        e[i] = K_CONTIGUOUS ? element(base, ld, gr, gl + i, limit, k)
                                            : element(base, ld, gr + i, gl, limit, k);
                    vectors[s] = u32x4_t{e[0] | unsigned(e[1]) << 16, e[2] | unsigned(e[3]) << 16,
                                         e[4] | unsigned(e[5]) << 16, e[6] | unsigned(e[7]) << 16};
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < ELEMENTS; ++s) {
                const int e = s * THREADS + thread;
                const int r = K_CONTIGUOUS ? e / DEPTH : e % ROWS, l = K_CONTIGUOUS ? e % DEPTH : e / ROWS;
                elements[s] = element(base, ld, row0 + r, l0 + l, limit, k);
            }
        }
    }

    __device__ __forceinline__ void stash(unsigned short *tile, int thread) const
    {
        if constexpr (VECTOR) {
#pragma unroll
            for (int s = 0; s < VECTORS; ++s) {
                const int v = s * THREADS + thread;
                if constexpr (K_CONTIGUOUS) {
                    const int r = v / (DEPTH / 8), l = (v % (DEPTH / 8)) * 8;
                    *reinterpret_cast<u32x4_t *>(tile + r * PITCH + l) = vectors[s];
                } else {
                    const int r = (v % (ROWS / 8)) * 8, l = v / (ROWS / 8);
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        tile[(r + i) * PITCH + l] = (unsigned short)(vectors[s][i / 2] >> (16 * (i % 2)));
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < ELEMENTS; ++s) {
                const int e = s * THREADS + thread;
                const int r = K_CONTIGUOUS ? e / DEPTH : e % ROWS, l = K_CONTIGUOUS ? e % DEPTH : e / ROWS;
                tile[r * PITCH + l] = elements[s];
            }
        }
    }
};

template <bool TA, bool TB, int COLUMNS, bool VECTOR>
__global__ __launch_bounds__(THREADS) void bgemm_any_kernel(int m, int n, int k, float alpha,
                                                            const unsigned short *a, int lda,
                                                            const unsigned short *b, int ldb, float beta,
                                                            unsigned short *c, int ldc, int row_tiles)
{
    // one-dimensional grid: the row tile is the fast index (neither dimension is capped at 65535)
    const int row0 = int(blockIdx.x % unsigned(row_tiles)) * TILE;
    const int col0 = int(blockIdx.x / unsigned(row_tiles)) * COLUMNS;
    __shared__ __attribute__((aligned(16))) unsigned short tile_a[TILE * PITCH];
    __shared__ __attribute__((aligned(16))) unsigned short tile_b[COLUMNS * PITCH];
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    constexpr int WJ = COLUMNS / 64; // 32-column tiles per wavefront
    // A(i, l) is a[l + i*lda] when transposed (K contiguous); B(l, j) is b[l + j*ldb] when not
    OperandStage<TILE, TA, VECTOR> stage_a;
    OperandStage<COLUMNS, !TB, VECTOR> stage_b;

    const int wave_i = (wave % 2) * 64, wave_j = (wave / 2) * (32 * WJ);
    const int frag_row = lane % 32, frag_k = (lane / 32) * 8;
    f32x16_t acc[2][WJ];
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < WJ; ++y)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[x][y][r] = 0.f;

    stage_a.fetch(a, lda, row0, m, 0, k, thread);
    stage_b.fetch(b, ldb, col0, n, 0, k, thread);
    for (int l0 = 0; l0 < k; l0 += DEPTH) {
        stage_a.stash(tile_a, thread);
        stage_b.stash(tile_b, thread);
        __syncthreads();
        if (l0 + DEPTH < k) { // the next step's operands travel while this one is multiplied
            stage_a.fetch(a, lda, row0, m, l0 + DEPTH, k, thread);
            stage_b.fetch(b, ldb, col0, n, l0 + DEPTH, k, thread);
        }
#pragma unroll
        for (int s = 0; s < DEPTH / 16; ++s) {
            bf16x8_t av[2], bv[WJ];
#pragma unroll
            for (int x = 0; x < 2; ++x)
                av[x] = *reinterpret_cast<const bf16x8_t *>(tile_a + (wave_i + x * 32 + frag_row) * PITCH +
                                                            16 * s + frag_k);
#pragma unroll
            for (int y = 0; y < WJ; ++y)
                bv[y] = *reinterpret_cast<const bf16x8_t *>(tile_b + (wave_j + y * 32 + frag_row) * PITCH +
                                                            16 * s + frag_k);
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int y = 0; y < WJ; ++y)
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[x], bv[y], acc[x][y], 0, 0, 0);
        }
        __syncthreads();
    }

    // accumulator register 4q+e of lane l: row 8q + 4*(l/32) + e, column l%32 of the 32 x 32 tile;
    // the four rows of a q are contiguous in column-major C
    const bool vector = ldc % 4 == 0 && reinterpret_cast<uintptr_t>(c) % 8 == 0;
#pragma unroll
    for (int y = 0; y < WJ; ++y) {
        const int j = col0 + wave_j + y * 32 + frag_row;
        if (j >= n)
            continue;
#pragma unroll
        for (int x = 0; x < 2; ++x) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int i = row0 + wave_i + x * 32 + 8 * q + 4 * (lane / 32);
                if (i >= m)
                    continue;
                unsigned short *out = c + i + size_t(j) * ldc;
                float value[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    value[e] = alpha * acc[x][y][4 * q + e];
                if (vector && i + 3 < m) {
                    if (beta != 0.f) {
                        const u32x2_t old = *reinterpret_cast<const u32x2_t *>(out);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            value[e] = fmaf(beta, bf16_bits_to_float((unsigned short)(old[e / 2] >> (16 * (e % 2)))),
                                            value[e]);
                    }
                    *reinterpret_cast<u32x2_t *>(out) =
                        u32x2_t{pack_bf16x2(value[0], value[1]), pack_bf16x2(value[2], value[3])};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (i + e >= m)
                            break;
                        const float sum = beta != 0.f ? fmaf(beta, bf16_bits_to_float(out[e]), value[e]) : value[e];
                        out[e] = float_to_bf16_bits(sum);
                    }
                }
            }
        }
    }
}

template <bool TA, bool TB, int COLUMNS>
hipError_t launch_layout(hipStream_t stream, bool vector, dim3 grid, int m, int n, int k, float alpha,
                         const unsigned short *a, int lda, const unsigned short *b, int ldb, float beta,
                         unsigned short *c, int ldc, int row_tiles)
{
    if (vector)
        bgemm_any_kernel<TA, TB, COLUMNS, true>
            <<<grid, THREADS, 0, stream>>>(m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, row_tiles);
    else
        bgemm_any_kernel<TA, TB, COLUMNS, false>
            <<<grid, THREADS, 0, stream>>>(m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, row_tiles);
    return launch_status();
}

template <int COLUMNS>
hipError_t launch_columns(hipStream_t stream, bool ta, bool tb, int m, int n, int k, float alpha,
                          const unsigned short *a, int lda, const unsigned short *b, int ldb, float beta,
                          unsigned short *c, int ldc)
{
    const long long row_tiles = (m + TILE - 1) / TILE, column_tiles = (n + COLUMNS - 1) / COLUMNS;
    if (row_tiles * column_tiles > 0x7fffffffLL)
        return hipErrorInvalidValue;
    const dim3 grid(unsigned(row_tiles * column_tiles), 1, 1);
    const bool vector = lda % 8 == 0 && ldb % 8 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 &&
                        reinterpret_cast<uintptr_t>(b) % 16 == 0;
    if (!ta && !tb)
        return launch_layout<false, false, COLUMNS>(stream, vector, grid, m, n, k, alpha, a, lda, b, ldb, beta, c,
                                                    ldc, int(row_tiles));
    if (!ta && tb)
        return launch_layout<false, true, COLUMNS>(stream, vector, grid, m, n, k, alpha, a, lda, b, ldb, beta, c,
                                                   ldc, int(row_tiles));
    if (ta && !tb)
        return launch_layout<true, false, COLUMNS>(stream, vector, grid, m, n, k, alpha, a, lda, b, ldb, beta, c,
                                                   ldc, int(row_tiles));
    return launch_layout<true, true, COLUMNS>(stream, vector, grid, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc,
                                              int(row_tiles));
}
// dst[c * ld_dst + r] = src[r * ld_src + c] for a 2-byte element matrix of `rows` strided rows and
// `cols` contiguous columns: 64 x 64 tiles through LDS, 8-byte global accesses on both sides when
// VECTOR (tile rows start 8-byte aligned on both sides), else element by element. The LDS pitch of
// 65 elements makes both the row-wise writes and the column-wise reads conflict-poor.
template <bool VECTOR>
__global__ __launch_bounds__(256) void transpose_bf16_kernel(int rows, int cols, const unsigned short *src,
                                                              int ld_src, unsigned short *dst, int ld_dst,
                                                              int col_tiles)
{
    constexpr int TILE = 64, PITCH = TILE + 1;
    __shared__ unsigned short tile[TILE * PITCH];
    const int r0 = int(blockIdx.x / col_tiles) * TILE, c0 = int(blockIdx.x % col_tiles) * TILE;
    const int thread = threadIdx.x, quad = thread % 16, line = thread / 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = line + 16 * i, c = quad * 4;
        unsigned short v[4] = {0, 0, 0, 0};
        if (r0 + r < rows) {
            const unsigned short *from = src + size_t(r0 + r) * ld_src + c0 + c;
            if (VECTOR && c0 + c + 3 < cols) {
                const u32x2_t packed = *reinterpret_cast<const u32x2_t *>(from);
                v[0] = packed[0] & 0xffffu, v[1] = packed[0] >> 16, v[2] = packed[1] & 0xffffu, v[3] = packed[1] >> 16;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (c0 + c + e < cols)
                        v[e] = from[e];
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
            tile[r * PITCH + c + e] = v[e];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = line + 16 * i, r = quad * 4; // output row c0 + c, output columns r0 + r ..
        if (c0 + c >= cols)
            continue;
        unsigned short v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            v[e] = tile[(r + e) * PITCH + c];
        unsigned short *to = dst + size_t(c0 + c) * ld_dst + r0 + r;
        if (VECTOR && r0 + r + 3 < rows) {
            *reinterpret_cast<u32x2_t *>(to) = u32x2_t{unsigned(v[0]) | unsigned(v[1]) << 16,
                                                       unsigned(v[2]) | unsigned(v[3]) << 16};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (r0 + r + e < rows)
                    to[e] = v[e];
        }
    }
}
} // namespace

hipError_t launch_transpose_bf16(hipStream_t stream, int rows, int cols, const void *src, int ld_src, void *dst,
                                 int ld_dst)
{
    const size_t row_tiles = (size_t(rows) + 63) / 64, col_tiles = (size_t(cols) + 63) / 64;
    if (rows < 1 || cols < 1 || row_tiles * col_tiles > 0x7fffffffu)
        return hipErrorInvalidValue;
    const bool vector = ld_src % 4 == 0 && ld_dst % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 8 == 0 &&
                        reinterpret_cast<uintptr_t>(dst) % 8 == 0;
    const unsigned short *from = static_cast<const unsigned short *>(src);
    unsigned short *to = static_cast<unsigned short *>(dst);
    const unsigned grid = unsigned(row_tiles * col_tiles);
    if (vector)
        transpose_bf16_kernel<true><<<grid, 256, 0, stream>>>(rows, cols, from, ld_src, to, ld_dst, int(col_tiles));
    else
        transpose_bf16_kernel<false><<<grid, 256, 0, stream>>>(rows, cols, from, ld_src, to, ld_dst, int(col_tiles));
    return launch_status();
}

// wide: 128 x 128 tiles, else 128 x 64
hipError_t launch_bgemm_any(hipStream_t stream, bool wide, bool ta, bool tb, int m, int n, int k, float alpha,
                            const void *a, int lda, const void *b, int ldb, float beta, void *c, int ldc)
{
    const unsigned short *ap = static_cast<const unsigned short *>(a);
    const unsigned short *bp = static_cast<const unsigned short *>(b);
    unsigned short *cp = static_cast<unsigned short *>(c);
    return wide ? launch_columns<128>(stream, ta, tb, m, n, k, alpha, ap, lda, bp, ldb, beta, cp, ldc)
                : launch_columns<64>(stream, ta, tb, m, n, k, alpha, ap, lda, bp, ldb, beta, cp, ldc);
}
} // namespace camblas_hip
