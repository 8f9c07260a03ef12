// BF16 linear y[M,N] = alpha * x[M,K] * W[N,K]^T + beta * y on gfx950 matrix cores.
//
// This is the shape every linear arrives in (camblas_cuda_bgemm 'T','N', m=N outputs, n=M tokens;
// ref: src/cuda/torch_bindings.cpp:146-199, src/cuda/bfloat16.cuh:11-57): both operands are
// K-contiguous, the output is row-major [M, N]. One templated kernel covers the compute-bound
// prefill tiles (256x256 .. 128x128) and the bandwidth-bound decode tiles (128x32, 64x32 with
// deep K and split-K); the planner picks the variant.
//
// Data movement: every thread fetches 16-byte chunks (8 BF16 along K) with 128-byte-contiguous
// groups of 8 lanes, holds the next K tile in registers while the current one is multiplied, and
// stores it into an XOR-swizzled LDS tile so that both the 128-bit stores and the 128-bit
// MFMA-layout reads are bank-conflict free. Each wavefront owns a (TN x TM) grid of 32x32 MFMA
// accumulators (v_mfma_f32_32x32x16_bf16, FP32 accumulate). W rows are the MFMA "A" operand so a
// lane ends up with four consecutive output features and writes them as one 8-byte store.
// Workgroups are renumbered so that each XCD (own L2) receives a contiguous, 2-D compact block of
// output tiles.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
struct TnParams {
    const unsigned short *w;
    const unsigned short *x;
    unsigned short *y;
    float *partials;
    int lda, ldb, ldc;
    int n, m, k;
    float alpha, beta;
    int tiles_n, tiles_m, k_per_split;
    int vector_store; // y (and z) rows allow 8-byte accesses (ldc, ldz % 4 == 0, 8-byte aligned)
    const unsigned short *z; // what beta multiplies: z[token * ldz + feature] (y and ldc by default)
    int ldz;
};

// XOR applied to the 16-byte chunk index inside an LDS row. With CH chunks per row the pattern
// keeps any 8 consecutive rows (and any 16 consecutive rows when the LDS has 64 banks) on
// distinct banks for a fixed logical chunk.
template <int CH> __device__ __forceinline__ int swizzle(int row)
{
    if constexpr (CH == 8)
        return ((row >> 1) & 7) ^ ((row & 1) << 2);
    else if constexpr (CH == 16)
        return row & 15;
    else
        return 0;
}

template <int BN, int BM, int BK, int WN, int WM, int STAGES>
__global__ __launch_bounds__(WN *WM * 64) void bgemm_tn_kernel(TnParams p)
{
    constexpr int T = WN * WM * 64, CH = BK / 8;
    constexpr int TN = BN / (WN * 32), TM = BM / (WM * 32);
    constexpr int A_ITERS = BN * CH / T, B_ITERS = BM * CH / T;
    constexpr int ROWS_PER_ITER = T / CH;
    constexpr int STAGE_SLOTS = (BN + BM) * CH;
    static_assert(BN % (WN * 32) == 0 && BM % (WM * 32) == 0, "wave tiling");
    static_assert((BN * CH) % T == 0 && (BM * CH) % T == 0 && T % CH == 0, "load tiling");
    static_assert(CH == 8 || CH == 16, "swizzle defined for 64- and 128-deep tiles");

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];
    u32x4_t *lds = reinterpret_cast<u32x4_t *>(lds_bytes);

    // ---- workgroup -> output tile (XCD-contiguous, grouped along N for L2 reuse)
    const int total = p.tiles_n * p.tiles_m;
    int logical;
    {
        int b = blockIdx.x, per = total / 8, rem = total % 8, xcd = b % 8, local = b / 8;
        logical = xcd * per + (xcd < rem ? xcd : rem) + local;
    }
    constexpr int GROUP = 8;
    const int span = GROUP * p.tiles_m;
    const int first_n = (logical / span) * GROUP;
    const int group_size = (p.tiles_n - first_n) < GROUP ? (p.tiles_n - first_n) : GROUP;
    const int tile_n = first_n + (logical % span) % group_size;
    const int tile_m = (logical % span) / group_size;
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int k_begin = blockIdx.y * p.k_per_split;
    const int k_end = (k_begin + p.k_per_split) < p.k ? (k_begin + p.k_per_split) : p.k;
    const int k_tiles = (k_end - k_begin + BK - 1) / BK;

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int wn = wave % WN, wm = wave / WN;

    // ---- global -> LDS descriptors: chunk column is fixed per thread, rows advance per iteration
    const int chunk = thread % CH, row_in_iter = thread / CH;
    unsigned a_off[A_ITERS], b_off[B_ITERS];
    int a_slot[A_ITERS], b_slot[B_ITERS];
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
        int row = it * ROWS_PER_ITER + row_in_iter;
        int global_row = n0 + row < p.n ? n0 + row : p.n - 1;
        a_off[it] = unsigned(global_row - n0) * unsigned(p.lda) + unsigned(chunk * 8);
        a_slot[it] = row * CH + (chunk ^ swizzle<CH>(row));
    }
#pragma unroll
    for (int it = 0; it < B_ITERS; ++it) {
        int row = it * ROWS_PER_ITER + row_in_iter;
        int global_row = m0 + row < p.m ? m0 + row : p.m - 1;
        b_off[it] = unsigned(global_row - m0) * unsigned(p.ldb) + unsigned(chunk * 8);
        b_slot[it] = BN * CH + row * CH + (chunk ^ swizzle<CH>(row));
    }
    // (global_row - n0) may be negative only when the tile starts past the matrix, which the grid
    // never produces; the unsigned product then stays inside the operand.
    const unsigned short *a_base = p.w + size_t(n0) * p.lda + k_begin;
    const unsigned short *b_base = p.x + size_t(m0) * p.ldb + k_begin;

    u32x4_t a_reg[A_ITERS], b_reg[B_ITERS];
    auto fetch = [&](int tile) {
        const int k0 = tile * BK;
        const bool valid = k_begin + k0 + chunk * 8 < k_end;
#pragma unroll
        for (int it = 0; it < A_ITERS; ++it) {
            u32x4_t value = {0u, 0u, 0u, 0u};
            if (valid)
                value = *reinterpret_cast<const u32x4_t *>(a_base + k0 + a_off[it]);
            a_reg[it] = value;
        }
#pragma unroll
        for (int it = 0; it < B_ITERS; ++it) {
            u32x4_t value = {0u, 0u, 0u, 0u};
            if (valid)
                value = *reinterpret_cast<const u32x4_t *>(b_base + k0 + b_off[it]);
            b_reg[it] = value;
        }
    };
    auto stash = [&](int stage) {
        u32x4_t *base = lds + stage * STAGE_SLOTS;
#pragma unroll
        for (int it = 0; it < A_ITERS; ++it)
            base[a_slot[it]] = a_reg[it];
#pragma unroll
        for (int it = 0; it < B_ITERS; ++it)
            base[b_slot[it]] = b_reg[it];
    };

    // ---- MFMA-layout read positions: lane -> row (lane % 32), K half (lane / 32)
    const int frag_row = lane % 32, half = lane / 32;
    const int frag_swizzle = swizzle<CH>(frag_row);
    const int a_frag_base = (wn * TN * 32 + frag_row) * CH;
    const int b_frag_base = BN * CH + (wm * TM * 32 + frag_row) * CH;

    f32x16_t acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    auto multiply = [&](int stage) {
        const u32x4_t *base = lds + stage * STAGE_SLOTS;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const int column = (ks * 2 + half) ^ frag_swizzle;
            bf16x8_t a_frag[TN], b_frag[TM];
#pragma unroll
            for (int i = 0; i < TN; ++i)
                a_frag[i] = __builtin_bit_cast(bf16x8_t, base[a_frag_base + i * 32 * CH + column]);
#pragma unroll
            for (int j = 0; j < TM; ++j)
                b_frag[j] = __builtin_bit_cast(bf16x8_t, base[b_frag_base + j * 32 * CH + column]);
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_frag[i], b_frag[j],
                                                                        acc[i][j], 0, 0, 0);
        }
    };

    if (k_tiles > 0) {
        fetch(0);
        stash(0);
        __syncthreads();
        for (int tile = 0; tile < k_tiles; ++tile) {
            const bool more = tile + 1 < k_tiles;
            if constexpr (STAGES == 2) {
                if (more)
                    fetch(tile + 1);
                multiply(tile & 1);
                if (more)
                    stash((tile + 1) & 1);
                __syncthreads();
            } else {
                if (more)
                    fetch(tile + 1);
                multiply(0);
                __syncthreads();
                if (more)
                    stash(0);
                __syncthreads();
            }
        }
    }

    // ---- epilogue. Accumulator register r of lane l holds output feature
    // n = 8*(r/4) + 4*(l/32) + r%4 and token m = l%32 inside its 32x32 tile.
    const bool split = gridDim.y > 1;
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const int m = m0 + (wm * TM + j) * 32 + frag_row;
            if (m >= p.m)
                continue;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + (wn * TN + i) * 32 + q * 8 + half * 4;
                if (n >= p.n)
                    continue;
                float v[4] = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                              acc[i][j][q * 4 + 3]};
                if (split) {
                    float *out = p.partials + (size_t(blockIdx.y) * p.m + m) * p.n + n;
                    if (n + 3 < p.n && (p.n & 3) == 0) {
                        f32x4_t packed = {v[0], v[1], v[2], v[3]};
                        *reinterpret_cast<f32x4_t *>(out) = packed;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < p.n)
                                out[e] = v[e];
                    }
                    continue;
                }
                unsigned short *out = p.y + size_t(m) * p.ldc + n;
                const unsigned short *source = p.z + size_t(m) * p.ldz + n;
                if (n + 3 < p.n && p.vector_store) {
                    if (p.beta != 0.f) {
                        u32x2_t old = *reinterpret_cast<const u32x2_t *>(source);
                        v[0] = fmaf(p.beta, __uint_as_float(old[0] << 16), p.alpha * v[0]);
                        v[1] = fmaf(p.beta, __uint_as_float(old[0] & 0xffff0000u), p.alpha * v[1]);
                        v[2] = fmaf(p.beta, __uint_as_float(old[1] << 16), p.alpha * v[2]);
                        v[3] = fmaf(p.beta, __uint_as_float(old[1] & 0xffff0000u), p.alpha * v[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] *= p.alpha;
                    }
                    u32x2_t packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                    *reinterpret_cast<u32x2_t *>(out) = packed;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e >= p.n)
                            break;
                        float value = p.alpha * v[e];
                        if (p.beta != 0.f)
                            value = fmaf(p.beta, bf16_bits_to_float(source[e]), value);
                        out[e] = float_to_bf16_bits(value);
                    }
                }
            }
        }
}

// Ordered split-K reduction: y = alpha * (p_0 + p_1 + ...) + beta * z, partials added in index
// order so the result does not depend on scheduling.
__global__ void splitk_reduce_kernel(int m, int n, int splits, float alpha, float beta,
                                     const float *partials, unsigned short *y, int ldc,
                                     const unsigned short *z, int ldz)
{
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t count = size_t(m) * n;
    if (index >= count)
        return;
    float sum = partials[index];
    for (int s = 1; s < splits; ++s)
        sum += partials[size_t(s) * count + index];
    unsigned short *out = y + (index / n) * size_t(ldc) + index % n;
    float value = alpha * sum;
    if (beta != 0.f)
        value = fmaf(beta, bf16_bits_to_float(z[(index / n) * size_t(ldz) + index % n]), value);
    *out = float_to_bf16_bits(value);
}

template <int BN, int BM, int BK, int WN, int WM, int STAGES>
hipError_t launch_variant(hipStream_t stream, const TnParams &p, int split_k)
{
    constexpr size_t lds_bytes = size_t(STAGES) * (BN + BM) * BK * 2;
    auto kernel = bgemm_tn_kernel<BN, BM, BK, WN, WM, STAGES>;
    static LdsLimitFlags limits; // (one per instantiation)
    const hipError_t status = raise_lds_limit(limits, reinterpret_cast<const void *>(kernel), lds_bytes);
    if (status != hipSuccess)
        return status;
    dim3 grid(unsigned(p.tiles_n) * unsigned(p.tiles_m), unsigned(split_k));
    kernel<<<grid, WN * WM * 64, lds_bytes, stream>>>(p);
    return launch_status();
}

const TnVariant variants[] = {
    {"mfma256x256x64", 256, 256, 64, 256}, {"mfma256x128x64", 256, 128, 64, 256},
    {"mfma128x128x64", 128, 128, 64, 256}, {"mfma128x64x64", 128, 64, 64, 256},
    {"mfma128x32x64", 128, 32, 64, 256},   {"mfma128x32x128", 128, 32, 128, 256},
    {"mfma64x32x128", 64, 32, 128, 128},   {"mfma64x32x64", 64, 32, 64, 128},
};
} // namespace

int tn_variant_count() { return int(sizeof(variants) / sizeof(variants[0])); }
const TnVariant &tn_variant(int index) { return variants[index]; }

hipError_t launch_bgemm_tn(hipStream_t stream, int variant, int split_k, int n_out, int m_rows,
                           int k, float alpha, const void *w, int lda, const void *x, int ldb,
                           float beta, void *y, int ldc, float *partials, const BetaSource &source)
{
    if (variant < 0 || variant >= tn_variant_count() || split_k < 1 || split_k > 65535)
        return hipErrorInvalidValue;
    const TnVariant &v = variants[variant];
    TnParams p;
    p.w = static_cast<const unsigned short *>(w);
    p.x = static_cast<const unsigned short *>(x);
    p.y = static_cast<unsigned short *>(y);
    p.partials = partials;
    p.lda = lda;
    p.ldb = ldb;
    p.ldc = ldc;
    p.n = n_out;
    p.m = m_rows;
    p.k = k;
    p.alpha = alpha;
    p.beta = beta;
    p.tiles_n = (n_out + v.block_n - 1) / v.block_n;
    p.tiles_m = (m_rows + v.block_m - 1) / v.block_m;
    int k_tiles = (k + v.block_k - 1) / v.block_k;
    int tiles_per_split = (k_tiles + split_k - 1) / split_k;
    split_k = (k_tiles + tiles_per_split - 1) / tiles_per_split; // no empty partitions
    p.k_per_split = tiles_per_split * v.block_k;
    p.z = source.z ? static_cast<const unsigned short *>(source.z) : p.y;
    p.ldz = source.z ? source.ldz : ldc;
    p.vector_store = ldc % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 8 == 0 && p.ldz % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(p.z) % 8 == 0;
    if (split_k > 1 && !partials)
        return hipErrorInvalidValue;
    if (size_t(p.tiles_n) * size_t(p.tiles_m) > 0x7fffffffu)
        return hipErrorInvalidValue;
    hipError_t status;
    switch (variant) {
    case 0: status = launch_variant<256, 256, 64, 2, 2, 2>(stream, p, split_k); break;
    case 1: status = launch_variant<256, 128, 64, 2, 2, 2>(stream, p, split_k); break;
    case 2: status = launch_variant<128, 128, 64, 2, 2, 2>(stream, p, split_k); break;
    case 3: status = launch_variant<128, 64, 64, 4, 1, 2>(stream, p, split_k); break;
    case 4: status = launch_variant<128, 32, 64, 4, 1, 2>(stream, p, split_k); break;
    case 5: status = launch_variant<128, 32, 128, 4, 1, 2>(stream, p, split_k); break;
    case 6: status = launch_variant<64, 32, 128, 2, 1, 2>(stream, p, split_k); break;
    default: status = launch_variant<64, 32, 64, 2, 1, 2>(stream, p, split_k); break;
    }
    if (status != hipSuccess || split_k == 1)
        return status;
    size_t count = size_t(m_rows) * n_out;
    splitk_reduce_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(
        m_rows, n_out, split_k, alpha, beta, partials, static_cast<unsigned short *>(y), ldc, p.z, p.ldz);
    return launch_status();
}
} // namespace camblas_hip
