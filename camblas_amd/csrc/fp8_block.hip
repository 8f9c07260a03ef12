// FP8 E4M3fn block-scaled linear out[M,N] = sum_g (a[M, g] . w[N, g]) * a_scale[M,g] * w_scale[N/128,g]
// with 1x128 activation groups and 128x128 weight blocks (FP32 scales), BF16 output.
//
// Arithmetic rule (ref: camblas/_hopper.py:118-126 and :168-182): per 128-wide K group the
// unscaled dot product in FP32 on the matrix cores, then acc = fma(dot_g, a_s * w_s, acc) for g
// ascending, with a_s * w_s rounded to FP32 first, and a single BF16 rounding at the end.
//
// One K tile is exactly one scale group (128 bytes per row), so the LDS geometry matches the BF16
// kernel: 8 chunks of 16 bytes per row, XOR-swizzled. A group's dot product is two
// v_mfma_scale_f32_32x32x64_f8f6f4 instructions (unit E8M0 scales: the hardware block scale is not
// used because the scales here are FP32 per 128) into a zeroed temporary; the scaled accumulate runs
// on the vector ALU while the matrix pipeline works on the next tile. With split-K each partition
// keeps the ordered chain over its own groups and partitions are added in index order.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
struct Fp8Params {
    const unsigned char *w;
    const unsigned char *a;
    const float *w_scale;
    const float *a_scale;
    unsigned short *out;
    float *partials;
    int n, m, k, groups, scale_blocks;
    int tiles_n, tiles_m, groups_per_split;
};

__device__ __forceinline__ int swizzle8(int row) { return ((row >> 1) & 7) ^ ((row & 1) << 2); }

// Weight bytes: a tile with at most 32 tokens belongs to a decode-sized call whose weights are read
// exactly once, so they are loaded non-temporally (they do not displace the activations and
// scales in the caches); larger token tiles re-read the weights through L2 and load them normally.
template <bool STREAMED> __device__ __forceinline__ u32x4_t weight_load(const unsigned char *address)
{
    if constexpr (STREAMED)
        return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(address));
    else
        return *reinterpret_cast<const u32x4_t *>(address);
}

template <int BN, int BM, int WN, int WM>
__global__ __launch_bounds__(WN *WM * 64) void fp8_block_kernel(Fp8Params p)
{
    constexpr int T = WN * WM * 64, CH = 8, BK = 128;
    constexpr int TN = BN / (WN * 32), TM = BM / (WM * 32);
    constexpr int A_ITERS = BN * CH / T, B_ITERS = BM * CH / T;
    constexpr int ROWS_PER_ITER = T / CH;
    constexpr int STAGE_SLOTS = (BN + BM) * CH;
    static_assert(BN % (WN * 32) == 0 && BM % (WM * 32) == 0, "wave tiling");
    static_assert((BN * CH) % T == 0 && (BM * CH) % T == 0, "load tiling");

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];
    u32x4_t *lds = reinterpret_cast<u32x4_t *>(lds_bytes);

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
    const int g_begin = blockIdx.y * p.groups_per_split;
    const int g_end = (g_begin + p.groups_per_split) < p.groups ? (g_begin + p.groups_per_split)
                                                                : p.groups;

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int wn = wave % WN, wm = wave / WN;
    const int chunk = thread % CH, row_in_iter = thread / CH;

    unsigned a_off[A_ITERS], b_off[B_ITERS];
    int a_slot[A_ITERS], b_slot[B_ITERS];
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
        int row = it * ROWS_PER_ITER + row_in_iter;
        int global_row = n0 + row < p.n ? n0 + row : p.n - 1;
        a_off[it] = unsigned(global_row - n0) * unsigned(p.k) + unsigned(chunk * 16);
        a_slot[it] = row * CH + (chunk ^ swizzle8(row));
    }
#pragma unroll
    for (int it = 0; it < B_ITERS; ++it) {
        int row = it * ROWS_PER_ITER + row_in_iter;
        int global_row = m0 + row < p.m ? m0 + row : p.m - 1;
        b_off[it] = unsigned(global_row - m0) * unsigned(p.k) + unsigned(chunk * 16);
        b_slot[it] = BN * CH + row * CH + (chunk ^ swizzle8(row));
    }
    const unsigned char *a_base = p.w + size_t(n0) * p.k;
    const unsigned char *b_base = p.a + size_t(m0) * p.k;

    // scale addresses: one activation scale per lane and token tile, one weight scale per wave and
    // feature tile (a 32-row tile never straddles a 128-row block)
    const int frag_row = lane % 32, half = lane / 32;
    const float *as_ptr[TM];
    const float *ws_ptr[TN];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        int m = m0 + (wm * TM + j) * 32 + frag_row;
        m = m < p.m ? m : p.m - 1;
        as_ptr[j] = p.a_scale + size_t(m) * p.groups;
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        int block = (n0 + (wn * TN + i) * 32) / 128;
        block = block < p.scale_blocks ? block : p.scale_blocks - 1;
        ws_ptr[i] = p.w_scale + size_t(block) * p.groups;
    }

    u32x4_t a_reg[A_ITERS], b_reg[B_ITERS];
    float as_next[TM], ws_next[TN];
    auto fetch = [&](int g) {
        const size_t k0 = size_t(g) * BK;
#pragma unroll
        for (int it = 0; it < A_ITERS; ++it)
            a_reg[it] = weight_load<BM <= 32>(a_base + k0 + a_off[it]);
#pragma unroll
        for (int it = 0; it < B_ITERS; ++it)
            b_reg[it] = *reinterpret_cast<const u32x4_t *>(b_base + k0 + b_off[it]);
#pragma unroll
        for (int j = 0; j < TM; ++j)
            as_next[j] = as_ptr[j][g];
#pragma unroll
        for (int i = 0; i < TN; ++i)
            ws_next[i] = ws_ptr[i][g];
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

    const int frag_swizzle = swizzle8(frag_row);
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

    constexpr int UNIT = 0x7f7f7f7f; // E8M0 exponent 127 = scale 1.0 in every byte
    auto multiply = [&](int stage, const float (&as_now)[TM], const float (&ws_now)[TN]) {
        const u32x4_t *base = lds + stage * STAGE_SLOTS;
        i32x8_t a_frag[TN][2], b_frag[TM][2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int c0 = (ks * 4 + half * 2) ^ frag_swizzle, c1 = (ks * 4 + half * 2 + 1) ^ frag_swizzle;
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                u32x4_t lo = base[a_frag_base + i * 32 * CH + c0];
                u32x4_t hi = base[a_frag_base + i * 32 * CH + c1];
                a_frag[i][ks] = i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                                        int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
            }
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                u32x4_t lo = base[b_frag_base + j * 32 * CH + c0];
                u32x4_t hi = base[b_frag_base + j * 32 * CH + c1];
                b_frag[j][ks] = i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                                        int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
            }
        }
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                f32x16_t dot;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    dot[r] = 0.f;
                dot = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    a_frag[i][0], b_frag[j][0], dot, 0, 0, 0, UNIT, 0, UNIT);
                dot = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    a_frag[i][1], b_frag[j][1], dot, 0, 0, 0, UNIT, 0, UNIT);
                const float scale = __fmul_rn(as_now[j], ws_now[i]);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = fmaf(dot[r], scale, acc[i][j][r]);
            }
    };

    if (g_end > g_begin) {
        float as_now[TM], ws_now[TN];
        fetch(g_begin);
        stash(0);
#pragma unroll
        for (int j = 0; j < TM; ++j)
            as_now[j] = as_next[j];
#pragma unroll
        for (int i = 0; i < TN; ++i)
            ws_now[i] = ws_next[i];
        __syncthreads();
        for (int g = g_begin; g < g_end; ++g) {
            const bool more = g + 1 < g_end;
            const int stage = (g - g_begin) & 1;
            if (more)
                fetch(g + 1);
            multiply(stage, as_now, ws_now);
            if (more) {
                stash(stage ^ 1);
#pragma unroll
                for (int j = 0; j < TM; ++j)
                    as_now[j] = as_next[j];
#pragma unroll
                for (int i = 0; i < TN; ++i)
                    ws_now[i] = ws_next[i];
            }
            __syncthreads();
        }
    }

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
                unsigned short *out = p.out + size_t(m) * p.n + n;
                if (n + 3 < p.n && (p.n & 3) == 0) {
                    u32x2_t packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                    *reinterpret_cast<u32x2_t *>(out) = packed;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < p.n)
                            out[e] = float_to_bf16_bits(v[e]);
                }
            }
        }
}

__global__ void fp8_splitk_reduce_kernel(size_t count, int splits, const float *partials,
                                         unsigned short *out)
{
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= count)
        return;
    float sum = partials[index];
    for (int s = 1; s < splits; ++s)
        sum += partials[size_t(s) * count + index];
    out[index] = float_to_bf16_bits(sum);
}

// Dynamic 1x128 quantiser (ref: camblas/_hopper.py:82-98). Sixteen lanes own one group (8 values
// each); four groups per wavefront.
__global__ __launch_bounds__(256) void fp8_quantise_kernel(int rows, int inner,
                                                           const unsigned short *x,
                                                           unsigned char *q, float *scale)
{
    const int groups = inner / 128;
    const size_t group = (size_t(blockIdx.x) * 256 + threadIdx.x) / 16;
    const int part = threadIdx.x % 16;
    if (group >= size_t(rows) * groups)
        return; // whole 16-lane clusters leave together; the shuffles below stay inside a cluster
    const size_t offset = group * 128 + size_t(part) * 8;
    u32x4_t raw = *reinterpret_cast<const u32x4_t *>(x + offset);
    float v[8];
    float amax = 1e-10f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(raw[e] << 16);
        v[2 * e + 1] = __uint_as_float(raw[e] & 0xffff0000u);
        amax = fmaxf(amax, fmaxf(fabsf(v[2 * e]), fabsf(v[2 * e + 1])));
    }
#pragma unroll
    for (int offset_lane = 8; offset_lane; offset_lane >>= 1)
        amax = fmaxf(amax, __shfl_xor(amax, offset_lane, 64));
    const float inv = 448.0f / amax;
    unsigned packed[2] = {0u, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float scaled = fminf(fmaxf(v[e] * inv, -448.f), 448.f);
        packed[e / 4] |= f32_to_e4m3_sat(scaled) << (8 * (e % 4));
    }
    u32x2_t store = {packed[0], packed[1]};
    *reinterpret_cast<u32x2_t *>(q + offset) = store;
    if (part == 0)
        scale[group] = amax * (1.0f / 448.0f);
}

template <int BN, int BM, int WN, int WM>
hipError_t launch_variant(hipStream_t stream, const Fp8Params &p, int split_k)
{
    constexpr size_t lds_bytes = size_t(2) * (BN + BM) * 128;
    auto kernel = fp8_block_kernel<BN, BM, WN, WM>;
    static LdsLimitFlags limits; // (one per instantiation)
    const hipError_t status = raise_lds_limit(limits, reinterpret_cast<const void *>(kernel), lds_bytes);
    if (status != hipSuccess)
        return status;
    dim3 grid(unsigned(p.tiles_n) * unsigned(p.tiles_m), unsigned(split_k));
    kernel<<<grid, WN * WM * 64, lds_bytes, stream>>>(p);
    return launch_status();
}

const TnVariant variants[] = {
    {"fp8mfma128x128x128", 128, 128, 128, 256},
    {"fp8mfma128x32x128", 128, 32, 128, 256},
    {"fp8mfma256x128x128", 256, 128, 128, 256},
    {"fp8mfma64x32x128", 64, 32, 128, 128},
};
} // namespace

int fp8_variant_count() { return int(sizeof(variants) / sizeof(variants[0])); }
const TnVariant &fp8_variant(int index) { return variants[index]; }

hipError_t launch_fp8_block(hipStream_t stream, int variant, int split_k, int rows, int outputs,
                            int inner, const void *a, const float *a_scale, const void *w,
                            const float *w_scale, void *out, float *partials)
{
    if (variant < 0 || variant >= fp8_variant_count() || split_k < 1 || split_k > 65535)
        return hipErrorInvalidValue;
    if (size_t(outputs) * size_t(inner) > 0xffffffffu && outputs > (1 << 22))
        return hipErrorInvalidValue;
    const TnVariant &v = variants[variant];
    Fp8Params p;
    p.w = static_cast<const unsigned char *>(w);
    p.a = static_cast<const unsigned char *>(a);
    p.w_scale = w_scale;
    p.a_scale = a_scale;
    p.out = static_cast<unsigned short *>(out);
    p.partials = partials;
    p.n = outputs;
    p.m = rows;
    p.k = inner;
    p.groups = inner / 128;
    p.scale_blocks = (outputs + 127) / 128;
    p.tiles_n = (outputs + v.block_n - 1) / v.block_n;
    p.tiles_m = (rows + v.block_m - 1) / v.block_m;
    int per_split = (p.groups + split_k - 1) / split_k;
    split_k = (p.groups + per_split - 1) / per_split;
    p.groups_per_split = per_split;
    if (split_k > 1 && !partials)
        return hipErrorInvalidValue;
    hipError_t status;
    switch (variant) {
    case 0: status = launch_variant<128, 128, 2, 2>(stream, p, split_k); break;
    case 1: status = launch_variant<128, 32, 4, 1>(stream, p, split_k); break;
    case 2: status = launch_variant<256, 128, 2, 2>(stream, p, split_k); break;
    default: status = launch_variant<64, 32, 2, 1>(stream, p, split_k); break;
    }
    if (status != hipSuccess || split_k == 1)
        return status;
    return launch_fp8_split_sum(stream, split_k, size_t(rows) * outputs, partials, out);
}

// out[i] = bf16(partials[0][i] + partials[1][i] + ...), planes of `count` FP32 sums in index order
hipError_t launch_fp8_split_sum(hipStream_t stream, int splits, size_t count, const float *partials, void *out)
{
    fp8_splitk_reduce_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(
        count, splits, partials, static_cast<unsigned short *>(out));
    return launch_status();
}

hipError_t launch_fp8_quantise(hipStream_t stream, int rows, int inner, const void *x, void *q,
                               float *scale)
{
    size_t clusters = size_t(rows) * (inner / 128);
    unsigned blocks = unsigned((clusters * 16 + 255) / 256);
    fp8_quantise_kernel<<<blocks, 256, 0, stream>>>(rows, inner,
                                                    static_cast<const unsigned short *>(x),
                                                    static_cast<unsigned char *>(q), scale);
    return launch_status();
}
} // namespace camblas_hip
