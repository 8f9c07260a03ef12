// FP8 E4M3fn block-scaled prefill linear (1x128 activation groups, 128x128 weight blocks, FP32
// scales, BF16 out) on the gfx950 matrix cores, operands streamed straight into LDS.
//
// Arithmetic rule (ref: camblas/_hopper.py:118-126 and :168-182): per 128-wide K group the
// unscaled FP32 dot product on the matrix cores, then acc = fma(dot_g, a_s * w_s, acc) for g
// ascending with a_s * w_s rounded to FP32 first, one BF16 rounding at the end.
//
// A workgroup of 2 x WM wavefronts owns a 256 x (32*WM*TM) output tile; each wavefront owns 128
// weight rows (exactly one 128-row scale block) by 32*TM tokens. One K step is one scale group:
// 128 bytes per row, the same LDS geometry (8 chunks of 16 bytes, XOR swizzle) as a 64-deep BF16
// step, two stages filled by buffer_load ... lds. A group's dot product is two
// v_mfma_scale_f32_32x32x64_f8f6f4 (unit hardware scales) into a zeroed temporary; the scaled
// accumulate of one 32x32 tile runs on the vector ALU while the matrix cores work on the next tile.
// Weight scales for 64 consecutive groups are fetched with one coalesced load and broadcast with
// v_readlane, activation scales are one 4-byte load per lane, token tile and step, fetched a step
// ahead.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
struct Fp8DmaParams {
    const unsigned char *w;
    const unsigned char *a;
    const float *w_scale;
    const float *a_scale;
    unsigned short *out;
    int n, m, k, groups, scale_blocks;
    int tiles_n, tiles_m;
};

template <int TM, int WM>
__global__ __launch_bounds__(128 * WM) void fp8_dma_kernel(Fp8DmaParams p)
{
    constexpr int TN = 4, WAVES = 2 * WM, CH = 8, BK = 128;
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    constexpr int ROWS_PER_LOAD = 8;
    constexpr int A_ITERS = BN / (WAVES * ROWS_PER_LOAD), B_ITERS = BM / (WAVES * ROWS_PER_LOAD);
    constexpr int SLOTS = (BN + BM) * CH;
    static_assert(BN % (WAVES * ROWS_PER_LOAD) == 0 && BM % (WAVES * ROWS_PER_LOAD) == 0, "loads");
    __shared__ u32x4_t stage0[SLOTS];
    __shared__ u32x4_t stage1[SLOTS];

    int tile_n, tile_m;
    xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int wn = wave % 2, wm = wave / 2;

    unsigned a_off[A_ITERS], b_off[B_ITERS];
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
        int row = (it * WAVES + wave) * ROWS_PER_LOAD + lane / CH;
        int chunk = (lane % CH) ^ lds_swizzle<CH>(row);
        int global_row = n0 + row < p.n ? n0 + row : p.n - 1;
        a_off[it] = unsigned(global_row - n0) * unsigned(p.k) + unsigned(chunk * 16);
    }
#pragma unroll
    for (int it = 0; it < B_ITERS; ++it) {
        int row = (it * WAVES + wave) * ROWS_PER_LOAD + lane / CH;
        int chunk = (lane % CH) ^ lds_swizzle<CH>(row);
        int global_row = m0 + row < p.m ? m0 + row : p.m - 1;
        b_off[it] = unsigned(global_row - m0) * unsigned(p.k) + unsigned(chunk * 16);
    }
    const int a_rows = p.n - n0 < BN ? p.n - n0 : BN, b_rows = p.m - m0 < BM ? p.m - m0 : BM;
    const __amdgpu_buffer_rsrc_t a_resource =
        make_resource(p.w + size_t(n0) * p.k, unsigned(a_rows) * unsigned(p.k));
    const __amdgpu_buffer_rsrc_t b_resource =
        make_resource(p.a + size_t(m0) * p.k, unsigned(b_rows) * unsigned(p.k));
    const unsigned last_k_bytes = unsigned(p.groups - 1) * BK;
    unsigned k_bytes = 0;
    auto issue = [&](u32x4_t *stage) {
#pragma unroll
        for (int it = 0; it < A_ITERS; ++it)
            load_to_lds(a_resource, a_off[it], k_bytes, stage + (it * WAVES + wave) * 64);
#pragma unroll
        for (int it = 0; it < B_ITERS; ++it)
            load_to_lds(b_resource, b_off[it], k_bytes, stage + BN * CH + (it * WAVES + wave) * 64);
        k_bytes = k_bytes + BK < last_k_bytes ? k_bytes + BK : last_k_bytes;
    };

    // ---- scales. The wavefront's 128 weight rows lie in one scale block: lane l holds the scale
    // of group (64*window + l); v_readlane broadcasts the current one. Activation scales: one per
    // lane (token = lane % 32) and token tile, loaded one step ahead.
    const int frag_row = lane % 32, half = lane / 32;
    int block = (n0 + wn * 128) / 128;
    block = block < p.scale_blocks ? block : p.scale_blocks - 1;
    const float *ws_row = p.w_scale + size_t(block) * p.groups;
    auto load_ws = [&](int window) {
        int g = window * 64 + lane;
        return ws_row[g < p.groups ? g : p.groups - 1];
    };
    const float *as_ptr[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        int m = m0 + (wm * TM + j) * 32 + frag_row;
        m = m < p.m ? m : p.m - 1;
        as_ptr[j] = p.a_scale + size_t(m) * p.groups;
    }

    const int frag_swizzle = lds_swizzle<CH>(frag_row);
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
    auto fragment = [&](const u32x4_t *stage, int base, int ks) {
        u32x4_t lo = stage[base + ((ks * 4 + half * 2) ^ frag_swizzle)];
        u32x4_t hi = stage[base + ((ks * 4 + half * 2 + 1) ^ frag_swizzle)];
        return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                       int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
    };
    // One K group. All fragments are read first; then the tiles are walked in a software pipeline:
    // the two MFMAs of tile t+1 are issued before the 16 scaled accumulates of tile t, so the vector
    // ALU work of one tile runs while the matrix cores execute the next (sched_barrier pins it).
    auto multiply = [&](const u32x4_t *stage, const float (&as_now)[TM], float ws_now) {
        i32x8_t a_frag[TN][2], b_frag[TM][2];
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            b_frag[j][0] = fragment(stage, b_frag_base + j * 32 * CH, 0);
            b_frag[j][1] = fragment(stage, b_frag_base + j * 32 * CH, 1);
        }
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            a_frag[i][0] = fragment(stage, a_frag_base + i * 32 * CH, 0);
            a_frag[i][1] = fragment(stage, a_frag_base + i * 32 * CH, 1);
        }
        float scale[TM];
#pragma unroll
        for (int j = 0; j < TM; ++j)
            scale[j] = __fmul_rn(as_now[j], ws_now);
        f32x16_t dot[2];
        auto product = [&](int tile, f32x16_t &d) {
            const int i = tile / TM, j = tile % TM;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                d[r] = 0.f;
            d = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_frag[i][0], b_frag[j][0], d, 0, 0,
                                                                0, UNIT, 0, UNIT);
            d = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_frag[i][1], b_frag[j][1], d, 0, 0,
                                                                0, UNIT, 0, UNIT);
        };
        auto accumulate = [&](int tile, const f32x16_t &d) {
            const int i = tile / TM, j = tile % TM;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = fmaf(d[r], scale[j], acc[i][j][r]);
        };
        __builtin_amdgcn_sched_barrier(0);
        product(0, dot[0]);
#pragma unroll
        for (int tile = 1; tile < TN * TM; ++tile) {
            __builtin_amdgcn_sched_barrier(0);
            product(tile, dot[tile & 1]);
            __builtin_amdgcn_sched_barrier(0);
            accumulate(tile - 1, dot[(tile - 1) & 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
        accumulate(TN * TM - 1, dot[(TN * TM - 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
    };

    float ws_window = load_ws(0);
    float as_now[TM], as_next[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j)
        as_now[j] = as_ptr[j][0];
    issue(stage0);
    wait_loads<0>();
    __syncthreads();
    for (int g = 0; g < p.groups; g += 2) {
        // even group: stage0 is current
        {
            const int next = g + 1 < p.groups ? g + 1 : p.groups - 1;
#pragma unroll
            for (int j = 0; j < TM; ++j)
                as_next[j] = as_ptr[j][next];
            __builtin_amdgcn_sched_barrier(0);
            issue(stage1);
            __builtin_amdgcn_sched_barrier(0);
            float ws_now = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ws_window), g & 63));
            multiply(stage0, as_now, ws_now);
            wait_loads<0>();
            __syncthreads();
        }
        if (g + 1 < p.groups) {
            const int next = g + 2 < p.groups ? g + 2 : p.groups - 1;
#pragma unroll
            for (int j = 0; j < TM; ++j)
                as_now[j] = as_ptr[j][next];
            __builtin_amdgcn_sched_barrier(0);
            issue(stage0);
            __builtin_amdgcn_sched_barrier(0);
            float ws_now = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ws_window), (g + 1) & 63));
            multiply(stage1, as_next, ws_now);
            if (((g + 2) & 63) == 0) // the next group starts a new window of 64 weight scales
                ws_window = load_ws((g + 2) / 64);
            wait_loads<0>();
            __syncthreads();
        }
    }
    wait_loads<0>();

    // ---- epilogue: accumulator register 4q+e of lane l is feature 8q + 4*(l/32) + e, token l%32
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + (wm * TM + j) * 32 + frag_row;
        unsigned short *row = p.out + size_t(m) * p.n + n0 + wn * TN * 32 + half * 4;
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int offset = i * 32 + q * 8;
                if (m < p.m && n0 + wn * TN * 32 + half * 4 + offset < p.n) {
                    u32x2_t packed = {pack_bf16x2(acc[i][j][q * 4], acc[i][j][q * 4 + 1]),
                                      pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3])};
                    *reinterpret_cast<u32x2_t *>(row + offset) = packed;
                }
            }
        }
    }
}

template <int TM, int WM> hipError_t launch_one(hipStream_t stream, Fp8DmaParams p)
{
    constexpr int BN = 256, BM = 32 * WM * TM;
    p.tiles_n = (p.n + BN - 1) / BN;
    p.tiles_m = (p.m + BM - 1) / BM;
    if (size_t(p.tiles_n) * size_t(p.tiles_m) > 0x7fffffffu)
        return hipErrorInvalidValue;
    fp8_dma_kernel<TM, WM><<<unsigned(p.tiles_n) * unsigned(p.tiles_m), 128 * WM, 0, stream>>>(p);
    return launch_status();
}

const TnVariant variants[] = {
    {"fp8dma256x256x128w8", 256, 256, 128, 512},
    {"fp8dma256x128x128w8", 256, 128, 128, 512},
    {"fp8dma256x128x128w4", 256, 128, 128, 256},
    {"fp8dma256x64x128w4", 256, 64, 128, 256},
};
} // namespace

int fp8_dma_variant_count() { return int(sizeof(variants) / sizeof(variants[0])); }
const TnVariant &fp8_dma_variant(int index) { return variants[index]; }

// Needs outputs % 4 == 0 (8-byte BF16 stores) and 16-byte aligned a, w (rows are multiples of 128).
hipError_t launch_fp8_dma(hipStream_t stream, int variant, int rows, int outputs, int inner,
                          const void *a, const float *a_scale, const void *w, const float *w_scale,
                          void *out)
{
    if (outputs % 4 || inner % 128 || reinterpret_cast<uintptr_t>(out) % 8)
        return hipErrorInvalidValue;
    if (size_t(256) * size_t(inner) >= (size_t(1) << 32))
        return hipErrorInvalidValue;
    Fp8DmaParams p;
    p.w = static_cast<const unsigned char *>(w);
    p.a = static_cast<const unsigned char *>(a);
    p.w_scale = w_scale;
    p.a_scale = a_scale;
    p.out = static_cast<unsigned short *>(out);
    p.n = outputs;
    p.m = rows;
    p.k = inner;
    p.groups = inner / 128;
    p.scale_blocks = (outputs + 127) / 128;
    p.tiles_n = p.tiles_m = 0;
    switch (variant) {
    case 0: return launch_one<2, 4>(stream, p);
    case 1: return launch_one<1, 4>(stream, p);
    case 2: return launch_one<2, 2>(stream, p);
    case 3: return launch_one<1, 2>(stream, p);
    default: return hipErrorInvalidValue;
    }
}
} // namespace camblas_hip
