// Single-token FP8 E4M3fn decode product with 32-wide scale blocks: out[n] = sum over blocks b of
// (w[n, b] . x[b]) * sw[n/32, b] * sx[b], FP32 scales with element strides, BF16 out
// (contract: ref include/camblas_cuda.h:124-155, src/cuda/backend.cu:1193-1256; arithmetic:
// src/cuda/fp8_decode.cuh:150-157, sum = fma(dot_b * sw, sx, sum) for b ascending; the optional
// activation quantiser: src/cuda/fp8_decode.cuh:58-72, scale = 2^ceil(log2(amax / 448))).
//
// Bandwidth-bound on W. A wavefront owns 16 weight rows for the whole K extent and keeps the
// reference's single ascending chain per row; there is no cross-wavefront sum and no scratch.
// One 128-byte step of a row holds four scale blocks, which one
// v_mfma_scale_f32_16x16x128_f8f6f4 separates: in its operand layout lane group c = lane/16
// supplies K bytes 32c .. 32c+31, i.e. exactly block c, so a B operand that carries x's block c in
// column c and zeros elsewhere makes output column c the dot product of block c alone. The lane
// that owns column c multiplies by its weight scale, the four products are gathered into column 0
// with row shifts (DPP) and chained there. W is loaded with eight lanes per 128-byte line
// (non-temporal, eight steps in flight per wavefront) and transposed to the operand layout
// through a private swizzled LDS patch, as in the 128-block streaming kernel.
// A wavefront runs its steps one after another with few wavefronts per SIMD to hide them (16 rows per
// wavefront: 1152 wavefronts for 18432 outputs), so the loop is kept short: the weight scales of the
// wavefront's rows are copied to LDS once instead of being fetched per step, and when K is whole steps
// (EXACT) the weight loads are buffer loads with fixed lane offsets and the K position in the scalar
// offset, a step past the end reading through a descriptor of no bytes.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
struct Block32Params {
    const unsigned char *w;
    const void *x;    // E4M3 bytes, or BF16 when the kernel quantises
    const float *sx;  // unused when the kernel quantises
    const float *sw;
    unsigned short *out;
    int n, k, sx_stride, sw_row, sw_col;
};

constexpr int DEPTH = 8, STEP = 128, MAX_K = 8192;
constexpr int UNIT = 0x7f7f7f7f; // E8M0 exponent 127 = scale 1.0 in every byte

// WAVES: wavefronts (of 16 rows each) per workgroup. Few outputs take fewer, so that the wavefronts spread
// over more compute units: what a compute unit can draw is bounded by what it keeps in flight
// ([4096, 7168]: 16.0 us on 64 workgroups of four wavefronts, measured below on 256 of one).
template <bool QUANTISE, bool EXACT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void fp8_block32_decode_kernel(Block32Params p)
{
    // x and its scales, zero-padded to a whole number of DEPTH-step rounds
    __shared__ __attribute__((aligned(16))) unsigned x_words[MAX_K / 4];
    __shared__ __attribute__((aligned(16))) float x_scale[MAX_K / 32];
    __shared__ __attribute__((aligned(16))) u32x4_t patch[WAVES][2 * 128]; // two steps' tiles
    // the scales of each wavefront's rows (16 rows lie in one 32-row block: one scale per 32-input block)
    __shared__ float w_scale[WAVES][MAX_K / 32];
    const int thread = threadIdx.x, lane = thread % 64, wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const int blocks = p.k / 32, steps = (p.k + STEP - 1) / STEP;
    const int rounds = (steps + DEPTH - 1) / DEPTH, padded_steps = rounds * DEPTH;

    // ---- addresses first, so that the weight stream can start before the token is staged. A
    // wavefront past the last row keeps valid addresses (row 0) and leaves after the barrier.
    const bool owns_rows = (blockIdx.x * WAVES + wave) * 16 < p.n;
    const int first_row = owns_rows ? (blockIdx.x * WAVES + wave) * 16 : 0;
    const int column = lane % 16, chunk = lane / 16; // operand column / row, 32-byte chunk = block
    const int load_row = lane / 8, piece = lane % 8; // load layout: 8 lanes per 128-byte line
    const unsigned char *row_base[2] = {p.w + size_t(first_row + load_row) * p.k,
                                        p.w + size_t(first_row + 8 + load_row) * p.k};
    const float *sw_row = p.sw + size_t(first_row / 32) * p.sw_row;
    auto slot = [](int r, int q) { return r * 8 + (q ^ ((r >> 1) & 7)); };
    const int store_slot[2] = {slot(load_row, piece), slot(load_row + 8, piece)};
    const int read_slot[2] = {slot(column, 2 * chunk), slot(column, 2 * chunk + 1)};
    u32x4_t *mine = &patch[wave][0];

    // Loads only (nothing here may use a loaded value). Bytes past the end of a row in a partial
    // last step, and whole steps past the end, re-read the row's last 16 bytes: x is zero there.
    u32x4_t raw[DEPTH][2];
    const unsigned lane_offset[2] = {unsigned(load_row) * unsigned(p.k) + unsigned(piece) * 16u,
                                     unsigned(load_row + 8) * unsigned(p.k) + unsigned(piece) * 16u};
    auto fetch = [&](int step, u32x4_t(&data)[2]) {
        if constexpr (EXACT) { // (cache policy 2: non-temporal)
            const __amdgpu_buffer_rsrc_t rows =
                make_resource(p.w + size_t(first_row) * p.k, step < steps ? 16u * unsigned(p.k) : 0u);
            data[0] = __builtin_amdgcn_raw_buffer_load_b128(rows, int(lane_offset[0]), step * STEP, 2);
            data[1] = __builtin_amdgcn_raw_buffer_load_b128(rows, int(lane_offset[1]), step * STEP, 2);
        } else {
            int offset = step * STEP + piece * 16;
            offset = offset < p.k ? offset : p.k - 16;
            data[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(row_base[0] + offset));
            data[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(row_base[1] + offset));
        }
    };

    // ---- the token: its loads are issued first, the first DEPTH weight steps right behind them,
    // and only then are the token's values used (loads return in order, so waiting for the token
    // does not wait for the weights): the weight stream's first latency overlaps the staging.
    // Every loop below has a fixed trip count (MAX_K bounds it) so that the compiler can count the
    // loads in flight instead of waiting for all of them.
    constexpr int WORDS_PER_THREAD = MAX_K / 4 / (WAVES * 64), BLOCKS_PER_THREAD = MAX_K / 32 / (WAVES * 64);
    const unsigned *source = static_cast<const unsigned *>(p.x);
    unsigned staged[QUANTISE ? 16 * BLOCKS_PER_THREAD : WORDS_PER_THREAD];
    float staged_scale[BLOCKS_PER_THREAD] = {};
    if constexpr (QUANTISE) {
#pragma unroll
        for (int i = 0; i < BLOCKS_PER_THREAD; ++i) {
            const int block = thread + i * WAVES * 64;
            const int b = block < blocks ? block : blocks - 1; // BF16 pairs of a 32-value block
#pragma unroll
            for (int e = 0; e < 16; ++e)
                staged[16 * i + e] = source[b * 16 + e];
        }
    } else {
#pragma unroll
        for (int i = 0; i < WORDS_PER_THREAD; ++i) {
            const int word = thread + i * WAVES * 64;
            staged[i] = source[word < p.k / 4 ? word : p.k / 4 - 1];
        }
#pragma unroll
        for (int i = 0; i < BLOCKS_PER_THREAD; ++i) {
            const int b = thread + i * WAVES * 64;
            staged_scale[i] = p.sx[size_t(b < blocks ? b : blocks - 1) * p.sx_stride];
        }
    }
    // the wavefront's weight scales, block lane + 64 i (past the end: the last one again; x is zero there)
    constexpr int SCALES_PER_LANE = MAX_K / 32 / 64;
    float staged_weight_scale[SCALES_PER_LANE];
#pragma unroll
    for (int i = 0; i < SCALES_PER_LANE; ++i) {
        const int b = lane + 64 * i;
        staged_weight_scale[i] = sw_row[size_t(b < blocks ? b : blocks - 1) * p.sw_col];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        fetch(d, raw[d]);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < SCALES_PER_LANE; ++i)
        w_scale[wave][lane + 64 * i] = staged_weight_scale[i];
    if constexpr (QUANTISE) {
#pragma unroll
        for (int i = 0; i < BLOCKS_PER_THREAD; ++i) {
        const int b = thread + i * WAVES * 64;
        if (b < padded_steps * 4) {
            float value[32];
            float amax = 1e-10f;
            if (b < blocks) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const unsigned pair = staged[16 * i + e];
                    value[2 * e] = __uint_as_float(pair << 16);
                    value[2 * e + 1] = __uint_as_float(pair & 0xffff0000u);
                    amax = fmaxf(amax, fmaxf(fabsf(value[2 * e]), fabsf(value[2 * e + 1])));
                }
                // power of two not below amax / 448: exponent of the product, plus one unless it
                // is already a power of two
                unsigned bits = __float_as_uint(__fmul_rn(amax, 1.f / 448.f));
                int exponent = int((bits >> 23) & 255u) - 127 + int((bits & 0x7fffffu) != 0);
                x_scale[b] = __uint_as_float(unsigned(exponent + 127) << 23);
                float multiplier = __uint_as_float(unsigned(127 - exponent) << 23);
#pragma unroll
                for (int word = 0; word < 8; ++word) {
                    unsigned packed = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        packed |= f32_to_e4m3_sat(fminf(__fmul_rn(value[4 * word + e], multiplier), 448.f))
                                  << (8 * e);
                    x_words[b * 8 + word] = packed;
                }
            } else {
                x_scale[b] = 0.f;
#pragma unroll
                for (int word = 0; word < 8; ++word)
                    x_words[b * 8 + word] = 0u;
            }
        }
        } // blocks of this thread
    } else {
#pragma unroll
        for (int i = 0; i < WORDS_PER_THREAD; ++i) {
            const int word = thread + i * WAVES * 64;
            if (word < padded_steps * 32)
                x_words[word] = word < p.k / 4 ? staged[i] : 0u;
        }
#pragma unroll
        for (int i = 0; i < BLOCKS_PER_THREAD; ++i) {
            const int b = thread + i * WAVES * 64;
            if (b < padded_steps * 4)
                x_scale[b] = b < blocks ? staged_scale[i] : 0.f;
        }
    }
    // (not __syncthreads(): its fence would wait for every weight load issued above; the LDS
    // stores are waited for explicitly, the weight loads stay in flight)
    pipeline_barrier<63>();
    if (!owns_rows)
        return; // no barrier below this point

    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    // Two steps at a time: their LDS round trips, matrix instructions and row shifts overlap, and only the
    // chains of fused multiply-adds run in the order of the blocks (a wavefront has nobody to hide a step's
    // latencies behind: [4096, 7168] took 56 steps x 0.24 us whatever the memory system did).
    auto multiply = [&](int step, const u32x4_t(&first)[2], const u32x4_t(&second)[2]) {
        mine[store_slot[0]] = first[0];
        mine[store_slot[1]] = first[1];
        mine[128 + store_slot[0]] = second[0];
        mine[128 + store_slot[1]] = second[1];
        // other lanes' stores are read below: keep the compiler from moving the loads up (the
        // hardware executes one wavefront's LDS operations in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const unsigned keep = column == chunk ? 0xffffffffu : 0u; // block c only in column c
        float scaled[2][4];
        f32x4_t scales[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const u32x4_t lo = mine[128 * half + read_slot[0]], hi = mine[128 * half + read_slot[1]];
            const u32x4_t *x_step = reinterpret_cast<const u32x4_t *>(x_words) + (step + half) * 8 + chunk * 2;
            const u32x4_t x_lo = x_step[0], x_hi = x_step[1];
            const i32x8_t a = {int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                               int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
            const i32x8_t b = {int(x_lo[0] & keep), int(x_lo[1] & keep), int(x_lo[2] & keep), int(x_lo[3] & keep),
                               int(x_hi[0] & keep), int(x_hi[1] & keep), int(x_hi[2] & keep), int(x_hi[3] & keep)};
            const f32x4_t dot = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                a, b, f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, UNIT, 0, UNIT);
            const float scale = w_scale[wave][(step + half) * 4 + (column & 3)];
            scales[half] = *reinterpret_cast<const f32x4_t *>(x_scale + (step + half) * 4);
#pragma unroll
            for (int r = 0; r < 4; ++r)
                scaled[half][r] = __fmul_rn(dot[r], scale);
        }
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // column c holds block c of row 4*chunk + r; bring blocks 1..3 to column 0 and chain
                const float value = scaled[half][r];
                const float block1 = dpp_move<0x101>(value), block2 = dpp_move<0x102>(value),
                            block3 = dpp_move<0x103>(value);
                sum[r] = fmaf(value, scales[half][0], sum[r]);
                sum[r] = fmaf(block1, scales[half][1], sum[r]);
                sum[r] = fmaf(block2, scales[half][2], sum[r]);
                sum[r] = fmaf(block3, scales[half][3], sum[r]);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    static_assert(DEPTH % 2 == 0, "steps go in pairs");
    for (int step = 0; step < padded_steps; step += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d += 2) {
            __builtin_amdgcn_sched_barrier(0);
            multiply(step + d, raw[d], raw[d + 1]);
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + d + DEPTH, raw[d]);
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + d + 1 + DEPTH, raw[d + 1]);
        }
    }
    if (column == 0) {
        unsigned short *out = p.out + first_row + chunk * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            out[r] = float_to_bf16_bits(sum[r]);
    }
}
} // namespace

// x: E4M3 bytes with FP32 scales sx (element stride sx_stride), or BF16 quantised on the fly when
// sx is null. outputs a positive multiple of 16, inner a multiple of 32 in [32, 8192], w 16-byte
// and x 4-byte aligned.
hipError_t launch_fp8_block32_decode(hipStream_t stream, int outputs, int inner, const void *x,
                                     const float *sx, int sx_stride, const void *w, const float *sw,
                                     int sw_row, int sw_col, void *out, int forced_waves)
{
    if (outputs < 16 || outputs % 16 || inner < 32 || inner > MAX_K || inner % 32)
        return hipErrorInvalidValue;
    Block32Params p;
    p.w = static_cast<const unsigned char *>(w);
    p.x = x;
    p.sx = sx;
    p.sw = sw;
    p.out = static_cast<unsigned short *>(out);
    p.n = outputs;
    p.k = inner;
    p.sx_stride = sx_stride;
    p.sw_row = sw_row;
    p.sw_col = sw_col;
    const bool exact = inner % STEP == 0; // (16 rows of at most 8192 bytes fit any descriptor)
    const auto grid_of = [outputs](int waves) { return unsigned((outputs + waves * 16 - 1) / (waves * 16)); };
    // (one wavefront per workgroup spreads the wavefronts evenly over the compute units: [18432, 7168] 25.1 us
    // against 29.9 with four, [4096, 7168] 13.6 against 16.2; the others are kept for tests)
    // (the quantising form keeps four: every workgroup quantises the whole token first, and with one
    // wavefront that takes four times as long: [18432, 7168] 28.6 us with four, 29.2 with one)
    const int waves = forced_waves ? forced_waves : sx ? 1 : 4;
#define CAMBLAS_BLOCK32(QUANTISE, WAVES) \
    (exact ? fp8_block32_decode_kernel<QUANTISE, true, WAVES> : fp8_block32_decode_kernel<QUANTISE, false, WAVES>) \
        <<<grid_of(WAVES), WAVES * 64, 0, stream>>>(p)
    switch (waves * 2 + (sx ? 0 : 1)) {
    case 2: CAMBLAS_BLOCK32(false, 1); break;
    case 3: CAMBLAS_BLOCK32(true, 1); break;
    case 4: CAMBLAS_BLOCK32(false, 2); break;
    case 5: CAMBLAS_BLOCK32(true, 2); break;
    case 8: CAMBLAS_BLOCK32(false, 4); break;
    case 9: CAMBLAS_BLOCK32(true, 4); break;
    default: return hipErrorInvalidValue;
    }
#undef CAMBLAS_BLOCK32
    return launch_status();
}
} // namespace camblas_hip
