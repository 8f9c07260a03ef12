// Bandwidth-bound FP8 E4M3fn block-scaled decode linear (few tokens): out[M,N] =
// sum_g (a[M,g] . w[N,g]) * a_scale[M,g] * w_scale[N/128,g], 1x128 activation groups, 128x128
// weight blocks, FP32 scales, BF16 out. Rule: ref camblas/_hopper.py:118-126 and :168-182 (which
// covers one token); here up to 64 tokens share one pass over the weights.
//
// The whole cost is reading W once, so the kernel is the FP8 sibling of the BF16 weight-streaming
// kernel: a workgroup owns 16*NT consecutive weight rows for the whole K extent, no split-K pass
// and no scratch. One K group (128 bytes per row) is exactly one v_mfma_scale_f32_16x16x128_f8f6f4
// per 16x16 output tile. The four wavefronts take groups g = 4s + wave and never synchronise in
// the loop: a wavefront loads its group of a 16-row tile with two 128-bit loads per lane in which
// eight lanes cover one whole 128-byte line (loading straight in the MFMA operand layout would
// touch every line from eight different quarter-wave passes, which the L1 tag pipeline cannot
// sustain), transposes it to the operand layout (row lane%16, 32 bytes lane/16) through a private,
// XOR-swizzled 2 KB LDS patch, which needs no barrier because LDS operations of one wavefront
// execute in order, and multiplies. Each wavefront keeps the ascending fma chain
// acc = fma(dot_g, a_s * w_s, acc) over its own groups (hardware block scales are set to one: the
// scales here are FP32), and the four partial sums are added in wavefront order at the end, so
// results do not depend on scheduling. Weight loads are non-temporal (read once); two or three
// groups are in flight per wavefront.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
struct Fp8StreamParams {
    const unsigned char *w;
    const unsigned char *a;
    const float *w_scale;
    const float *a_scale;
    unsigned short *out;
    int n, m, k, groups, scale_blocks;
};

constexpr int WAVES = 4, GROUP = 128;
constexpr int UNIT = 0x7f7f7f7f; // E8M0 exponent 127 = scale 1.0 in every byte

// NT, MT: 16-row weight tiles and 16-token tiles per workgroup.
template <int NT, int MT>
__global__ __launch_bounds__(WAVES * 64) void fp8_stream_kernel(Fp8StreamParams p)
{
    // groups in flight per wavefront: three while the operand registers allow it
    constexpr int DEPTH = NT + MT <= 6 ? 3 : 2;
    constexpr int TILES = NT + MT; // weight tiles, then token tiles
    // (per wavefront: the 2 KB patches of its tiles, or, after the last step, its NT * MT partial tiles of 1 KB)
    constexpr int PATCH = TILES * 128 > NT * MT * 64 ? TILES * 128 : NT * MT * 64;
    __shared__ __attribute__((aligned(16))) u32x4_t patch[WAVES][PATCH];
    // The scales of the workgroup's tokens (one row of `groups` floats per token) and of the two
    // 128-row weight blocks its rows can lie in, copied to LDS once: a lane that fetched its
    // token's scale for every group itself would request a cache line per lane and group, the same
    // line for 32 groups (measured: 8 % of the launch at 32 tokens, 22 % at 64).
    constexpr int SCALE_ROWS = MT * 16 + 2, SCALE_PITCH = STREAM_SCALE_PITCH;
    __shared__ float scale_table[SCALE_ROWS * SCALE_PITCH];
    // after the last step the wavefront's patches hold its partial sums instead
    const int thread = threadIdx.x, lane = thread % 64, wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const int row = lane % 16, chunk = lane / 16; // operand row / token, 32-byte chunk of the group
    const int load_row = lane / 8, piece = lane % 8; // load layout: 8 lanes per 128-byte line
    const int n0 = blockIdx.x * (NT * 16), m0 = blockIdx.y * (MT * 16);
    const int steps = (p.groups + WAVES - 1) / WAVES; // groups per wavefront, padded

    // tile t < NT: weight rows n0 + 16 t ..; tile NT + j: tokens m0 + 16 j ..; half h: rows 8h ..
    // Weight and token rows are addressed by byte offsets inside descriptors of the rows that exist
    // for this workgroup; a row past the end, and every load of a step past the end of K, gets an
    // offset outside the descriptor, which reads as zero without a memory request. (Reading existing
    // bytes in their place costs: lanes that all read one existing row request its lines again while
    // the first request is in flight, which holds up the vector cache, and the re-read last group of
    // the prefetches beyond the loop came from HBM again: 11 % more bytes than the weights at one token.)
    unsigned weight_offset[NT][2], token_offset[MT][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const int n = i * 16 + h * 8 + load_row;
            weight_offset[i][h] = n0 + n < p.n ? unsigned(n) * unsigned(p.k) + unsigned(piece) * 16u : 0x80000000u;
        }
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int m = j * 16 + h * 8 + load_row;
            token_offset[j][h] = m0 + m < p.m ? unsigned(m) * unsigned(p.k) + unsigned(piece) * 16u : 0x80000000u;
        }
    }
    const unsigned weight_bytes = unsigned(p.n - n0 < NT * 16 ? p.n - n0 : NT * 16) * unsigned(p.k);
    const unsigned token_bytes = unsigned(p.m - m0 < MT * 16 ? p.m - m0 : MT * 16) * unsigned(p.k);
    // rows of the scale table: tokens m0 .., then the weight blocks first_block and first_block + 1
    const int first_block = n0 / 128;
    int ws_row[NT], as_row[MT];
#pragma unroll
    for (int i = 0; i < NT; ++i)
        ws_row[i] = (MT * 16 + (n0 + i * 16) / 128 - first_block) * SCALE_PITCH;
#pragma unroll
    for (int j = 0; j < MT; ++j)
        as_row[j] = (j * 16 + row) * SCALE_PITCH;
    // One 4-byte-per-lane direct-to-LDS load brings 64 consecutive groups of a row (lanes past the
    // row's end, and rows past the matrix, read zeros from the bounded buffer; the table's pitch
    // leaves room for whole loads). Issued before the first weight loads, complete with them.
    {
        const u32x4_t token_scales = uniform_descriptor(
            p.a_scale + size_t(m0) * p.groups, unsigned(p.m - m0 < MT * 16 ? p.m - m0 : MT * 16) * unsigned(p.groups) * 4u);
        const u32x4_t block_scales = uniform_descriptor(
            p.w_scale + size_t(first_block) * p.groups,
            unsigned(p.scale_blocks - first_block < 2 ? p.scale_blocks - first_block : 2) * unsigned(p.groups) * 4u);
        for (int r = __builtin_amdgcn_readfirstlane(wave); r < SCALE_ROWS; r += WAVES) {
            const bool token = r < MT * 16;
            const unsigned row_bytes = unsigned(token ? r : r - MT * 16) * unsigned(p.groups) * 4u;
            for (int g0 = 0; g0 < p.groups; g0 += 64)
                load_word_to_lds_untracked(token ? token_scales : block_scales, unsigned(lane) * 4u,
                                           row_bytes + unsigned(g0) * 4u, scale_table + r * SCALE_PITCH + g0);
        }
    }
    // LDS patch of one tile: 16 rows x 8 pieces of 16 bytes, piece index XORed with row bits 1..3,
    // which makes both the line-shaped stores and the operand-shaped loads conflict-free
    auto slot = [](int r, int q) { return r * 8 + (q ^ ((r >> 1) & 7)); };
    const int store_slot[2] = {slot(load_row, piece), slot(load_row + 8, piece)};
    const int read_slot[2] = {slot(row, 2 * chunk), slot(row, 2 * chunk + 1)};

    // Workgroups start at different groups and wrap around, which spreads the row-pitch-strided
    // requests of the chip over all HBM channels. Steps past the end (the padding of the last
    // round of four groups, and the DEPTH prefetches beyond the loop) re-read the last group and
    // are given a zero scale.
    const int start = int(blockIdx.x % unsigned(steps));
    auto group_of = [&](int step) {
        int rotated = (step < steps ? step : steps - 1) + start;
        rotated = rotated < steps ? rotated : rotated - steps;
        return rotated * WAVES + wave;
    };
    u32x4_t raw[DEPTH][TILES][2];
    int group_reg[DEPTH];
    float live_reg[DEPTH];
    // Nothing in a fetch may use a loaded value (that would wait for the loads just issued): a dead
    // step is remembered as a zero factor and applied to the scale when the group is multiplied.
    auto fetch = [&](int step, u32x4_t(&data)[TILES][2], int &group, float &live) {
        int g = group_of(step);
        const bool exists = step < steps && g < p.groups;
        live = exists ? 1.f : 0.f;
        g = g < p.groups ? g : p.groups - 1;
        group = g;
        // The lane offsets never change: the group's position along K is the scalar offset, and a step past
        // the end reads through descriptors of no bytes (zeros, no memory request), so a fetch costs the
        // vector ALU nothing (a wavefront runs its fetches, LDS transposes and products one after another).
        const int offset = g * GROUP;
        const __amdgpu_buffer_rsrc_t weight_resource = make_resource(p.w + size_t(n0) * p.k, exists ? weight_bytes : 0u);
        const __amdgpu_buffer_rsrc_t token_resource = make_resource(p.a + size_t(m0) * p.k, exists ? token_bytes : 0u);
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                // (weights: read once, so non-temporal, cache policy bit 1)
                if (t < NT)
                    data[t][h] = __builtin_amdgcn_raw_buffer_load_b128(weight_resource, int(weight_offset[t < NT ? t : 0][h]), offset, 2);
                else
                    data[t][h] = __builtin_amdgcn_raw_buffer_load_b128(token_resource, int(token_offset[t < NT ? 0 : t - NT][h]), offset, 0);
            }
    };

    f32x4_t acc[NT][MT];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
            acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const u32x4_t(&data)[TILES][2], int group, float live) {
        u32x4_t *mine = &patch[wave][0];
        float ws[NT], as[MT];
#pragma unroll
        for (int i = 0; i < NT; ++i)
            ws[i] = scale_table[ws_row[i] + group];
#pragma unroll
        for (int j = 0; j < MT; ++j)
            as[j] = scale_table[as_row[j] + group];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            mine[t * 128 + store_slot[0]] = data[t][0];
            mine[t * 128 + store_slot[1]] = data[t][1];
        }
        // other lanes' stores are read below: keep the compiler from moving the loads up (the
        // hardware executes one wavefront's LDS operations in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        i32x8_t operand[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            u32x4_t lo = mine[t * 128 + read_slot[0]], hi = mine[t * 128 + read_slot[1]];
            operand[t] = i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                                 int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
        }
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int j = 0; j < MT; ++j) {
                f32x4_t dot = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    operand[i], operand[NT + j], f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, UNIT, 0, UNIT);
                const float scale = __fmul_rn(as[j], ws[i]) * live;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[i][j][r] = fmaf(dot[r], scale, acc[i][j][r]);
            }
        // the next group's stores must not overtake these loads in the compiler either
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // sched_barrier(0) keeps the fetches of different steps apart so that the wait before a
    // multiply covers only the oldest of the groups in flight
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        fetch(d, raw[d], group_reg[d], live_reg[d]);
        __builtin_amdgcn_sched_barrier(0);
    }
    // the scale table's loads are older than the DEPTH * TILES * 2 loads of the fetches above (the
    // compiler does not count them, so the wait is explicit); the barrier shows every wavefront's
    // part of the table to the others
    wait_loads<DEPTH * TILES * 2>();
    __syncthreads();
    for (int step = 0; step < steps; step += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            __builtin_amdgcn_sched_barrier(0);
            multiply(raw[d], group_reg[d], live_reg[d]);
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + d + DEPTH, raw[d], group_reg[d], live_reg[d]);
        }
    }
    // ---- every wavefront parks its partial sums in its own patches (nobody else reads those);
    // after one barrier tile t is summed in wavefront order 0, 1, 2, 3 by wavefront t % 4
    f32x4_t *parked = reinterpret_cast<f32x4_t *>(&patch[wave][0]);
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
            parked[(i * MT + j) * 64 + lane] = acc[i][j];
    __syncthreads();
    // ---- epilogue: wavefront w writes tiles w, w+4, ...; register r of lane l is feature
    // 4*(l/16) + r and token l%16 inside the 16x16 tile
    const bool vector_store = p.n % 4 == 0 && reinterpret_cast<uintptr_t>(p.out) % 8 == 0;
#pragma unroll
    for (int index = 0; index < NT * MT; ++index) {
        if (index % WAVES != wave)
            continue;
        const int i = index / MT, j = index % MT;
        const int m = m0 + j * 16 + row;
        const int n = n0 + i * 16 + chunk * 4;
        if (m >= p.m || n >= p.n)
            continue;
        f32x4_t sum = reinterpret_cast<const f32x4_t *>(&patch[0][0])[index * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            sum = sum + reinterpret_cast<const f32x4_t *>(&patch[w][0])[index * 64 + lane];
        unsigned short *out = p.out + size_t(m) * p.n + n;
        if (n + 3 < p.n && vector_store) {
            u32x2_t packed = {pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3])};
            *reinterpret_cast<u32x2_t *>(out) = packed;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < p.n)
                    out[e] = float_to_bf16_bits(sum[e]);
        }
    }
}

template <int NT, int MT> hipError_t launch_one(hipStream_t stream, const Fp8StreamParams &p)
{
    // the prefetch registers grow with NT + MT: keep both groups in flight inside the register file
    if constexpr (NT * MT > 20 || NT + MT > 10) {
        return hipErrorInvalidValue;
    } else {
        dim3 grid(unsigned((p.n + NT * 16 - 1) / (NT * 16)), unsigned((p.m + MT * 16 - 1) / (MT * 16)));
        fp8_stream_kernel<NT, MT><<<grid, WAVES * 64, 0, stream>>>(p);
        return launch_status();
    }
}

template <int MT> hipError_t launch_rows(hipStream_t stream, int row_tiles, const Fp8StreamParams &p)
{
    switch (row_tiles) {
    case 1: return launch_one<1, MT>(stream, p);
    case 2: return launch_one<2, MT>(stream, p);
    case 3: return launch_one<3, MT>(stream, p);
    case 4: return launch_one<4, MT>(stream, p);
    case 5: return launch_one<5, MT>(stream, p);
    case 6: return launch_one<6, MT>(stream, p);
    case 7: return launch_one<7, MT>(stream, p);
    case 8: return launch_one<8, MT>(stream, p);
    default: return hipErrorInvalidValue;
    }
}
} // namespace

// row_tiles 1..8 (16 weight rows each), token_tiles 1 to 4 (16 tokens each), their product at most 20 and
// their sum at most 10; a, w 16-byte
// aligned, inner a multiple of 128.
hipError_t launch_fp8_stream(hipStream_t stream, int row_tiles, int token_tiles, int rows, int outputs,
                             int inner, const void *a, const float *a_scale, const void *w,
                             const float *w_scale, void *out)
{
    if (inner % GROUP || inner < GROUP || inner / GROUP > STREAM_SCALE_GROUPS || rows < 1 || outputs < 1)
        return hipErrorInvalidValue;
    if ((rows + token_tiles * 16 - 1) / (token_tiles * 16) > 65535)
        return hipErrorInvalidValue;
    // (a workgroup addresses its token rows with 31-bit byte offsets inside one descriptor)
    if (size_t(std::max(token_tiles, row_tiles)) * 16 * size_t(inner) >= (size_t(1) << 31))
        return hipErrorInvalidValue;
    Fp8StreamParams p;
    p.w = static_cast<const unsigned char *>(w);
    p.a = static_cast<const unsigned char *>(a);
    p.w_scale = w_scale;
    p.a_scale = a_scale;
    p.out = static_cast<unsigned short *>(out);
    p.n = outputs;
    p.m = rows;
    p.k = inner;
    p.groups = inner / GROUP;
    p.scale_blocks = (outputs + 127) / 128;
    switch (token_tiles) {
    case 1: return launch_rows<1>(stream, row_tiles, p);
    case 2: return launch_rows<2>(stream, row_tiles, p);
    case 3: return launch_rows<3>(stream, row_tiles, p);
    case 4: return launch_rows<4>(stream, row_tiles, p);
    default: return hipErrorInvalidValue;
    }
}
} // namespace camblas_hip
