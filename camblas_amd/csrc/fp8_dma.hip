// FP8 E4M3fn block-scaled prefill linear (1x128 activation groups, 128x128 weight blocks, FP32
// scales, BF16 out) on the gfx950 matrix cores, operands streamed straight into LDS.
//
// Arithmetic rule (ref: camblas/_hopper.py:118-126 and :168-182): per 128-wide K group the
// unscaled FP32 dot product on the matrix cores, then acc = fma(dot_g, a_s * w_s, acc) for g
// ascending with a_s * w_s rounded to FP32 first, one BF16 rounding at the end.
//
// A workgroup of 2 x WM wavefronts owns a (64*TN) x (32*WM*TM) output tile; each wavefront owns
// 32*TN weight rows (TN = 4: exactly one 128-row scale block; TN = 3 gives 192-row tiles, whose
// count fills the compute units better for some shapes) by 32*TM tokens. One K step is one scale group:
// 128 bytes per row, the same LDS geometry (8 chunks of 16 bytes, XOR swizzle) as a 64-deep BF16
// step, STAGES stages filled by buffer_load ... lds STAGES-1 groups ahead (one group of matrix
// work is shorter than the memory latency, so two stages leave the matrix cores waiting for
// loads). A group's dot product is two
// v_mfma_scale_f32_32x32x64_f8f6f4 (unit hardware scales) into a zeroed temporary; the scaled
// accumulate of one 32x32 tile runs on the vector ALU while the matrix cores work on the next tile.
// The scales reach the lanes through LDS as well: slabs of eight groups per token (and per weight
// block) are copied in with direct-to-LDS loads once per round of six or eight groups, and a lane
// reads the next group's scales from there at the end of a step.
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
    float *partials; // FP32 [splits, m, n] when the K groups are divided over blockIdx.y, else null
    int n, m, k, groups, scale_blocks;
    int out_pitch; // elements between tokens in `out` (the outputs of the whole product)
    int tiles_n, tiles_m;
    int split_groups; // K groups per blockIdx.y (all of them without a split)
};

// NARROW: the products run on v_mfma_scale_f32_16x16x128_f8f6f4 (one instruction per 16 x 16 tile and
// K group, four accumulator registers) instead of pairs of 32 x 32 x 64 ones: on operands with random
// bits the part sustains 4.5 PFLOP/s with the former against 4.05 with the latter (it holds a higher
// clock), and this kernel is limited by that clock.
template <int TM, int WM, int STAGES, int TN, bool NARROW = false>
__global__ __launch_bounds__(128 * WM) void fp8_dma_kernel(Fp8DmaParams p)
{
    // (a fourth and a fifth stage were measured, with few and with many tokens: no gain, the kernel
    // is not limited by bytes in flight)
    static_assert(STAGES == 2 || STAGES == 3, "two or three LDS stages");
    constexpr int WAVES = 2 * WM, CH = 8, BK = 128;
    // weight scales per wavefront and group: one when its rows are one scale block, else one per
    // 32-row tile (a 32-row tile never straddles a 128-row block)
    constexpr int WS = TN == 4 ? 1 : TN;
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    constexpr int ROWS_PER_LOAD = 8;
    constexpr int A_ITERS = BN / (WAVES * ROWS_PER_LOAD), B_ITERS = BM / (WAVES * ROWS_PER_LOAD);
    constexpr int SLOTS = (BN + BM) * CH, LOADS = A_ITERS + B_ITERS;
    static_assert(BN % (WAVES * ROWS_PER_LOAD) == 0 && BM % (WAVES * ROWS_PER_LOAD) == 0, "loads");
    // Scale slabs (below) behind the stages, in the same array: BM / 32 KB for two buffers of
    // activation scales, then two buffers of 64 weight scales.
    constexpr int SLAB_SLOTS = BM / 32 * 64, WEIGHT_SLAB_SLOTS = 16;
    __shared__ u32x4_t lds[STAGES * SLOTS + 2 * SLAB_SLOTS + 2 * WEIGHT_SLAB_SLOTS];
    auto stage_at = [&](int index) { return lds + index * SLOTS; };

    int tile_n, tile_m;
    xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int wn = wave % 2, wm = wave / 2;

    // Lane -> (row inside an 8-row load, swizzled 16-byte chunk). Successive loads of a thread are
    // WAVES*8 rows apart, which leaves the swizzle unchanged (it depends on row bits 0..3 only and
    // WAVES*8 is a multiple of 16), so one lane offset serves all of them and the row advance goes
    // into the scalar offset. Rows past the end of the matrix are outside the buffer resource and
    // read as zero.
    static_assert((WAVES * ROWS_PER_LOAD) % 16 == 0, "row step keeps the swizzle");
    const int load_row = wave * ROWS_PER_LOAD + lane / CH;
    const unsigned lane_off =
        unsigned(load_row) * unsigned(p.k) + unsigned(((lane % CH) ^ lds_swizzle<CH>(load_row)) * 16);
    const unsigned row_step = unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.k);
    const int a_rows = p.n - n0 < BN ? p.n - n0 : BN, b_rows = p.m - m0 < BM ? p.m - m0 : BM;
    const __amdgpu_buffer_rsrc_t a_resource =
        make_resource(p.w + size_t(n0) * p.k, unsigned(a_rows) * unsigned(p.k));
    const __amdgpu_buffer_rsrc_t b_resource =
        make_resource(p.a + size_t(m0) * p.k, unsigned(b_rows) * unsigned(p.k));
    // this workgroup's share of the K groups: [first_group, first_group + group_count)
    const int first_group = int(blockIdx.y) * p.split_groups;
    const int group_count = p.groups - first_group < p.split_groups ? p.groups - first_group : p.split_groups;
    const unsigned last_k_bytes = unsigned(first_group + group_count - 1) * BK;
    unsigned k_bytes = unsigned(first_group) * BK;
    // Load number `index` (0 .. LOADS-1) of the group at k_bytes; advance() moves to the next group.
    auto issue_one = [&](u32x4_t *stage, int index) {
        if (index < A_ITERS)
            load_to_lds(a_resource, lane_off, k_bytes + unsigned(index) * row_step,
                        stage + (index * WAVES + wave) * 64);
        else
            load_to_lds(b_resource, lane_off, k_bytes + unsigned(index - A_ITERS) * row_step,
                        stage + BN * CH + ((index - A_ITERS) * WAVES + wave) * 64);
    };
    auto advance = [&]() { k_bytes = k_bytes + BK < last_k_bytes ? k_bytes + BK : last_k_bytes; };
    auto issue = [&](u32x4_t *stage) {
#pragma unroll
        for (int index = 0; index < LOADS; ++index)
            issue_one(stage, index);
        advance();
    };

    // ---- scales. The activation scales are one per token and group, rows of `groups` floats per
    // token. If every lane fetched its token's scale of the next group into a register (a cache
    // line per lane, the same line again for each of the 32 groups it holds), the kernel would lose
    // 6 % at 4096 tokens and 16 % at 256 (measured). Instead each wavefront copies, once per PERIOD
    // groups, 16 bytes per lane (four consecutive groups of a token, the two lanes of a token side
    // by side in memory) straight into LDS: lane l of loader w holds groups 4 * (l / 32) .. + 3 of
    // the slab for token 32 * w + l % 32, and a lane reads its tokens' scales from there (tokens 16
    // apart share a bank: two-way at worst). Slab number i holds SLAB_GROUPS groups from group
    // i * PERIOD of this workgroup's share on (PERIOD: the largest multiple of STAGES within
    // SLAB_GROUPS, so that a slab begins where a round of stages begins) and is loaded when slab
    // i - 1 comes into use, into the buffer that slab i - 2 has left.
    // Both the slab loads and the reads are kept out of the compiler's bookkeeping
    // (load_to_lds_untracked, lds_read_unordered): when it sees an LDS read that a direct-to-LDS
    // load might have written, it waits for every outstanding load, the stage fills included, in
    // the middle of a step, which cost all of the gain. The order is by construction: a slab load
    // is older than the fills of the step that follows, so that step's wait covers it PERIOD - 1
    // steps before the slab is first read; a read is issued a few instructions before the step's
    // wait and its value is used after it.
    // (32-wide instruction: operand row lane % 32, K half lane / 32; 16-wide: row lane % 16, K quarter lane / 16)
    constexpr int FRAG_ROWS = NARROW ? 16 : 32, NJ = NARROW ? 2 * TM : TM; // token tiles per wavefront
    const int frag_row = lane % FRAG_ROWS, half = lane / FRAG_ROWS;
    constexpr int LANES_PER_TOKEN = 2, SLAB_GROUPS = 4 * LANES_PER_TOKEN;
    constexpr int TOKENS_PER_WAVE = 64 / LANES_PER_TOKEN, LOADERS = BM / TOKENS_PER_WAVE;
    constexpr int PERIOD = SLAB_GROUPS / STAGES * STAGES;
    // (with 32 tokens per wavefront tile and one token tile per wavefront, two wavefronts load the
    // same piece: same bytes to the same place)
    static_assert(WAVES % LOADERS == 0 && PERIOD >= 3, "every wavefront loads one piece of a slab");
    static_assert(LOADERS * 64 == SLAB_SLOTS, "slab size");
    auto slab_at = [&](int index) { return lds + STAGES * SLOTS + (index & 1) * SLAB_SLOTS; };
    const int loader = __builtin_amdgcn_readfirstlane(wave) % LOADERS;
    const u32x4_t scale_resource =
        uniform_descriptor(p.a_scale + size_t(m0) * p.groups, unsigned(b_rows) * unsigned(p.groups) * 4u);
    const int slab_token = loader * TOKENS_PER_WAVE + lane % TOKENS_PER_WAVE;
    const unsigned slab_lane_off =
        (unsigned(slab_token < b_rows ? slab_token : b_rows - 1) * unsigned(p.groups) +
         unsigned(lane / TOKENS_PER_WAVE) * 4u) * 4u;
    // bytes past the end of the scales read as zero and are never used
    auto load_slab = [&](int slab) {
        load_to_lds_untracked(scale_resource, slab_lane_off, unsigned(first_group + slab * PERIOD) * 4u,
                              slab_at(slab) + loader * 64);
    };
    int as_index[NJ]; // float index of this lane's token inside a slab buffer (part 0, word 0)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int token = wm * TM * 32 + j * FRAG_ROWS + frag_row;
        as_index[j] = ((token / TOKENS_PER_WAVE) * 64 + token % TOKENS_PER_WAVE) * 4;
    }
    // (read with lds_read_unordered: the compiler would otherwise wait for every outstanding
    // direct-to-LDS load before a read of memory that such a load may write)
    auto activation_scale = [&](int j, int group) { // group counted from first_group
        const float *slab = reinterpret_cast<const float *>(slab_at(group / PERIOD));
        const int position = group % PERIOD;
        return lds_read_unordered(slab + as_index[j] + position / 4 * (TOKENS_PER_WAVE * 4) + position % 4);
    };
    // The weight scales travel the same way: the tile's rows lie in two or three 128-row blocks
    // (room for eight), and lane l of one 4-byte-per-lane load brings group l % 8 of the slab for
    // block l / 8 (every wavefront issues the same load: same bytes to the same place).
    static_assert(SLAB_GROUPS == 8 && BN <= 7 * 128, "eight blocks of eight groups per load");
    auto weight_slab_at = [&](int index) {
        return reinterpret_cast<float *>(lds + STAGES * SLOTS + 2 * SLAB_SLOTS + (index & 1) * WEIGHT_SLAB_SLOTS);
    };
    const int first_block = n0 / 128;
    const u32x4_t weight_scale_resource =
        uniform_descriptor(p.w_scale + size_t(first_block) * p.groups,
                      unsigned(p.scale_blocks - first_block < 8 ? p.scale_blocks - first_block : 8) *
                          unsigned(p.groups) * 4u);
    const unsigned weight_slab_lane_off = (unsigned(lane / 8) * unsigned(p.groups) + unsigned(lane % 8)) * 4u;
    int ws_index[WS];
#pragma unroll
    for (int s = 0; s < WS; ++s)
        ws_index[s] = ((n0 + wn * TN * 32 + s * 32) / 128 - first_block) * 8;
    auto weight_scale = [&](int s, int group) { // group counted from first_group
        return lds_read_unordered(weight_slab_at(group / PERIOD) + ws_index[s] + group % PERIOD);
    };
    auto load_slabs = [&](int slab) {
        load_slab(slab);
        load_word_to_lds_untracked(weight_scale_resource, weight_slab_lane_off,
                                   unsigned(first_group + slab * PERIOD) * 4u, weight_slab_at(slab));
    };

    const int frag_swizzle = lds_swizzle<CH>(frag_row);
    const int a_frag_base = (wn * TN * 32 + frag_row) * CH;
    const int b_frag_base = BN * CH + (wm * TM * 32 + frag_row) * CH;
    f32x16_t acc[NARROW ? 1 : TN][NARROW ? 1 : TM];
    constexpr int NI = 2 * TN; // 16-row weight tiles per wavefront
    f32x4_t acc16[NARROW ? NI : 1][NARROW ? NJ : 1];
    if constexpr (NARROW) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                acc16[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    } else {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = 0.f;
    }

    constexpr int UNIT = 0x7f7f7f7f; // E8M0 exponent 127 = scale 1.0 in every byte
    auto fragment = [&](const u32x4_t *stage, int base, int ks) {
        u32x4_t lo = stage[base + ((ks * 4 + half * 2) ^ frag_swizzle)];
        u32x4_t hi = stage[base + ((ks * 4 + half * 2 + 1) ^ frag_swizzle)];
        return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                       int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
    };
    // operand of the 16-wide instruction: lane quarter c holds K positions 16c .. 16c+15 of its row in
    // its first 16 bytes and 64+16c .. 64+16c+15 in its second 16 bytes
    auto fragment16 = [&](const u32x4_t *stage, int base) {
        u32x4_t lo = stage[base + (half ^ frag_swizzle)];
        u32x4_t hi = stage[base + ((4 + half) ^ frag_swizzle)];
        return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                       int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
    };
    // One K group on the 16-wide instruction. The token fragments are read once; the weight fragments
    // travel one 16-row tile ahead in two register buffers; the tiles are walked in a software
    // pipeline: the matrix instruction of tile t, a share of the LDS fills for the group STAGES-1
    // ahead, then the four scaled accumulates of tile t-1.
    auto multiply16 = [&](const u32x4_t *stage, u32x4_t *fill, const float (&as_now)[NJ], const float (&ws_now)[WS]) {
        constexpr int TILES = NI * NJ, SHARE = (LOADS + TILES - 1) / TILES;
        i32x8_t a_frag[2], b_frag[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            b_frag[j] = fragment16(stage, b_frag_base + j * 16 * CH);
        a_frag[0] = fragment16(stage, a_frag_base);
        float scale[WS][NJ];
#pragma unroll
        for (int s = 0; s < WS; ++s)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                scale[s][j] = __fmul_rn(as_now[j], ws_now[s]);
        f32x4_t dot[2];
#pragma unroll
        for (int tile = 0; tile < TILES; ++tile) {
            const int i = tile / NJ, j = tile % NJ;
            __builtin_amdgcn_sched_barrier(0);
            if (j == 0 && i + 1 < NI)
                a_frag[(i + 1) & 1] = fragment16(stage, a_frag_base + (i + 1) * 16 * CH);
            __builtin_amdgcn_sched_barrier(0);
            dot[tile & 1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                a_frag[i & 1], b_frag[j], f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, UNIT, 0, UNIT);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int index = tile * SHARE; index < (tile + 1) * SHARE && index < LOADS; ++index)
                issue_one(fill, index);
            __builtin_amdgcn_sched_barrier(0);
            if (tile > 0) {
                const int pi = (tile - 1) / NJ, pj = (tile - 1) % NJ;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc16[pi][pj][r] = fmaf(dot[(tile - 1) & 1][r], scale[WS == 1 ? 0 : pi / 2][pj], acc16[pi][pj][r]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        advance();
#pragma unroll
        for (int r = 0; r < 4; ++r)
            acc16[NI - 1][NJ - 1][r] =
                fmaf(dot[(TILES - 1) & 1][r], scale[WS == 1 ? 0 : (NI - 1) / 2][NJ - 1], acc16[NI - 1][NJ - 1][r]);
        __builtin_amdgcn_sched_barrier(0);
    };
    // One K group. The token fragments are read once; the weight fragments are streamed one
    // 32-row tile ahead (two register buffers), and the tiles are walked in a software pipeline: the
    // two MFMAs of tile t are issued, then a share of the LDS fills for the group STAGES-1 ahead,
    // then the 16 scaled accumulates of tile t-1, so that the vector ALU work and the load issue of
    // one tile run while the matrix cores execute the next (sched_barrier pins it).
    auto multiply = [&](const u32x4_t *stage, u32x4_t *fill, const float (&as_now)[NJ],
                        const float (&ws_now)[WS]) {
        constexpr int TILES = TN * TM, SHARE = (LOADS + TILES - 1) / TILES;
        // (eight tiles per wavefront at two wavefronts per SIMD leave no registers for a second
        // weight-fragment buffer: with it the 256 x 256 tile spilled 21 registers)
        constexpr int A_BUFFERS = TILES >= 8 && WAVES == 8 ? 1 : 2;
        i32x8_t a_frag[A_BUFFERS][2], b_frag[TM][2];
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            b_frag[j][0] = fragment(stage, b_frag_base + j * 32 * CH, 0);
            b_frag[j][1] = fragment(stage, b_frag_base + j * 32 * CH, 1);
        }
        a_frag[0][0] = fragment(stage, a_frag_base, 0);
        a_frag[0][1] = fragment(stage, a_frag_base, 1);
        float scale[WS][TM];
#pragma unroll
        for (int s = 0; s < WS; ++s)
#pragma unroll
            for (int j = 0; j < TM; ++j)
                scale[s][j] = __fmul_rn(as_now[j], ws_now[s]);
        f32x16_t dot[2];
        auto product = [&](int tile, f32x16_t &d) {
            const int i = tile / TM, j = tile % TM;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                d[r] = 0.f;
            d = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_frag[i % A_BUFFERS][0], b_frag[j][0], d, 0,
                                                                0, 0, UNIT, 0, UNIT);
            d = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_frag[i % A_BUFFERS][1], b_frag[j][1], d, 0,
                                                                0, 0, UNIT, 0, UNIT);
        };
        auto accumulate = [&](int tile, const f32x16_t &d) {
            const int i = tile / TM, j = tile % TM;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = fmaf(d[r], scale[WS == 1 ? 0 : i][j], acc[i][j][r]);
        };
#pragma unroll
        for (int tile = 0; tile < TILES; ++tile) {
            __builtin_amdgcn_sched_barrier(0);
            if (A_BUFFERS == 2 && tile % TM == 0 && tile / TM + 1 < TN) { // next weight tile into the other buffer
                const int row = tile / TM + 1;
                a_frag[row % A_BUFFERS][0] = fragment(stage, a_frag_base + row * 32 * CH, 0);
                a_frag[row % A_BUFFERS][1] = fragment(stage, a_frag_base + row * 32 * CH, 1);
            }
            if (A_BUFFERS == 1 && tile % TM == 0 && tile > 0) { // this row's weight tile, the last row's MFMAs being issued
                a_frag[0][0] = fragment(stage, a_frag_base + (tile / TM) * 32 * CH, 0);
                a_frag[0][1] = fragment(stage, a_frag_base + (tile / TM) * 32 * CH, 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            product(tile, dot[tile & 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int index = tile * SHARE; index < (tile + 1) * SHARE && index < LOADS; ++index)
                issue_one(fill, index);
            __builtin_amdgcn_sched_barrier(0);
            if (tile > 0)
                accumulate(tile - 1, dot[(tile - 1) & 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
        advance();
        accumulate(TILES - 1, dot[(TILES - 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
    };

    float ws_now[WS], as_now[NJ];
    // One group: start the loads of the group STAGES-1 ahead into the stage that was read last,
    // multiply the current stage, read the next group's scales, then wait until only the newest
    // loads are still in flight (the wait also covers the scale reads).
    auto step = [&](int g, const u32x4_t *current, u32x4_t *fill) {
        const int next = g + 1 < group_count ? g + 1 : group_count - 1;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NARROW)
            multiply16(current, fill, as_now, ws_now);
        else
            multiply(current, fill, as_now, ws_now);
#pragma unroll
        for (int s = 0; s < WS; ++s)
            ws_now[s] = weight_scale(s, next);
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            as_now[j] = activation_scale(j, next);
        pipeline_barrier<(STAGES - 2) * LOADS>();
        tie_after_wait(ws_now, as_now);
    };
    // Group g is read from stage g % STAGES while group g + STAGES - 1 is loaded into the stage
    // that was read last.
    load_slabs(0); // (the oldest loads: complete at the first wait)
#pragma unroll
    for (int s = 0; s + 1 < STAGES; ++s) {
        __builtin_amdgcn_sched_barrier(0);
        issue(stage_at(s));
    }
    pipeline_barrier<(STAGES - 2) * LOADS>();
#pragma unroll
    for (int s = 0; s < WS; ++s)
        ws_now[s] = weight_scale(s, 0);
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        as_now[j] = activation_scale(j, 0);
    __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
    tie_after_wait(ws_now, as_now);
    // whole rounds of STAGES groups run without a branch between the steps; the remainder follows
    int g = 0;
    for (int slab = 1; g + STAGES <= group_count; ++slab) {
        // (older than the fills of the step that follows: landed at that step's wait, PERIOD - 1
        // steps before its first scale is read)
        load_slabs(slab);
        const int end = slab * PERIOD < group_count ? slab * PERIOD : group_count;
        for (; g + STAGES <= end; g += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; ++s)
                step(g + s, stage_at(s), stage_at((s + STAGES - 1) % STAGES));
        }
    }
#pragma unroll
    for (int s = 0; s + 1 < STAGES; ++s)
        if (g + s < group_count)
            step(g + s, stage_at(s), stage_at((s + STAGES - 1) % STAGES));
    wait_loads<0>();

    if constexpr (NARROW) {
        // register e of lane l in tile (i, j) is feature 16 i + 4 (l / 16) + e, token 16 j + l % 16
        float *plane = p.partials ? p.partials + size_t(blockIdx.y) * size_t(p.m) * size_t(p.n) : nullptr;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int m = m0 + wm * TM * 32 + j * 16 + frag_row;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int n = n0 + wn * TN * 32 + i * 16 + half * 4;
                if (m >= p.m || n >= p.n)
                    continue;
                if (plane)
                    *reinterpret_cast<f32x4_t *>(plane + size_t(m) * p.n + n) = acc16[i][j];
                else
                    *reinterpret_cast<u32x2_t *>(p.out + size_t(m) * p.out_pitch + n) =
                        u32x2_t{pack_bf16x2(acc16[i][j][0], acc16[i][j][1]), pack_bf16x2(acc16[i][j][2], acc16[i][j][3])};
            }
        }
        return;
    }
    // ---- epilogue: accumulator register 4q+e of lane l is feature 8q + 4*(l/32) + e, token l%32
    if (p.partials) { // a share of the K groups: FP32 sums for the ordered reduction
        float *plane = p.partials + size_t(blockIdx.y) * size_t(p.m) * size_t(p.n);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const int m = m0 + (wm * TM + j) * 32 + frag_row;
            float *row = plane + size_t(m) * p.n + n0 + wn * TN * 32 + half * 4;
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int offset = i * 32 + q * 8;
                    if (m < p.m && n0 + wn * TN * 32 + half * 4 + offset < p.n)
                        *reinterpret_cast<f32x4_t *>(row + offset) = f32x4_t{
                            acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + (wm * TM + j) * 32 + frag_row;
        unsigned short *row = p.out + size_t(m) * p.out_pitch + n0 + wn * TN * 32 + half * 4;
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

template <int TM, int WM, int STAGES, int TN = 4, bool NARROW = false>
hipError_t launch_one(hipStream_t stream, Fp8DmaParams p, int splits)
{
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    p.tiles_n = (p.n + BN - 1) / BN;
    p.tiles_m = (p.m + BM - 1) / BM;
    if (size_t(p.tiles_n) * size_t(p.tiles_m) > 0x7fffffffu)
        return hipErrorInvalidValue;
    fp8_dma_kernel<TM, WM, STAGES, TN, NARROW>
        <<<dim3(unsigned(p.tiles_n) * unsigned(p.tiles_m), unsigned(splits)), 128 * WM, 0, stream>>>(p);
    return launch_status();
}

const TnVariant variants[] = {
    {"fp8dma256x256x128w8", 256, 256, 128, 512},
    {"fp8dma256x128x128w8", 256, 128, 128, 512},
    {"fp8dma256x128x128w4", 256, 128, 128, 256},
    {"fp8dma256x64x128w4", 256, 64, 128, 256},
    {"fp8dma256x128x128s3w8", 256, 128, 128, 512},
    {"fp8dma256x128x128s3w4", 256, 128, 128, 256},
    {"fp8dma256x64x128s3w4", 256, 64, 128, 256},
    {"fp8dma192x128x128s3w8", 192, 128, 128, 512},
    {"fp8dma192x256x128w8", 192, 256, 128, 512},
    {"fp8dma192x64x128s3w4", 192, 64, 128, 256},
    // the same tiles on the 16 x 16 x 128 matrix instruction (variants 0, 4, 6, 7, 8, 9)
    {"fp8dma16-256x256x128w8", 256, 256, 128, 512},
    {"fp8dma16-256x128x128s3w8", 256, 128, 128, 512},
    {"fp8dma16-256x64x128s3w4", 256, 64, 128, 256},
    {"fp8dma16-192x128x128s3w8", 192, 128, 128, 512},
    {"fp8dma16-192x256x128w8", 192, 256, 128, 512},
    {"fp8dma16-192x64x128s3w4", 192, 64, 128, 256},
    // four wavefronts, one per SIMD, K loop in generated assembly (fp8_wave4.hip)
    {"fp8wave4-192x256x128", 192, 256, 128, 256},
};
} // namespace

int fp8_dma_variant_count() { return int(sizeof(variants) / sizeof(variants[0])); }
const TnVariant &fp8_dma_variant(int index) { return variants[index]; }

// Needs outputs % 4 == 0 (8-byte BF16 stores) and 16-byte aligned a, w (rows are multiples of 128).
// With split_k > 1 the K groups are divided evenly over that many workgroups per tile, each writes
// an FP32 plane of `partials` ([split_k, rows, outputs], 16-byte aligned) and the planes are summed
// in index order before the one BF16 rounding: few tokens leave most compute units without a tile
// otherwise (256 tokens by 18432 outputs are 72 tiles of 256 x 256).
namespace
{
hipError_t launch_rows(hipStream_t stream, int variant, int splits, const Fp8DmaParams &p)
{
    switch (variant) {
    case 0: return launch_one<2, 4, 2>(stream, p, splits);
    case 1: return launch_one<1, 4, 2>(stream, p, splits);
    case 2: return launch_one<2, 2, 2>(stream, p, splits);
    case 3: return launch_one<1, 2, 2>(stream, p, splits);
    case 4: return launch_one<1, 4, 3>(stream, p, splits);
    case 5: return launch_one<2, 2, 3>(stream, p, splits);
    case 6: return launch_one<1, 2, 3>(stream, p, splits);
    case 7: return launch_one<1, 4, 3, 3>(stream, p, splits);
    case 8: return launch_one<2, 4, 2, 3>(stream, p, splits);
    case 9: return launch_one<1, 2, 3, 3>(stream, p, splits);
    case 10: return launch_one<2, 4, 2, 4, true>(stream, p, splits);
    case 11: return launch_one<1, 4, 3, 4, true>(stream, p, splits);
    case 12: return launch_one<1, 2, 3, 4, true>(stream, p, splits);
    case 13: return launch_one<1, 4, 3, 3, true>(stream, p, splits);
    case 14: return launch_one<2, 4, 2, 3, true>(stream, p, splits);
    case 15: return launch_one<1, 2, 3, 3, true>(stream, p, splits);
    case 16:
        if (splits != 1)
            return hipErrorInvalidValue;
        return launch_fp8_wave4(stream, p.m, p.n, p.k, p.a, p.a_scale, p.w, p.w_scale, p.out, p.out_pitch);
    default: return hipErrorInvalidValue;
    }
}
} // namespace

// tail_outputs > 0 (undivided K only): the last tail_outputs outputs, starting at a multiple of 128,
// run on tail_variant in a launch of their own, so that both launches are whole rounds of
// workgroups where one tiling would end in a partly filled round.
hipError_t launch_fp8_dma(hipStream_t stream, int variant, int split_k, int rows, int outputs, int inner,
                          const void *a, const float *a_scale, const void *w, const float *w_scale,
                          void *out, float *partials, int tail_variant, int tail_outputs)
{
    if (outputs % 4 || inner % 128 || reinterpret_cast<uintptr_t>(out) % 8)
        return hipErrorInvalidValue;
    if (split_k < 1 || split_k > 64 || split_k > inner / 128 || (split_k > 1 && !partials) ||
        reinterpret_cast<uintptr_t>(partials) % 16)
        return hipErrorInvalidValue;
    if (size_t(256) * size_t(inner) >= (size_t(1) << 32))
        return hipErrorInvalidValue;
    if (tail_outputs < 0 || tail_outputs >= outputs || (tail_outputs && (split_k > 1 || (outputs - tail_outputs) % 128)))
        return hipErrorInvalidValue;
    Fp8DmaParams p;
    p.w = static_cast<const unsigned char *>(w);
    p.a = static_cast<const unsigned char *>(a);
    p.w_scale = w_scale;
    p.a_scale = a_scale;
    p.out = static_cast<unsigned short *>(out);
    p.n = outputs - tail_outputs;
    p.out_pitch = outputs;
    p.m = rows;
    p.k = inner;
    p.groups = inner / 128;
    p.scale_blocks = (p.n + 127) / 128;
    p.tiles_n = p.tiles_m = 0;
    p.split_groups = (p.groups + split_k - 1) / split_k;
    // every blockIdx.y must own at least one group
    const int splits = (p.groups + p.split_groups - 1) / p.split_groups;
    p.partials = splits > 1 ? partials : nullptr;
    hipError_t status = launch_rows(stream, variant, splits, p);
    if (status == hipSuccess && tail_outputs) {
        const size_t first = size_t(p.n);
        p.w += first * size_t(inner);
        p.w_scale += (first / 128) * size_t(p.groups);
        p.out += first;
        p.n = tail_outputs;
        p.scale_blocks = (tail_outputs + 127) / 128;
        status = launch_rows(stream, tail_variant, 1, p);
    }
    if (status != hipSuccess || splits == 1)
        return status;
    return launch_fp8_split_sum(stream, splits, size_t(rows) * size_t(outputs), partials, out);
}
} // namespace camblas_hip
