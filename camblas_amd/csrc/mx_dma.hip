// Prefill-sized E8M0 block-scaled product on the gfx950 matrix cores with hardware scales:
// out[M,N] = x[M,K] . w[N,K]^T, x E4M3 with one E8M0 scale per 32 (or 128) inputs, w E4M3 with one
// scale per 32 x 32 block or packed E2M1 with one scale per row and 32 inputs, BF16 out; plain and
// grouped (contract: ref include/camblas_cuda.h:110-167, src/cuda/backend.cu:1165-1191, :1258-1303;
// value semantics: tests/test_quantized.py:12-50 of the reference).
//
// v_mfma_scale_f32_32x32x64_f8f6f4 multiplies a 32 x 64 by a 64 x 32 tile and applies one E8M0 scale
// per row and 32 inputs on either side, so the whole scaling rule is inside the instruction and the
// accumulators are never touched by the vector ALU. Operand layout (checked against a host product
// of random operands and scales): of the 64 K positions of one instruction, lane group c = lane/32
// of an 8-bit operand holds positions 16c..16c+15 in its first 16 bytes and 32+16c..32+16c+15 in
// its second 16 bytes; a 4-bit operand holds positions 32c..32c+31 in its first 16 bytes; the scale
// byte supplied by lane group g applies to positions 32g..32g+31 of that lane's row.
//
// Structure: as the FP32-scaled FP8 prefill kernel. A workgroup of 2 x WM wavefronts owns
// (64*TN) weight rows x (32*WM*TM) tokens, a K step is 128 inputs (128 bytes of an E4M3 row, 64 of
// an E2M1 row), operands go straight from memory into XOR-swizzled LDS stages STAGES-1 steps ahead
// (buffer_load ... lds; rows outside the matrix read as zero). The four scale bytes of a row and
// step are one 32-bit word, read from the address rounded down to four bytes; v_alignbyte of two
// consecutive words undoes any misalignment of the scale pointer, which is the same for every row
// because a scale row is a multiple of four bytes long. The words reach the lanes through LDS slabs:
// once per round of three or four steps every wavefront copies, with one direct-to-LDS load, the
// next four words of 64 scale rows (16 bytes per lane: the rows of the tile's E2M1 weights and of its
// tokens; for E4M3 weights the tile's 32-row blocks, one word per lane), and a lane reads the word
// of its row two steps ahead of its use. A lane that fetched its row's word for every step itself
// would request a cache line per lane and step, the same line for 32 steps (measured 7 to 25 % of
// the kernel). Tokens with one scale byte per 128 inputs keep a byte load per lane and step.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"
#include "mx_grouped.hpp"

namespace camblas_hip
{
namespace
{
struct MxDmaParams {
    const unsigned char *input, *input_scale, *weight, *weight_scale;
    unsigned short *out;
    int rows, outputs, inner, steps; // steps = inner / 128
    int tiles_n, tiles_m;
    // grouped form
    const unsigned long long *metadata;
    const int32_t *active, *counts;
    int weight_groups, groups;
    int out_pitch; // elements between tokens in `out` (the outputs of the whole product)
    // plain product with K divided over gridDim.y workgroups per tile: each takes `share_steps` steps
    // and leaves its FP32 sums in plane blockIdx.y of `planes` ([share][token][output of this launch])
    float *planes;
    int share_steps;
};

// WIDE_X: one activation scale per 128 inputs (one byte per step) instead of one per 32
template <bool PACKED, bool WIDE_X, bool GROUPED, int TN, int TM, int WM, int STAGES, int RING>
__global__ __launch_bounds__(128 * WM) void mx_dma_kernel(MxDmaParams p)
{
    static_assert(RING >= 2 && RING <= 4, "weight fragments in flight");
    static_assert(STAGES == 2 || STAGES == 3, "two or three LDS stages");
    static_assert(PACKED || !WIDE_X, "128-input activation scales go with E2M1 weights only");
    constexpr int WAVES = 2 * WM, BK = 128;
    constexpr int CHW = PACKED ? 4 : 8, CHX = 8;        // 16-byte chunks of a row per step
    constexpr int W_ROWS = 64 / CHW, X_ROWS = 64 / CHX; // rows covered by one wavefront load
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    constexpr int A_ITERS = BN / (WAVES * W_ROWS), B_ITERS = BM / (WAVES * X_ROWS);
    static_assert(BN % (WAVES * W_ROWS) == 0 && BM % (WAVES * X_ROWS) == 0, "loads");
    static_assert((WAVES * W_ROWS) % 16 == 0 && (WAVES * X_ROWS) % 16 == 0, "row step keeps the swizzle");
    constexpr int W_SLOTS = BN * CHW, SLOTS = W_SLOTS + BM * CHX, LOADS = A_ITERS + B_ITERS;
    // scale rows whose words travel through LDS slabs: the weight rows when every row has its own
    // scales (E2M1), the token rows unless the tokens have one scale byte per step; for E4M3 weights
    // the tile's 32-row blocks have a small slab of their own
    constexpr int SLAB_ROWS = (PACKED ? BN : 0) + (WIDE_X ? 0 : BM);
    constexpr int PIECES = SLAB_ROWS / 64; // 64 rows per wavefront load, 16 bytes (four steps) per row
    constexpr int PERIOD = STAGES == 3 ? 3 : 4; // steps between slabs: a whole number of rounds
    constexpr int BLOCK_SLAB = PACKED ? 0 : 16; // u32x4 of the block slab: 16 blocks x 4 words
    static_assert(SLAB_ROWS % 64 == 0 && (PACKED ? BN : 0) % 64 == 0 && PIECES <= WAVES && BN / 32 <= 16,
                  "one load per wavefront and slab");
    __shared__ u32x4_t lds[STAGES * SLOTS + 2 * SLAB_ROWS + 2 * BLOCK_SLAB];
    auto stage_at = [&](int index) { return lds + index * SLOTS; };
    auto slab_at = [&](int slab) { return lds + STAGES * SLOTS + (slab & 1) * SLAB_ROWS; };
    auto block_slab_at = [&](int slab) { return lds + STAGES * SLOTS + 2 * SLAB_ROWS + (slab & 1) * BLOCK_SLAB; };

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    int tile_n, tile_m, group = 0;
    if constexpr (GROUPED) {
        grouped_tile<BM>(p, lane, blockIdx.x, group, tile_n, tile_m);
    } else {
        xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    }
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int wn = wave % 2, wm = wave / 2;
    const int scale_pitch = p.inner / 32; // bytes of a row of 32-input scales: a multiple of four

    const unsigned char *input = p.input, *input_scale = p.input_scale, *weight = p.weight,
                        *weight_scale = p.weight_scale;
    unsigned short *out = p.out;
    int valid_rows = p.rows;
    if constexpr (GROUPED) {
        // ref: include/camblas_cuda.h:156-167 — weights come from a device table indexed by
        // active[group]; invalid indices and rows at or beyond counts[group] produce zeros
        // (values that are the same for the whole workgroup are moved to scalar registers)
        const int index = __builtin_amdgcn_readfirstlane(p.active[group]);
        const int count = __builtin_amdgcn_readfirstlane(p.counts[group]);
        valid_rows = index >= 0 && index < p.weight_groups ? min(max(count, 0), p.rows) : 0;
        input += size_t(group) * p.rows * p.inner;
        input_scale += size_t(group) * p.rows * (WIDE_X ? p.steps : scale_pitch);
        out += size_t(group) * p.rows * p.out_pitch;
        if (m0 >= valid_rows) { // nothing to multiply: this tile of the output is zero
            for (int item = thread; item < BM * (BN / 4); item += 128 * WM) {
                const int m = m0 + item / (BN / 4), n = n0 + (item % (BN / 4)) * 4;
                if (m < p.rows && n < p.outputs)
                    *reinterpret_cast<u32x2_t *>(out + size_t(m) * p.out_pitch + n) = u32x2_t{0u, 0u};
            }
            return;
        }
        weight = reinterpret_cast<const unsigned char *>(uniform(p.metadata[2 * size_t(index)]));
        weight_scale = reinterpret_cast<const unsigned char *>(uniform(p.metadata[2 * size_t(index) + 1]));
    }

    // a share of K: the same kernel over steps first_step .. first_step + steps - 1, by moving every
    // operand to its first step (scale words are four bytes per step, so their alignment is kept)
    constexpr unsigned W_STEP_BYTES = PACKED ? BK / 2 : BK;
    const int first_step = GROUPED ? 0 : int(blockIdx.y) * p.share_steps;
    const int steps = GROUPED ? p.steps : (p.steps - first_step < p.share_steps ? p.steps - first_step : p.share_steps);
    weight += size_t(first_step) * W_STEP_BYTES;
    input += size_t(first_step) * BK;
    weight_scale += size_t(first_step) * 4;
    input_scale += size_t(first_step) * (WIDE_X ? 1 : 4);

    // ---- operand loads. Lane -> (row inside one wavefront load, swizzled chunk); successive loads
    // of a thread are WAVES*rows apart, which leaves the swizzle unchanged, so one lane offset
    // serves all of them and the row advance goes into the wave-uniform offset.
    const unsigned w_pitch = PACKED ? unsigned(p.inner) / 2 : unsigned(p.inner);
    const int w_load_row = wave * W_ROWS + lane / CHW, x_load_row = wave * X_ROWS + lane / CHX;
    const unsigned w_lane_off =
        unsigned(w_load_row) * w_pitch + unsigned(((lane % CHW) ^ lds_swizzle<CHW>(w_load_row)) * 16);
    const unsigned x_lane_off = unsigned(x_load_row) * unsigned(p.inner) +
                                unsigned(((lane % CHX) ^ lds_swizzle<CHX>(x_load_row)) * 16);
    const unsigned w_row_step = unsigned(WAVES * W_ROWS) * w_pitch;
    const unsigned x_row_step = unsigned(WAVES * X_ROWS) * unsigned(p.inner);
    const int w_rows = p.outputs - n0 < BN ? p.outputs - n0 : BN;
    const int x_rows = valid_rows - m0 < BM ? valid_rows - m0 : BM;
    const __amdgpu_buffer_rsrc_t w_resource = make_resource(
        weight + size_t(n0) * w_pitch, unsigned(w_rows) * w_pitch - unsigned(first_step) * W_STEP_BYTES);
    const __amdgpu_buffer_rsrc_t x_resource = make_resource(
        input + size_t(m0) * p.inner, unsigned(x_rows) * unsigned(p.inner) - unsigned(first_step) * BK);
    const int last_step = steps - 1;
    int load_step = 0;
    auto issue_one = [&](u32x4_t *stage, int index) {
        if (index < A_ITERS)
            load_to_lds(w_resource, w_lane_off,
                        unsigned(load_step) * W_STEP_BYTES + unsigned(index) * w_row_step,
                        stage + (index * WAVES + wave) * 64);
        else
            load_to_lds(x_resource, x_lane_off,
                        unsigned(load_step) * BK + unsigned(index - A_ITERS) * x_row_step,
                        stage + W_SLOTS + ((index - A_ITERS) * WAVES + wave) * 64);
    };
    auto advance = [&]() { load_step = load_step < last_step ? load_step + 1 : last_step; };
    auto issue = [&](u32x4_t *stage) {
#pragma unroll
        for (int index = 0; index < LOADS; ++index)
            issue_one(stage, index);
        advance();
    };

    // ---- scales: per lane (operand row lane%32) one 32-bit word per 32-row tile and step, taken
    // from the 4-byte aligned address at or below the row's scales. Slab number i holds words
    // PERIOD * i .. PERIOD * i + 3 of every listed row (weight rows of the tile first, then its token
    // rows), lane l of piece q the row 64 q + l; it is loaded when slab i - 1 comes into use, into
    // the buffer that slab i - 2 has left. Loads and reads are kept out of the compiler's
    // bookkeeping (it would make every LDS read that such a load might have written wait for all
    // outstanding loads, the stage fills included): a slab load is older than the fills of the step
    // that follows, whose wait therefore covers it, at least two steps before its first word is
    // read; a word is read a few instructions before a step's wait and used after it.
    const int frag_row = lane % 32, half = lane / 32;
    const unsigned w_skew = unsigned(reinterpret_cast<uintptr_t>(weight_scale)) & 3u;
    const unsigned x_skew = WIDE_X ? 0u : unsigned(reinterpret_cast<uintptr_t>(input_scale)) & 3u;
    const int piece = __builtin_amdgcn_readfirstlane(wave) % (PIECES > 0 ? PIECES : 1);
    const bool piece_of_weights = PACKED && piece * 64 < BN; // wave-uniform
    unsigned slab_lane_off = 0;
    u32x4_t slab_resource = {0u, 0u, 0u, 0u};
    if constexpr (PIECES > 0) {
        const int listed = piece * 64 + lane;
        int row = piece_of_weights ? n0 + listed : m0 + listed - (PACKED ? BN : 0);
        const int rows = piece_of_weights ? p.outputs : valid_rows;
        row = row < rows ? row : rows - 1;
        slab_lane_off = unsigned(row) * unsigned(scale_pitch);
        const unsigned skew = piece_of_weights ? w_skew : x_skew;
        slab_resource = uniform_descriptor((piece_of_weights ? weight_scale : input_scale) - skew,
                                           unsigned(rows) * unsigned(scale_pitch) + (skew ? 4u : 0u) -
                                               unsigned(first_step) * 4u);
    }
    // E4M3 weights: one scale row per 32 weight rows; lane l brings word l % 4 of the slab for the
    // tile's block l / 4 (every wavefront issues the same load: same bytes to the same place)
    const int block_rows = (p.outputs + 31) / 32;
    const int lane_block = n0 / 32 + lane / 4 < block_rows ? n0 / 32 + lane / 4 : block_rows - 1;
    const unsigned block_lane_off = unsigned(lane_block) * unsigned(scale_pitch) + unsigned(lane % 4) * 4u;
    const u32x4_t block_resource =
        uniform_descriptor(weight_scale - w_skew, unsigned(block_rows) * unsigned(scale_pitch) + (w_skew ? 4u : 0u) -
                                                      unsigned(first_step) * 4u);
    auto load_slabs = [&](int slab) {
        if constexpr (PIECES > 0)
            load_to_lds_untracked(slab_resource, slab_lane_off, unsigned(slab * PERIOD) * 4u,
                                  slab_at(slab) + piece * 64);
        if constexpr (!PACKED)
            load_word_to_lds_untracked(block_resource, block_lane_off, unsigned(slab * PERIOD) * 4u,
                                       block_slab_at(slab));
    };
    int ws_index[TN], xs_index[TM]; // word index of this lane's row inside a slab buffer
#pragma unroll
    for (int i = 0; i < TN; ++i)
        ws_index[i] = PACKED ? ((wn * TN + i) * 32 + frag_row) * 4 : (wn * TN + i) * 4;
#pragma unroll
    for (int j = 0; j < TM; ++j)
        xs_index[j] = ((PACKED ? BN : 0) + (wm * TM + j) * 32 + frag_row) * 4;
    // word number `step` of the weight tile i / token tile j (reads of steps past the end return
    // words that are never used)
    auto weight_word = [&](int i, int step) {
        const unsigned *words = reinterpret_cast<const unsigned *>(PACKED ? slab_at(step / PERIOD) : block_slab_at(step / PERIOD));
        return lds_read_unordered(words + ws_index[i] + step % PERIOD);
    };
    auto token_word = [&](int j, int step) {
        const unsigned *words = reinterpret_cast<const unsigned *>(slab_at(step / PERIOD));
        return lds_read_unordered(words + xs_index[j] + step % PERIOD);
    };
    unsigned xs_byte_offset[TM]; // one scale byte per token and step: loaded a step ahead
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        int m = m0 + (wm * TM + j) * 32 + frag_row;
        m = m < valid_rows ? m : valid_rows - 1;
        xs_byte_offset[j] = unsigned(m) * unsigned(p.steps);
    }
    unsigned ws_now[TN], ws_next[TN], xs_now[TM], xs_next[TM];
    auto fetch_token_bytes = [&](int step, unsigned (&x)[TM]) {
        const int x_byte = step < last_step ? step : last_step;
        if constexpr (WIDE_X) {
#pragma unroll
            for (int j = 0; j < TM; ++j)
                x[j] = unsigned(input_scale[xs_byte_offset[j] + unsigned(x_byte)]);
        }
    };

    const int w_swizzle = lds_swizzle<CHW>(frag_row), x_swizzle = lds_swizzle<CHX>(frag_row);
    const int w_frag_base = (wn * TN * 32 + frag_row) * CHW;
    const int x_frag_base = W_SLOTS + (wm * TM * 32 + frag_row) * CHX;
    f32x16_t acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    // operand of the instruction that covers inputs 64*ks .. 64*ks+63 of the step
    auto fragment8 = [&](const u32x4_t *stage, int base, int swizzle, int ks) {
        const u32x4_t lo = stage[base + ((ks * 4 + half) ^ swizzle)];
        const u32x4_t hi = stage[base + ((ks * 4 + 2 + half) ^ swizzle)];
        return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                       int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
    };
    auto fragment4 = [&](const u32x4_t *stage, int base, int swizzle, int ks) {
        const u32x4_t lo = stage[base + ((ks * 2 + half) ^ swizzle)];
        return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]), 0, 0, 0, 0};
    };
    auto weight_fragment = [&](const u32x4_t *stage, int tile, int ks) {
        if constexpr (PACKED)
            return fragment4(stage, w_frag_base + tile * 32 * CHW, w_swizzle, ks);
        else
            return fragment8(stage, w_frag_base + tile * 32 * CHW, w_swizzle, ks);
    };

    // One K step, as two halves of 64 inputs. LDS reads return long after one or two matrix
    // instructions have issued, so the weight fragments (one per 32-row tile and half) are read
    // RING-1 fragments ahead of their use into a ring of register buffers, and the token
    // fragments of the second half while the first half is multiplied; the fills of the stage
    // STAGES-1 ahead are issued between the matrix instructions.
    auto multiply = [&](const u32x4_t *stage, u32x4_t *fill, const unsigned (&w_scale)[TN],
                        const unsigned (&x_scale)[TM]) {
        constexpr int PARTS = TN * 2, OPS = PARTS * TM;
        static_assert(LOADS <= OPS, "at most one fill per matrix instruction");
        // (a ring of two leaves no registers for both halves' token fragments: there the second
        // half's are read into the first half's registers when the first half is done)
        constexpr int XB = RING > 2 ? 2 : 1;
        i32x8_t w_frag[RING], x_frag[XB][TM];
#pragma unroll
        for (int t = 0; t < TM; ++t)
            x_frag[0][t] = fragment8(stage, x_frag_base + t * 32 * CHX, x_swizzle, 0);
#pragma unroll
        for (int part = 0; part < RING - 1 && part < PARTS; ++part)
            w_frag[part] = weight_fragment(stage, part % TN, part / TN);
#pragma unroll
        for (int op = 0; op < OPS; ++op) {
            const int part = op / TM, ks = part / TN, i = part % TN, j = op % TM;
            __builtin_amdgcn_sched_barrier(0);
            if (j == 0 && part + RING - 1 < PARTS)
                w_frag[(part + RING - 1) % RING] =
                    weight_fragment(stage, (part + RING - 1) % TN, (part + RING - 1) / TN);
            if (op == (XB == 2 ? TM : OPS / 2)) { // second half's tokens: read during the first half
#pragma unroll
                for (int t = 0; t < TM; ++t)
                    x_frag[XB - 1][t] = fragment8(stage, x_frag_base + t * 32 * CHX, x_swizzle, 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (ks == 0) // (the byte selects are immediates of the instruction)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    w_frag[part % RING], x_frag[0][j], acc[i][j], PACKED ? 4 : 0, 0, 0, int(w_scale[i]),
                    0, int(x_scale[j]));
            else
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    w_frag[part % RING], x_frag[XB - 1][j], acc[i][j], PACKED ? 4 : 0, 0, 2, int(w_scale[i]),
                    WIDE_X ? 0 : 2, int(x_scale[j]));
            __builtin_amdgcn_sched_barrier(0);
            // One fill per matrix instruction from the start of the step; the short steps of the
            // 128-token tile spread them evenly instead (measured: 10 % faster there, slower for
            // the long steps).
#pragma unroll
            for (int index = 0; index < LOADS; ++index)
                if ((STAGES == 3 && TM == 1 ? index * OPS / LOADS : index) == op)
                    issue_one(fill, index);
        }
        __builtin_amdgcn_sched_barrier(0);
        advance();
    };

    // The scale byte of this lane's block (lane group g supplies the scale of inputs 32g..32g+31 of
    // an instruction) is byte 2*ks + half of the step's word: the word is shifted by `half` bytes
    // and the instruction's byte select takes byte 2*ks.
    auto step = [&](int g, const u32x4_t *current, u32x4_t *fill) {
        fetch_token_bytes(g + 1, xs_next);
        unsigned w_scale[TN], x_scale[TM];
#pragma unroll
        for (int i = 0; i < TN; ++i)
            w_scale[i] = __builtin_amdgcn_alignbyte(ws_next[i], ws_now[i], w_skew) >> (8 * half);
#pragma unroll
        for (int j = 0; j < TM; ++j)
            x_scale[j] = WIDE_X ? xs_now[j]
                                : __builtin_amdgcn_alignbyte(xs_next[j], xs_now[j], x_skew) >> (8 * half);
        __builtin_amdgcn_sched_barrier(0);
        multiply(current, fill, w_scale, x_scale);
        // words of step g + 2 (their slab landed at an earlier step's wait); this step's wait
        // covers the reads
        unsigned ws_load[TN], xs_load[TM];
#pragma unroll
        for (int i = 0; i < TN; ++i)
            ws_load[i] = weight_word(i, g + 2);
#pragma unroll
        for (int j = 0; j < TM; ++j)
            xs_load[j] = WIDE_X ? xs_next[j] : token_word(j, g + 2);
        pipeline_barrier<(STAGES - 2) * LOADS>();
        tie_after_wait(ws_load, xs_load);
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            ws_now[i] = ws_next[i];
            ws_next[i] = ws_load[i];
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            xs_now[j] = xs_next[j];
            if constexpr (!WIDE_X)
                xs_next[j] = xs_load[j];
        }
    };

    load_slabs(0); // (the oldest loads: complete at the first wait)
    fetch_token_bytes(0, xs_now);
#pragma unroll
    for (int s = 0; s + 1 < STAGES; ++s) {
        __builtin_amdgcn_sched_barrier(0);
        issue(stage_at(s));
    }
    pipeline_barrier<(STAGES - 2) * LOADS>();
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        ws_now[i] = weight_word(i, 0);
        ws_next[i] = weight_word(i, 1);
    }
    if constexpr (!WIDE_X) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            xs_now[j] = token_word(j, 0);
            xs_next[j] = token_word(j, 1);
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
    tie_after_wait(ws_now, ws_next);
    if constexpr (!WIDE_X)
        tie_after_wait(xs_now, xs_next);
    // whole rounds of STAGES steps run without a branch between the steps; the remainder follows
    int g = 0;
    for (int slab = 1; g + STAGES <= steps; ++slab) {
        load_slabs(slab);
        const int end = slab * PERIOD < steps ? slab * PERIOD : steps;
        for (; g + STAGES <= end; g += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; ++s)
                step(g + s, stage_at(s), stage_at((s + STAGES - 1) % STAGES));
        }
    }
#pragma unroll
    for (int s = 0; s + 1 < STAGES; ++s)
        if (g + s < steps)
            step(g + s, stage_at(s), stage_at((s + STAGES - 1) % STAGES));
    wait_loads<0>();

    if constexpr (!GROUPED) {
        if (gridDim.y > 1) { // a share of K: the plain sums, for sum_planes_kernel
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int m = m0 + (wm * TM + j) * 32 + frag_row;
                float *row = p.planes + (size_t(blockIdx.y) * p.rows + m) * p.outputs + n0 + wn * TN * 32 + half * 4;
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int offset = i * 32 + q * 8;
                        if (m < p.rows && n0 + wn * TN * 32 + half * 4 + offset < p.outputs)
                            *reinterpret_cast<f32x4_t *>(row + offset) = f32x4_t{
                                acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                    }
            }
            return;
        }
    }

    // ---- epilogue: accumulator register 4q+e of lane l is feature 8q + 4*(l/32) + e, token l%32
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + (wm * TM + j) * 32 + frag_row;
        const bool live = !GROUPED || m < valid_rows; // padding rows of a group are written as zeros
        unsigned short *row = out + size_t(m) * p.out_pitch + n0 + wn * TN * 32 + half * 4;
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int offset = i * 32 + q * 8;
                if (m < p.rows && n0 + wn * TN * 32 + half * 4 + offset < p.outputs) {
                    u32x2_t packed = {pack_bf16x2(acc[i][j][q * 4], acc[i][j][q * 4 + 1]),
                                      pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3])};
                    if (!live)
                        packed = u32x2_t{0u, 0u};
                    *reinterpret_cast<u32x2_t *>(row + offset) = packed;
                }
            }
        }
    }
}

// out = plane 0 + plane 1 + ... of a divided K, four outputs per thread, the planes added in index
// order so that the result does not depend on scheduling.
__global__ __launch_bounds__(256) void sum_planes_kernel(MxDmaParams p, int shares)
{
    const size_t quad = size_t(blockIdx.x) * 256 + threadIdx.x, per_row = size_t(p.outputs / 4);
    if (quad >= per_row * size_t(p.rows))
        return;
    const size_t m = quad / per_row, n = quad % per_row * 4, plane = size_t(p.rows) * p.outputs;
    const float *source = p.planes + m * p.outputs + n;
    f32x4_t sum = *reinterpret_cast<const f32x4_t *>(source);
    for (int share = 1; share < shares; ++share) {
        const f32x4_t more = *reinterpret_cast<const f32x4_t *>(source + share * plane);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            sum[e] += more[e];
    }
    const u32x2_t packed = {pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3])};
    *reinterpret_cast<u32x2_t *>(p.out + m * p.out_pitch + n) = packed;
}

template <bool PACKED, bool WIDE_X, bool GROUPED, int TN, int TM, int WM, int STAGES, int RING>
hipError_t launch_one(hipStream_t stream, MxDmaParams p, int groups, int shares)
{
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    p.tiles_n = (p.outputs + BN - 1) / BN;
    p.tiles_m = (p.rows + BM - 1) / BM;
    const size_t tiles = size_t(p.tiles_n) * size_t(p.tiles_m) * size_t(GROUPED ? groups : 1);
    if (tiles > 0x7fffffffu || (GROUPED && shares != 1))
        return hipErrorInvalidValue;
    p.groups = groups;
    p.share_steps = (p.steps + shares - 1) / shares;
    shares = (p.steps + p.share_steps - 1) / p.share_steps; // no empty share
    dim3 grid{unsigned(tiles), unsigned(shares)};
    mx_dma_kernel<PACKED, WIDE_X, GROUPED, TN, TM, WM, STAGES, RING>
        <<<grid, 128 * WM, 0, stream>>>(p);
    const hipError_t status = launch_status();
    if (shares == 1 || status != hipSuccess)
        return status;
    const size_t quads = size_t(p.rows) * size_t(p.outputs / 4);
    sum_planes_kernel<<<unsigned((quads + 255) / 256), 256, 0, stream>>>(p, shares);
    return launch_status();
}

// variant 0: 256 weight rows x 256 tokens (two stages for E4M3 weights, three for E2M1);
// variant 1: 256 x 128, three stages; variant 2: 192 x 256, two stages, E4M3 weights only (a
// wavefront load covers 16 rows of packed weights: 192 rows are not a whole number of rounds);
// variant 3: 128 x 128, three stages (twice the workgroups of variant 1 for small products)
template <bool PACKED, bool WIDE_X, bool GROUPED>
hipError_t launch_variant(hipStream_t stream, const MxDmaParams &p, int groups, int variant, int shares = 1)
{
    switch (variant) {
    case 0: return launch_one<PACKED, WIDE_X, GROUPED, 4, 2, 4, PACKED ? 3 : 2, PACKED || GROUPED ? 2 : 3>(stream, p, groups, shares);
    case 1: return launch_one<PACKED, WIDE_X, GROUPED, 4, 1, 4, 3, 4>(stream, p, groups, shares);
    case 2:
        if constexpr (!PACKED)
            return launch_one<false, false, GROUPED, 3, 2, 4, 2, 3>(stream, p, groups, shares);
        return hipErrorInvalidValue;
    case 3: return launch_one<PACKED, WIDE_X, GROUPED, 2, 1, 4, 3, 4>(stream, p, groups, shares);
    default: return hipErrorInvalidValue;
    }
}
} // namespace

int mx_dma_variant_count() { return 5; } // (4: the four-wavefront tile of mx_wave4.hip)

// The prefill kernel's conditions: K a multiple of 128, 16-byte aligned operands, an 8-byte aligned
// output (scale pointers may have any alignment).
bool mx_dma_supported(int outputs, int inner, const void *input, const void *weight, const void *out)
{
    // (32-bit byte offsets: a 256-row operand tile, and the scale bytes of all rows of an operand)
    return inner % 128 == 0 && outputs % 4 == 0 && size_t(256) * size_t(inner) < (size_t(1) << 32) &&
           (size_t(outputs) + 65536) * size_t(inner / 32) < (size_t(1) << 32) &&
           reinterpret_cast<uintptr_t>(out) % 8 == 0 && reinterpret_cast<uintptr_t>(input) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(weight) % 16 == 0;
}

// groups == 0: plain product; >= 1: grouped (weights and their scales from the device table)
namespace
{
// The plain product over outputs first .. first + count - 1 of `outputs` (first a multiple of 32).
hipError_t launch_mx_dma_rows(hipStream_t stream, int variant, bool packed, int rows, int outputs, int first,
                              int count, int inner, int activation_block, const void *input,
                              const void *input_scale, const void *weight, const void *weight_scale, void *out)
{
    const size_t scale_pitch = size_t(inner / 32), weight_pitch = packed ? size_t(inner) / 2 : size_t(inner);
    if (variant == 4) { // four wavefronts per workgroup, K loop in generated assembly
        if (activation_block != 32)
            return hipErrorInvalidValue;
        return launch_mx_wave4(stream, packed, rows, count, inner, input, input_scale,
                               static_cast<const unsigned char *>(weight) + size_t(first) * weight_pitch,
                               static_cast<const unsigned char *>(weight_scale) + size_t(packed ? first : first / 32) * scale_pitch,
                               static_cast<unsigned short *>(out) + first, outputs);
    }
    MxDmaParams p;
    p.input = static_cast<const unsigned char *>(input);
    p.input_scale = static_cast<const unsigned char *>(input_scale);
    p.weight = static_cast<const unsigned char *>(weight) + size_t(first) * weight_pitch;
    p.weight_scale = static_cast<const unsigned char *>(weight_scale) + size_t(packed ? first : first / 32) * scale_pitch;
    p.out = static_cast<unsigned short *>(out) + first;
    p.rows = rows;
    p.outputs = count;
    p.out_pitch = outputs;
    p.inner = inner;
    p.steps = inner / 128;
    p.tiles_n = p.tiles_m = 0;
    p.metadata = nullptr;
    p.active = p.counts = nullptr;
    p.weight_groups = 0;
    p.planes = nullptr;
    p.share_steps = 0;
    if (!packed)
        return launch_variant<false, false, false>(stream, p, 1, variant);
    return activation_block == 128 ? launch_variant<true, true, false>(stream, p, 1, variant)
                                   : launch_variant<true, false, false>(stream, p, 1, variant);
}
} // namespace

// tail_outputs > 0 (plain product only): the last tail_outputs outputs, starting at a multiple of 256,
// run on tail_variant in a launch of their own, so that both launches are whole rounds of
// workgroups where one tiling would end in a partly filled round.
// shares > 1 (plain product, one launch): K divided over that many workgroups per tile, with
// `planes` holding shares * rows * outputs floats.
hipError_t launch_mx_dma(hipStream_t stream, int variant, bool packed, int groups, int weight_groups,
                         int rows, int outputs, int inner, int activation_block, const void *input,
                         const void *input_scale, const void *weight, const void *weight_scale,
                         const void *metadata, const void *active, const void *counts, void *out,
                         int tail_variant, int tail_outputs, int shares, float *planes)
{
    if (!mx_dma_supported(outputs, inner, input, weight, out) ||
        (activation_block != 32 && !(packed && activation_block == 128)))
        return hipErrorInvalidValue;
    if (shares < 1 || shares > 64 || (shares > 1 && (!planes || groups != 0 || tail_outputs)) ||
        size_t(rows) * size_t(outputs / 4) > size_t(0x7fffffff) * 256)
        return hipErrorInvalidValue;
    if (tail_outputs) {
        if (groups != 0 || tail_outputs < 0 || tail_outputs >= outputs || (outputs - tail_outputs) % 256)
            return hipErrorInvalidValue;
        const int first = outputs - tail_outputs;
        hipError_t status = launch_mx_dma_rows(stream, variant, packed, rows, outputs, 0, first, inner, activation_block,
                                               input, input_scale, weight, weight_scale, out);
        if (status != hipSuccess)
            return status;
        return launch_mx_dma_rows(stream, tail_variant, packed, rows, outputs, first, tail_outputs, inner,
                                  activation_block, input, input_scale, weight, weight_scale, out);
    }
    if (variant == 4) {
        if (shares != 1)
            return hipErrorInvalidValue;
        if (groups != 0)
            return activation_block != 32 ? hipErrorInvalidValue
                                          : launch_mx_wave4(stream, packed, rows, outputs, inner, input, input_scale, nullptr,
                                                            nullptr, out, outputs, groups, weight_groups, metadata, active, counts);
        return launch_mx_dma_rows(stream, variant, packed, rows, outputs, 0, outputs, inner, activation_block, input,
                                  input_scale, weight, weight_scale, out);
    }
    MxDmaParams p;
    p.input = static_cast<const unsigned char *>(input);
    p.input_scale = static_cast<const unsigned char *>(input_scale);
    p.weight = static_cast<const unsigned char *>(weight);
    p.weight_scale = static_cast<const unsigned char *>(weight_scale);
    p.out = static_cast<unsigned short *>(out);
    p.rows = rows;
    p.outputs = outputs;
    p.out_pitch = outputs;
    p.inner = inner;
    p.steps = inner / 128;
    p.tiles_n = p.tiles_m = 0;
    p.metadata = static_cast<const unsigned long long *>(metadata);
    p.active = static_cast<const int32_t *>(active);
    p.counts = static_cast<const int32_t *>(counts);
    p.weight_groups = weight_groups;
    p.planes = planes;
    p.share_steps = 0;
    const bool wide = activation_block == 128;
    if (groups == 0) {
        if (!packed)
            return launch_variant<false, false, false>(stream, p, 1, variant, shares);
        return wide ? launch_variant<true, true, false>(stream, p, 1, variant, shares)
                    : launch_variant<true, false, false>(stream, p, 1, variant, shares);
    }
    if (!packed)
        return launch_variant<false, false, true>(stream, p, groups, variant);
    return wide ? launch_variant<true, true, true>(stream, p, groups, variant)
                : launch_variant<true, false, true>(stream, p, groups, variant);
}
} // namespace camblas_hip
