// Block-scaled (microscaling) linear with E8M0 scales: out[M,N] = x[M,K] . w[N,K]^T, x E4M3 with one
// E8M0 scale per 32 (or 128) inputs, w either E4M3 with one scale per 32 x 32 block or packed E2M1
// (two values per byte, low nibble first) with one scale per row and 32 inputs, FP32 accumulation,
// BF16 out; plus the grouped form that picks weights per group from a device table (contract: ref
// include/camblas_cuda.h:110-167, src/cuda/backend.cu:1165-1191, :1258-1303; value semantics pinned
// by the byte decoder of the reference's tests/test_quantized.py:12-50: a scale byte e means
// 2^(e-127), 255 means NaN).
//
// This is the operation gfx950's v_mfma_scale_f32_16x16x128_f8f6f4 implements natively: every lane
// supplies 32 consecutive K elements of its row (E4M3 or E2M1, chosen per operand) together with
// one E8M0 scale byte, and the instruction accumulates the scaled products in FP32. One 128-input
// group is one instruction per 16 x 16 tile, with no vector-ALU arithmetic at all.
//
// Operand layout of the instruction, as measured with single-element probes: call the 128 K
// positions of a group p and its four 32-input blocks b = p/32. A lane group c = lane/16 of a
// 4-bit operand holds positions 32c .. 32c+31; a lane group of an 8-bit operand holds positions
// 16c .. 16c+15 in its first 16 bytes and 64+16c .. 64+16c+15 in its second 16 bytes; and the scale
// byte supplied by lane group b applies to block b of that lane's row, whichever lanes hold the
// block's data. The loads below follow exactly this (an 8-bit lane reads two 16-byte pieces 64
// bytes apart), so one instruction handles E2M1 weights against E4M3 inputs with independent
// 32-input scales on both sides.
//
// The kernel streams the weights like the other decode kernels: a workgroup owns 16*NT weight rows
// for the whole K extent and up to 16*MT tokens, its four wavefronts take 128-byte spans of the
// rows in turn (span 4s + wave: one group of E4M3 weights, two of E2M1), load their span of a tile
// with whole-line 128-bit loads (non-temporal), transpose it to the
// operand layout through a private swizzled LDS patch (no barrier: LDS operations of one wavefront
// execute in order) and the four partial sums are added in wavefront order at the end.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
struct MxParams {
    const unsigned char *input;
    const unsigned char *input_scale;
    const unsigned char *weight;
    const unsigned char *weight_scale;
    unsigned short *out;
    int rows, outputs, inner, scale_shift; // activation scale covers 32 << scale_shift inputs
    bool out_aligned;                      // out is 8-byte aligned: four features go out in one store
    // grouped form
    const unsigned long long *metadata;
    const int32_t *active, *counts;
    int weight_groups;
};

constexpr int WAVES = 4, GROUP = 128;
// The weight scales of a workgroup's rows (E2M1: a scale row per weight row; E4M3: one per 32 weight
// rows) are one contiguous byte range; when it fits this many bytes it is copied to LDS once with
// whole 1 KB direct-to-LDS loads instead of being gathered a byte per lane and step (16 cache lines
// per gather for 64 useful bytes).
constexpr int STAGED_SCALE_BYTES = 32768;
// The scale bytes of a workgroup's tokens are one contiguous byte range too and are copied with it
// when they fit this many bytes (a byte per lane, token tile and step from memory is a cache line
// per lane; measured 14 to 17 % of the E2M1 launch at 1 to 16 tokens).
constexpr int STAGED_TOKEN_BYTES = 16384;

template <bool PACKED, bool GROUPED, bool STAGED, int NT, int MT>
__global__ __launch_bounds__(WAVES * 64) void mx_stream_kernel(MxParams p)
{
    // A step of a wavefront covers one 128-byte line of every weight row: one 128-input group of
    // E4M3 weights, two consecutive groups of packed E2M1 weights (a half-line step would leave the
    // other half of each line to another wavefront's request).
    constexpr int SUB = PACKED ? 2 : 1;
    constexpr int STEP_INPUTS = GROUP * SUB;
    // (deeper queues for workgroups of few rows were measured: no gain, few rows per workgroup
    // lose to the per-workgroup start and end whatever the queue depth)
    constexpr int DEPTH = NT + MT * SUB <= 6 ? 3 : 2; // steps in flight, by registers per step
    // per wavefront: NT weight tiles and MT input tiles of 16 x 128 bytes; after the last step the
    // same memory holds the wavefront's partial sums
    __shared__ __attribute__((aligned(16))) u32x4_t tiles[WAVES][NT + MT][128];
    static_assert(NT * MT * 64 <= (NT + MT) * 128, "partial sums must fit the wavefront's tile memory");
    // (direct-to-LDS loads write whole 1 KB pieces: a piece of slack behind each range)
    __shared__ __attribute__((aligned(16))) unsigned char staged[STAGED ? STAGED_SCALE_BYTES + 1024 : 16];
    __shared__ __attribute__((aligned(16))) unsigned char staged_tokens[STAGED ? STAGED_TOKEN_BYTES + 1024 : 16];
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int row = lane % 16, chunk = lane / 16; // operand row / token, 32-input chunk of the group
    const int n0 = blockIdx.x * (NT * 16), m0 = blockIdx.y * (MT * 16);
    const int blocks = p.inner / 32, spans = (p.inner + STEP_INPUTS - 1) / STEP_INPUTS;
    const int steps = (spans + WAVES - 1) / WAVES; // spans per wavefront, padded
    const size_t weight_pitch = PACKED ? size_t(p.inner) / 2 : size_t(p.inner);

    const unsigned char *input = p.input, *input_scale = p.input_scale, *weight = p.weight,
                        *weight_scale = p.weight_scale;
    unsigned short *out = p.out;
    int valid_rows = p.rows;
    if constexpr (GROUPED) {
        // ref: include/camblas_cuda.h:156-167 — weights come from a device table indexed by
        // active[group]; invalid indices and rows at or beyond counts[group] produce zeros
        const int group = blockIdx.z;
        const int index = p.active[group];
        const int count = p.counts[group];
        valid_rows = index >= 0 && index < p.weight_groups ? min(max(count, 0), p.rows) : 0;
        input += size_t(group) * p.rows * p.inner;
        input_scale += size_t(group) * p.rows * (p.inner >> (5 + p.scale_shift));
        out += size_t(group) * p.rows * p.outputs;
        if (m0 >= valid_rows) { // nothing to multiply: this tile of the output is zero
            for (int index2 = thread; index2 < MT * 16 * NT * 16; index2 += WAVES * 64) {
                const int m = m0 + index2 / (NT * 16), n = n0 + index2 % (NT * 16);
                if (m < p.rows && n < p.outputs)
                    out[size_t(m) * p.outputs + n] = 0;
            }
            return;
        }
        weight = reinterpret_cast<const unsigned char *>(p.metadata[2 * size_t(index)]);
        weight_scale = reinterpret_cast<const unsigned char *>(p.metadata[2 * size_t(index) + 1]);
    }

    // ---- per-lane sources. Tiles of 16 rows x 128 bytes (weights and inputs alike) are loaded with
    // eight lanes per line, two loads per lane (rows r and r + 8), and transposed to the operand
    // layout through LDS: loading them straight in the operand layout would touch every line from
    // eight quarter-wave passes.
    // Rows are addressed by byte offsets inside descriptors of the workgroup's existing weight rows
    // and token rows; a row past the end, and every load of a step past the end of K, gets an offset
    // outside the descriptor, which reads as zero without a memory request (an existing row read in
    // its place is requested again while its first request is in flight, which holds up the vector
    // cache; the re-read last span of the prefetches beyond the loop came from HBM a second time).
    const int load_row = lane / 8, piece = lane % 8;
    unsigned w_source[NT][2];
    const unsigned char *ws_source[NT];
    const __amdgpu_buffer_rsrc_t weight_resource = make_resource(
        weight + size_t(n0) * weight_pitch, unsigned(p.outputs - n0 < NT * 16 ? p.outputs - n0 : NT * 16) * unsigned(weight_pitch));
    const __amdgpu_buffer_rsrc_t input_resource = make_resource(
        input + size_t(m0) * p.inner, unsigned(valid_rows - m0 < MT * 16 ? valid_rows - m0 : MT * 16) * unsigned(p.inner));
#pragma unroll
    for (int i = 0; i < NT; ++i) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int n = i * 16 + h * 8 + load_row;
            w_source[i][h] = n0 + n < p.outputs ? unsigned(n) * unsigned(weight_pitch) : 0x80000000u;
        }
        int n = n0 + i * 16 + row;
        n = n < p.outputs ? n : p.outputs - 1;
        // E4M3 weights: one scale per 32 x 32 block; E2M1 weights: one per row and 32 inputs
        ws_source[i] = weight_scale + size_t(PACKED ? n : n / 32) * blocks;
    }
    unsigned x_source[MT][2];
    const unsigned char *xs_source[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int m = j * 16 + h * 8 + load_row;
            x_source[j][h] = m0 + m < valid_rows ? unsigned(m) * unsigned(p.inner) : 0x80000000u;
        }
        int m = m0 + j * 16 + row;
        m = m < valid_rows ? m : valid_rows - 1;
        xs_source[j] = input_scale + size_t(m) * (blocks >> p.scale_shift);
    }
    // LDS patch of one tile, XOR-swizzled so that the line-shaped stores and the operand-shaped
    // loads are both conflict-free. An 8-bit operand of lane group c is pieces c and 4 + c of the
    // line (the instruction's layout); of a 4-bit line, piece c is the operand of the first group
    // and piece 4 + c that of the second: the same two reads serve both formats.
    auto slot = [](int r, int q) { return r * 8 + (q ^ ((r >> 1) & 7)); };
    const int store_slot[2] = {slot(load_row, piece), slot(load_row + 8, piece)};
    const int read_slot[2] = {slot(row, chunk), slot(row, chunk + 4)};

    // Workgroups start at different spans and wrap around (spreads the row-pitch-strided requests
    // over the HBM channels). Steps past the end re-read the last span with zeroed activations.
    const int start = int(blockIdx.x % unsigned(steps));
    auto span_of = [&](int step) {
        step = step < steps ? step : steps - 1;
        int rotated = step + start;
        rotated = rotated < steps ? rotated : rotated - steps;
        return rotated * WAVES + wave;
    };
    u32x4_t w_raw[DEPTH][NT][2], x_raw[DEPTH][MT][SUB][2];
    unsigned ws_raw[DEPTH][NT][SUB], xs_raw[DEPTH][MT][SUB], keep_raw[DEPTH][SUB][2];
    // Loads only: nothing here may use a loaded value, or the wait would cover the newest loads.
    auto fetch = [&](int step, u32x4_t(&w)[NT][2], u32x4_t(&x)[MT][SUB][2], unsigned(&ws)[NT][SUB],
                     unsigned(&xs)[MT][SUB], unsigned(&keep)[SUB][2]) {
        int g = span_of(step);
        const bool live = step < steps && g < spans;
        g = g < spans ? g : spans - 1;
        // bytes past the end of a row in a partial last span re-read the row's last 16 bytes
        const unsigned dead = live ? 0u : 0x80000000u;
        unsigned w_offset = unsigned(g) * 128u + unsigned(piece) * 16u;
        w_offset = w_offset < unsigned(weight_pitch) ? w_offset : unsigned(weight_pitch) - 16u;
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) // (read once: non-temporal, cache policy bit 1)
                w[i][h] = __builtin_amdgcn_raw_buffer_load_b128(weight_resource, int((w_source[i][h] + w_offset) | dead), 0, 2);
#pragma unroll
        for (int s = 0; s < SUB; ++s) {
            const int first = g * STEP_INPUTS + s * GROUP; // first input of the 128-input group
            int block = first / 32 + chunk; // the 32-input block whose scales this lane supplies
            block = block < blocks ? block : blocks - 1;
            // the operand's two 16-byte input pieces are positions 16c.. and 64+16c.. of the group
#pragma unroll
            for (int h = 0; h < 2; ++h)
                keep[s][h] = live && first + 64 * h + chunk * 16 < p.inner ? 0xffffffffu : 0u;
            int x_offset = first + piece * 16;
            x_offset = x_offset < p.inner ? x_offset : p.inner - 16;
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                if constexpr (STAGED)
                    ws[i][s] = unsigned(block); // read from LDS at multiply time
                else
                    ws[i][s] = ws_source[i][block];
            }
#pragma unroll
            for (int j = 0; j < MT; ++j) {
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    x[j][s][h] = __builtin_amdgcn_raw_buffer_load_b128(input_resource, int((x_source[j][h] + unsigned(x_offset)) | dead), 0, 0);
                if constexpr (STAGED)
                    xs[j][s] = unsigned(block >> p.scale_shift); // read from LDS at multiply time
                else
                    xs[j][s] = xs_source[j][block >> p.scale_shift];
            }
        }
    };

    // Staged scales: two byte ranges, each copied into LDS by direct-to-LDS loads of 1 KB (16 bytes
    // per lane) from the 4-byte aligned address at or below its start: the weight scales of rows
    // n0 .. n0 + 16*NT - 1 (E2M1: a scale row per weight row; E4M3: a scale row per 32 weight rows),
    // cut at the matrix end, and the scales of the workgroup's tokens. The loads go out before the
    // first weight loads and are complete with them; bytes past a range's end are never read.
    int staged_shift = 0, token_shift = 0;
    int w_base[NT], x_base[MT]; // byte offset of this lane's scale row inside the staged ranges
    if constexpr (STAGED) {
        const int first_row = PACKED ? n0 : n0 / 32;
        const int last = min(n0 + NT * 16, p.outputs) - 1;
        const int staged_rows = (PACKED ? last : last / 32) - first_row + 1;
        const unsigned char *first = weight_scale + size_t(first_row) * blocks;
        staged_shift = int(reinterpret_cast<uintptr_t>(first) & 3);
        const unsigned bytes = unsigned(staged_shift + staged_rows * blocks);
        const u32x4_t range = uniform_descriptor(first - staged_shift, (bytes + 3u) & ~3u);
        for (unsigned piece = __builtin_amdgcn_readfirstlane(wave); piece * 1024u < bytes; piece += WAVES)
            load_to_lds_untracked(range, unsigned(lane) * 16u, piece * 1024u, staged + piece * 1024u);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            int n = n0 + i * 16 + (PACKED ? row : 0);
            n = n < p.outputs ? n : p.outputs - 1;
            w_base[i] = staged_shift + ((PACKED ? n : n / 32) - first_row) * blocks;
        }
        const int x_pitch = blocks >> p.scale_shift;
        const int tokens = min(MT * 16, valid_rows - m0);
        const unsigned char *first_token = input_scale + size_t(m0) * x_pitch;
        token_shift = int(reinterpret_cast<uintptr_t>(first_token) & 3);
        const unsigned token_bytes = unsigned(token_shift + tokens * x_pitch);
        const u32x4_t token_range = uniform_descriptor(first_token - token_shift, (token_bytes + 3u) & ~3u);
        for (unsigned piece = __builtin_amdgcn_readfirstlane(wave); piece * 1024u < token_bytes; piece += WAVES)
            load_to_lds_untracked(token_range, unsigned(lane) * 16u, piece * 1024u, staged_tokens + piece * 1024u);
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            int m = m0 + j * 16 + row;
            m = m < valid_rows ? m : valid_rows - 1;
            x_base[j] = token_shift + (m - m0) * x_pitch;
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    f32x4_t acc[NT][MT];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
            acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const u32x4_t(&w)[NT][2], const u32x4_t(&x)[MT][SUB][2],
                        const unsigned(&ws)[NT][SUB], const unsigned(&xs)[MT][SUB],
                        const unsigned(&keep)[SUB][2]) {
        u32x4_t *mine = &tiles[wave][0][0];
        u32x4_t *mine_x = &tiles[wave][NT][0];
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                mine[i * 128 + store_slot[h]] = w[i][h];
        u32x4_t w_lo[NT], w_hi[NT];
#pragma unroll
        for (int s = 0; s < SUB; ++s) {
#pragma unroll
            for (int j = 0; j < MT; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    mine_x[j * 128 + store_slot[h]] = x[j][s][h];
            // other lanes' stores are read below: keep the compiler from moving the loads up
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (s == 0) {
#pragma unroll
                for (int i = 0; i < NT; ++i) {
                    w_lo[i] = mine[i * 128 + read_slot[0]];
                    w_hi[i] = mine[i * 128 + read_slot[1]];
                }
            }
            i32x8_t a[NT];
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                const u32x4_t lo = PACKED && s == 1 ? w_hi[i] : w_lo[i];
                const u32x4_t hi = PACKED ? u32x4_t{0u, 0u, 0u, 0u} : w_hi[i];
                a[i] = i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                               int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
            }
            unsigned w_scale[NT];
#pragma unroll
            for (int i = 0; i < NT; ++i)
                w_scale[i] = STAGED ? unsigned(staged[w_base[i] + int(ws[i][s])]) : ws[i][s];
            unsigned x_scale[MT];
#pragma unroll
            for (int j = 0; j < MT; ++j)
                x_scale[j] = STAGED ? unsigned(staged_tokens[x_base[j] + int(xs[j][s])]) : xs[j][s];
            // inputs past the end of K (and of dead steps) are zero
#pragma unroll
            for (int j = 0; j < MT; ++j) {
                const u32x4_t lo = mine_x[j * 128 + read_slot[0]] & keep[s][0],
                              hi = mine_x[j * 128 + read_slot[1]] & keep[s][1];
                const i32x8_t b = {int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]),
                                   int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
#pragma unroll
                for (int i = 0; i < NT; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        a[i], b, acc[i][j], PACKED ? 4 : 0, 0, 0, int(w_scale[i]), 0, int(x_scale[j]));
            }
            // the patches are overwritten next: order the reads above before those stores
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    };

#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        fetch(d, w_raw[d], x_raw[d], ws_raw[d], xs_raw[d], keep_raw[d]);
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (STAGED) {
        // the staged ranges' loads are older than the loads of the DEPTH fetches above (the compiler
        // does not count them, so the wait is explicit; not __syncthreads(): its fence would wait
        // for every weight load as well); the barrier shows every wavefront's pieces to the others
        constexpr int FETCH_LOADS = 2 * (NT + MT * SUB);
        static_assert(DEPTH * FETCH_LOADS < 64, "vmcnt holds 6 bits");
        pipeline_barrier<DEPTH * FETCH_LOADS>();
    }
    for (int step = 0; step < steps; step += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            __builtin_amdgcn_sched_barrier(0);
            multiply(w_raw[d], x_raw[d], ws_raw[d], xs_raw[d], keep_raw[d]);
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + d + DEPTH, w_raw[d], x_raw[d], ws_raw[d], xs_raw[d], keep_raw[d]);
        }
    }
    // ---- every wavefront parks its partial sums in its own tile memory (nobody else reads that),
    // one barrier, then tile t is summed in wavefront order 0, 1, 2, 3 by wavefront t % 4 and
    // written. Register r of lane l is feature 4*(l/16) + r and token l%16 of the tile.
    f32x4_t *parked = reinterpret_cast<f32x4_t *>(&tiles[wave][0][0]);
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
            parked[(i * MT + j) * 64 + lane] = acc[i][j];
    __syncthreads();
#pragma unroll
    for (int index = 0; index < NT * MT; ++index) {
        if (index % WAVES != wave)
            continue;
        const int i = index / MT, j = index % MT;
        const int m = m0 + j * 16 + row;
        const int n = n0 + i * 16 + chunk * 4;
        if (m >= p.rows || n >= p.outputs)
            continue;
        f32x4_t sum = reinterpret_cast<const f32x4_t *>(&tiles[0][0][0])[index * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            sum = sum + reinterpret_cast<const f32x4_t *>(&tiles[w][0][0])[index * 64 + lane];
        const bool zero = GROUPED && m >= valid_rows; // padding rows of a group
        // outputs is a multiple of eight, so the four features are all inside the matrix
        unsigned short bits[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            bits[e] = zero ? (unsigned short)0 : float_to_bf16_bits(sum[e]);
        unsigned short *target = out + size_t(m) * p.outputs + n;
        if (p.out_aligned) {
            *reinterpret_cast<u32x2_t *>(target) =
                u32x2_t{bits[0] | unsigned(bits[1]) << 16, bits[2] | unsigned(bits[3]) << 16};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                target[e] = bits[e];
        }
    }
}

template <bool PACKED, bool GROUPED, int NT, int MT>
hipError_t launch_one(hipStream_t stream, const MxParams &p, int groups)
{
    if constexpr (NT * MT > 16 || NT + MT * (PACKED ? 2 : 1) > 10) {
        return hipErrorInvalidValue;
    } else {
        // (a workgroup addresses its weight rows and its token rows with 31-bit byte offsets)
        if (size_t(NT > MT ? NT : MT) * 16 * size_t(p.inner) >= (size_t(1) << 31))
            return hipErrorInvalidValue;
        dim3 grid(unsigned((p.outputs + NT * 16 - 1) / (NT * 16)),
                  unsigned((p.rows + MT * 16 - 1) / (MT * 16)), unsigned(groups));
        const int blocks = p.inner / 32;
        const int weight_scale_bytes = (PACKED ? NT * 16 : NT / 2 + 2) * blocks + 3;
        const int token_scale_bytes = MT * 16 * (blocks >> p.scale_shift) + 3;
        if (weight_scale_bytes <= STAGED_SCALE_BYTES && token_scale_bytes <= STAGED_TOKEN_BYTES)
            mx_stream_kernel<PACKED, GROUPED, true, NT, MT><<<grid, WAVES * 64, 0, stream>>>(p);
        else
            mx_stream_kernel<PACKED, GROUPED, false, NT, MT><<<grid, WAVES * 64, 0, stream>>>(p);
        return launch_status();
    }
}

template <bool PACKED, bool GROUPED>
hipError_t launch_shape(hipStream_t stream, const MxParams &p, int groups, int forced_row_tiles)
{
    // token tiles by row count; weight-row tiles so that about one workgroup lands on each compute
    // unit, all groups counted (decode-sized calls: the kernel is bound by the weight stream, and a
    // workgroup of few rows spends most of its time in its fixed start and end)
    // (E2M1 steps hold twice the input tiles: four token tiles would not fit the register file)
    const int token_tiles = p.rows <= 16 ? 1 : p.rows <= 32 || PACKED ? 2 : 4;
    const int tiles = (p.outputs + 15) / 16;
    int row_tiles = 1;
    const int most = PACKED ? (token_tiles == 2 ? 6 : 8) : (token_tiles == 4 ? 4 : 8);
    for (int candidate = most; candidate > 1; --candidate)
        if (static_cast<long long>(tiles / candidate) * groups >= 224) {
            row_tiles = candidate;
            break;
        }
    if (forced_row_tiles >= 1 && forced_row_tiles <= most)
        row_tiles = forced_row_tiles;
#define CAMBLAS_MX(NT, MT) launch_one<PACKED, GROUPED, NT, MT>(stream, p, groups)
    switch (token_tiles * 10 + row_tiles) {
    case 11: return CAMBLAS_MX(1, 1);
    case 12: return CAMBLAS_MX(2, 1);
    case 13: return CAMBLAS_MX(3, 1);
    case 14: return CAMBLAS_MX(4, 1);
    case 15: return CAMBLAS_MX(5, 1);
    case 16: return CAMBLAS_MX(6, 1);
    case 17: return CAMBLAS_MX(7, 1);
    case 18: return CAMBLAS_MX(8, 1);
    case 21: return CAMBLAS_MX(1, 2);
    case 22: return CAMBLAS_MX(2, 2);
    case 23: return CAMBLAS_MX(3, 2);
    case 24: return CAMBLAS_MX(4, 2);
    case 25: return CAMBLAS_MX(5, 2);
    case 26: return CAMBLAS_MX(6, 2);
    case 27: return CAMBLAS_MX(7, 2);
    case 28: return CAMBLAS_MX(8, 2);
    case 41: return CAMBLAS_MX(1, 4);
    case 42: return CAMBLAS_MX(2, 4);
    case 43: return CAMBLAS_MX(3, 4);
    default: return CAMBLAS_MX(4, 4);
    }
#undef CAMBLAS_MX
}
} // namespace

namespace
{
// How a product of more than 32 rows runs on the tiled kernel: the tile, the workgroups K is divided
// over, and for a product that would end in a partly filled round the tile of a second launch over
// the last outputs.
struct MxTilePlan {
    int variant = 0, shares = 1, tail_variant = 0, tail_outputs = 0;
};

// {microseconds per 128-input step of one tile, kilobytes a workgroup keeps in flight} per variant
struct MxTilePrice {
    double step_us, kilobytes_in_flight;
    int outputs, rows;
};
// (variant 4: the four-wavefront 192 x 256 tile of mx_wave4.hip, undivided K only; [18432, 7168] at 4096 rows
// 403 us against 450 for the best plan of the other tiles (E2M1 weights: 379 against 435), at 2048 rows 213
// against 237 (189 against 225), at 512 rows even (61 against 79))
const MxTilePrice mx_prices[2][5] = {
    {{1.60, 64, 256, 256}, {1.00, 96, 256, 128}, {1.35, 56, 192, 256}, {0.58, 64, 128, 128}, {1.20, 112, 192, 256}},
    {{1.60, 96, 256, 256}, {1.00, 64, 256, 128}, {1e30, 1, 192, 256}, {0.58, 48, 128, 128}, {1.13, 88, 192, 256}},
};

// Estimated microseconds of one launch (as for the BF16 tiles: rounds of workgroups times steps
// times the tile's time per step, or the weights streamed at what the workgroups in flight can
// draw if that is longer; a divided K adds the second kernel and the traffic of the FP32 planes).
// Prices from a sweep of every tile with 1..8 shares over seven projection shapes at 48..1536 rows,
// both weight formats: the choice by this estimate is within 1 % of the best measured candidate in
// the geometric mean.
double mx_launch_us(const MxTilePrice &price, bool packed, long long batches, int rows, int outputs, int inner,
                    int shares, int compute_units)
{
    const double workgroups =
        double((outputs + price.outputs - 1) / price.outputs) * ((rows + price.rows - 1) / price.rows) * batches * shares;
    const double rounds = std::ceil(workgroups / compute_units);
    const double steps = (inner / 128 + shares - 1) / shares;
    const double bytes_per_us =
        std::min(5.2e6, std::min(workgroups, double(compute_units)) * price.kilobytes_in_flight * 1024 / 2.6);
    double stream_us = double(batches) * outputs * inner / (packed ? 2 : 1) / bytes_per_us;
    if (workgroups > compute_units)
        stream_us *= rounds * compute_units / workgroups;
    double us = 0.8 + std::max(rounds * steps * price.step_us, stream_us);
    if (shares > 1)
        us += 5.0 + 2.0 * shares * double(rows) * outputs * 4 / 4.5e6;
    return us;
}

// four_wavefronts: the call meets what the four-wavefront tile needs beyond the other tiles (see
// mx_four_wavefront_tile_applies)
MxTilePlan mx_tile_plan(int compute_units, bool packed, int groups, int rows, int outputs, int inner,
                        bool four_wavefronts = false)
{
    MxTilePlan plan;
    const long long batches = groups > 0 ? groups : 1;
    const MxTilePrice(&prices)[5] = mx_prices[packed ? 1 : 0];
    double best = 1e300;
    const int counts[] = {1, 2, 3, 4, 6, 8};
    for (int variant = 0; variant < 5; ++variant) {
        if (prices[variant].step_us > 1e29 || (prices[variant].rows > 128 && rows <= 128) ||
            (variant == 4 && !four_wavefronts))
            continue;
        for (const int shares : counts) {
            if (variant == 4 && shares > 1)
                continue;
            // a share has at least eight steps, the planes at most 256 MB; grouped products are not divided
            if (shares > 1 && (groups > 0 || inner / 128 / shares < 8 ||
                               double(shares) * rows * outputs * 4 > double(1 << 28)))
                continue;
            const double us = mx_launch_us(prices[variant], packed, batches, rows, outputs, inner, shares, compute_units);
            if (us < best) {
                best = us;
                plan.variant = variant;
                plan.shares = shares;
            }
        }
    }
    // A plain product whose 256 x 256 tiles end in a partly filled round: whole rounds over the
    // first outputs, and the rest on the tile that covers them soonest
    // (18432 outputs by 4096 tokens: four rounds, then 2048 outputs as one round of 256 x 128).
    if (groups == 0 && rows > 128) {
        const long long token_tiles = (rows + 255) / 256;
        const long long whole = static_cast<long long>((outputs + 255) / 256) * token_tiles / compute_units;
        const long long main_outputs = whole * compute_units / token_tiles * 256;
        if (whole >= 1 && main_outputs > 0 && main_outputs < outputs) {
            const double main_us = mx_launch_us(prices[0], packed, 1, rows, int(main_outputs), inner, 1, compute_units);
            for (int variant = 0; variant < 4; ++variant) {
                if (prices[variant].step_us > 1e29)
                    continue;
                const double us = main_us + 3.0 + mx_launch_us(prices[variant], packed, 1, rows, outputs - int(main_outputs),
                                                               inner, 1, compute_units);
                if (us < 0.97 * best) {
                    best = us / 0.97;
                    plan.variant = 0;
                    plan.shares = 1;
                    plan.tail_variant = variant;
                    plan.tail_outputs = outputs - int(main_outputs);
                }
            }
        }
    }
    return plan;
}
} // namespace

// Rows from which the tiled kernel takes over: above 32 (the measured crossover), and from 17 on
// when the streaming kernel could not hold the scale bytes of 32 tokens in its LDS table and would
// gather them a byte per lane and step ([7168, 18432] x 32 rows: 34 us against 24 at 16 rows and 26 on
// the tiles).
// What the four-wavefront tile needs beyond mx_dma_supported: a scale per 32 inputs, whole slabs of eight
// 128-input groups (at least two), input scale rows it can copy 16 bytes at a time, and the same of the
// per-row scales of packed weights, whose address the host has to know: no grouped product of packed weights.
static bool mx_four_wavefront_tile_applies(bool packed, int groups, int inner, int activation_block,
                                           const void *input_scale, const void *weight_scale)
{
    return activation_block == 32 && inner % 1024 == 0 && inner >= 2048 &&
           reinterpret_cast<uintptr_t>(input_scale) % 16 == 0 &&
           (packed ? groups == 0 && reinterpret_cast<uintptr_t>(weight_scale) % 16 == 0 : true);
}

static bool mx_rows_take_tiles(int rows, int inner, int activation_block)
{
    return rows > 32 || (rows > 16 && 32 * (inner / activation_block) + 3 > STAGED_TOKEN_BYTES);
}

int mx_matmul_shares(int kernel, int forced_shares, int compute_units, bool packed, int rows, int outputs,
                     int inner, int activation_block, const void *input, const void *weight, const void *out)
{
    if (kernel >= 20)
        return forced_shares > 1 ? forced_shares : 1;
    if (kernel >= 0 || !mx_rows_take_tiles(rows, inner, activation_block) ||
        !mx_dma_supported(outputs, inner, input, weight, out))
        return 1;
    return mx_tile_plan(compute_units, packed, 0, rows, outputs, inner).shares;
}

// groups == 0: plain product (weight, weight_scale given); groups >= 1: grouped product (metadata,
// active, counts given). activation_block 32 or 128. Weights 16-byte aligned. forced_shares: with a
// forced tile variant (kernel >= 20), the workgroups K is divided over; planes: room for a divided K
// (see mx_matmul_shares), without which K is not divided.
hipError_t launch_mx_matmul(hipStream_t stream, int kernel, int compute_units, bool packed, int groups,
                            int weight_groups, int rows, int outputs, int inner,
                            int activation_block, const void *input,
                            const void *input_scale, const void *weight, const void *weight_scale,
                            const void *metadata, const void *active, const void *counts, void *out,
                            int forced_shares, float *planes)
{
    // Above 32 rows the streaming kernel reads the weights once per 32-token slab; the tiled kernel
    // reads them once per 128 or 256 tokens (grouped weights come from the device table and are
    // 16-byte aligned by contract, so only the host-visible pointers are checked here).
    const void *checked_weight = groups == 0 ? weight : nullptr;
    if (kernel >= 20)
        return launch_mx_dma(stream, kernel - 20, packed, groups, weight_groups, rows, outputs, inner,
                             activation_block, input, input_scale, weight, weight_scale, metadata,
                             active, counts, out, 0, 0, planes && groups == 0 && forced_shares > 1 ? forced_shares : 1,
                             planes);
    if (kernel < 0 && mx_rows_take_tiles(rows, inner, activation_block) &&
        mx_dma_supported(outputs, inner, input, checked_weight, out)) {
        MxTilePlan plan = mx_tile_plan(compute_units, packed, groups, rows, outputs, inner,
                                       mx_four_wavefront_tile_applies(packed, groups, inner, activation_block, input_scale,
                                                                      weight_scale));
        if (plan.shares > 1 && !planes) // no room for the planes: the same tile with K undivided
            plan.shares = 1;
        return launch_mx_dma(stream, plan.variant, packed, groups, weight_groups, rows, outputs, inner,
                             activation_block, input, input_scale, weight, weight_scale, metadata,
                             active, counts, out, plan.tail_variant, plan.tail_outputs, plan.shares, planes);
    }
    MxParams p;
    p.input = static_cast<const unsigned char *>(input);
    p.input_scale = static_cast<const unsigned char *>(input_scale);
    p.weight = static_cast<const unsigned char *>(weight);
    p.weight_scale = static_cast<const unsigned char *>(weight_scale);
    p.out = static_cast<unsigned short *>(out);
    p.rows = rows;
    p.outputs = outputs;
    p.inner = inner;
    p.scale_shift = activation_block == 128 ? 2 : 0;
    p.out_aligned = reinterpret_cast<uintptr_t>(out) % 8 == 0;
    p.metadata = static_cast<const unsigned long long *>(metadata);
    p.active = static_cast<const int32_t *>(active);
    p.counts = static_cast<const int32_t *>(counts);
    p.weight_groups = weight_groups;
    if ((rows + 15) / 16 > 65535 || groups > 65535)
        return hipErrorInvalidValue;
    if (groups == 0)
        return packed ? launch_shape<true, false>(stream, p, 1, kernel) : launch_shape<false, false>(stream, p, 1, kernel);
    return packed ? launch_shape<true, true>(stream, p, groups, kernel)
                  : launch_shape<false, true>(stream, p, groups, kernel);
}
} // namespace camblas_hip
