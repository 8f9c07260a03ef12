// E8M0 block-scaled prefill product (E4M3 inputs with one scale byte per 32 inputs; E4M3 weights with
// one scale byte per 32 x 32 block, or packed E2M1 weights with one scale byte per row and 32 inputs;
// BF16 out; contract: ref include/camblas_cuda.h:110-123,
// src/cuda/backend.cu:1165-1191, value semantics tests/test_quantized.py:12-50 of the reference) on four
// wavefronts per workgroup, one per SIMD: a workgroup owns 192 weight rows x 256 tokens, a wavefront
// 96 x 128 = 6 x 8 tiles of v_mfma_scale_f32_16x16x128_f8f6f4 with the hardware applying both scales.
// Against the eight-wavefront tiles of mx_dma.hip a wavefront reads each weight fragment from LDS once
// per eight and each token fragment once per six matrix instructions, holds the fragments of two whole
// K groups in the accumulation registers, and shares its SIMD's issue with nobody.
//
// The K loop is one inline-assembly statement with every register named, written by
// gen_mx_wave4_loop.py into mx_wave4_loop_192x256*.inc at build time (its header describes the
// registers and the scale handling; the tile, fills and slabs are those of fp8_wave4.hip). Around it
// this file is ordinary HIP.
// Shape requirements: one input scale per 32 inputs, K a multiple of 1024 and at least 2048, scale rows
// the slab loads can copy (input scales 16-byte aligned; E2M1 weights' scales 16-byte aligned; the block
// scales of E4M3 weights may lie at any address), outputs % 4 == 0. The grouped product (weights from a
// device table, ref include/camblas_cuda.h:156-167) takes E4M3 weights only: the alignment of a table
// entry's scales is not known on the host.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"
#include "mx_grouped.hpp"

namespace camblas_hip
{
namespace
{
struct MxWave4Params {
    const unsigned char *w, *a, *w_scale, *a_scale;
    unsigned short *out;
    int n, k, k_groups, block_rows, out_pitch, tiles_n, tiles_m;
    int rows; // tokens (grouped: the capacity of a group)
    // grouped form
    const unsigned long long *metadata;
    const int32_t *active, *counts;
    int weight_groups, groups;
};

constexpr int NA = 6, NB = 8, BN = 32 * NA, BM = 256, CH = 8;

template <bool PACKED, bool GROUPED> __global__ __launch_bounds__(256) void mx_wave4_kernel(MxWave4Params p)
{
    // Two stages of operands (weight rows of 128 bytes, or 64 when packed, then token rows); two 8 KB
    // buffers of token scale words [256 tokens][8 groups] 8 KB apart; the weights' scale words likewise
    // (E2M1: a word per row) or as two 256-byte buffers [8 block rows][8 groups] (E4M3). The loop switches
    // between the two buffers of a slab by flipping one address bit, so the slabs start where that bit is
    // clear, and the array lies at LDS address 0 (it is the only LDS object of the kernel).
    constexpr int A_ROW = PACKED ? 64 : 128, A_BYTES = BN * A_ROW, STAGE_BYTES = A_BYTES + BM * 128;
    constexpr int A_SLAB = PACKED ? 0x18000 : 2 * STAGE_BYTES, W_SLAB = A_SLAB + 0x4000;
    constexpr int LDS_BYTES = W_SLAB + (PACKED ? 0x4000 : 512);
    static_assert(2 * STAGE_BYTES <= A_SLAB && A_SLAB % 0x4000 == 0 && W_SLAB % 0x4000 == 0, "slab addresses");
    __shared__ u32x4_t lds[LDS_BYTES / 16];

    const int thread = threadIdx.x, lane = thread % 64;
    int tile_n, tile_m, group = 0;
    if constexpr (GROUPED)
        grouped_tile<BM>(p, lane, blockIdx.x, group, tile_n, tile_m);
    else
        xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const int wn = wave % 2, wm = wave / 2;
    const unsigned pitch = PACKED ? unsigned(p.k) / 2u : unsigned(p.k); // bytes of a weight row

    const unsigned char *input = p.a, *input_scale = p.a_scale, *weight = p.w, *weight_scale = p.w_scale;
    unsigned short *out = p.out;
    int valid_rows = p.rows;
    if constexpr (GROUPED) {
        // weights come from a device table indexed by active[group]; invalid indices and rows at or beyond
        // counts[group] produce zeros
        const int index = __builtin_amdgcn_readfirstlane(p.active[group]);
        const int count = __builtin_amdgcn_readfirstlane(p.counts[group]);
        valid_rows = index >= 0 && index < p.weight_groups ? min(max(count, 0), p.rows) : 0;
        input += size_t(group) * p.rows * p.k;
        input_scale += size_t(group) * p.rows * p.k_groups * 4;
        out += size_t(group) * p.rows * p.out_pitch;
        if (m0 >= valid_rows) { // nothing to multiply: this tile of the output is zero
            for (int item = thread; item < BM * (BN / 4); item += 256) {
                const int m = m0 + item / (BN / 4), n = n0 + (item % (BN / 4)) * 4;
                if (m < p.rows && n < p.n)
                    *reinterpret_cast<u32x2_t *>(out + size_t(m) * p.out_pitch + n) = u32x2_t{0u, 0u};
            }
            return;
        }
        weight = reinterpret_cast<const unsigned char *>(uniform(p.metadata[2 * size_t(index)]));
        weight_scale = reinterpret_cast<const unsigned char *>(uniform(p.metadata[2 * size_t(index) + 1]));
    }

    // ---- fills: wave instruction (it, wave) fills LDS slots [(it*4 + wave)*64, +64) of a stage; rows of
    // 128 bytes: rows (it*4 + wave)*8 + lane/8, chunk lane%8; rows of 64 bytes: rows (it*4 + wave)*16 +
    // lane/4, chunk lane%4; the slot holds logical chunk (chunk ^ swizzle(row)). Weight rows first, token
    // rows behind them. Rows past the end of a matrix are outside the descriptor and read as zero.
    const int load_row = wave * 8 + lane / CH;
    unsigned b_offset = unsigned(load_row) * unsigned(p.k) + unsigned(((lane % CH) ^ lds_swizzle<CH>(load_row)) * 16);
    unsigned a_offset = b_offset;
    const unsigned row_step = __builtin_amdgcn_readfirstlane(32u * unsigned(p.k));
    unsigned row_step_a = row_step;
    if constexpr (PACKED) {
        const int packed_row = wave * 16 + lane / 4;
        a_offset = unsigned(packed_row) * pitch + unsigned(((lane % 4) ^ lds_swizzle<4>(packed_row)) * 16);
        row_step_a = __builtin_amdgcn_readfirstlane(64u * pitch);
    }
    const int a_rows = p.n - n0 < BN ? p.n - n0 : BN, b_rows = valid_rows - m0 < BM ? valid_rows - m0 : BM;
    const u32x4_t a_resource = uniform_descriptor(weight + size_t(n0) * pitch, unsigned(a_rows) * pitch);
    const u32x4_t b_resource = uniform_descriptor(input + size_t(m0) * p.k, unsigned(b_rows) * unsigned(p.k));
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));
    const unsigned fill_base = __builtin_amdgcn_readfirstlane(lds_base + unsigned(wave) * 1024u);

    // ---- scale slabs: the four scale bytes of a row and K group are one word. Wavefront w copies pieces
    // 2w and 2w + 1 of the token slab (32 tokens each): lane l brings groups 4 (l / 32) .. + 3 of token
    // l % 32 of the piece, 16 bytes, so that a piece lands as two halves of [token][4 groups] and sixteen
    // tokens in a row lie in sixteen different banks. Rows that do not exist read as zero. Weight words, E2M1 (a word per row): pieces w and w + 4 of eight in the same way, of
    // which six hold the tile's rows; E4M3: lane l < 63 of one 4-byte load brings word l % 9 of block row
    // l / 9 from the tile's first 32-row block row (the tile's 192 rows are six of them), counted from the
    // aligned address at or below the block row's scales: with the ninth word the slab holds all of its
    // 32 bytes wherever they lie, and a lane reads its byte `skew` bytes further on.
    const u32x4_t a_scale_resource =
        uniform_descriptor(input_scale + size_t(m0) * p.k_groups * 4, unsigned(b_rows) * unsigned(p.k_groups) * 4u);
    const unsigned slab_offset = (unsigned(wave * 64 + lane % 32) * unsigned(p.k_groups) + unsigned(lane / 32) * 4u) * 4u;
    const unsigned slab_rows = __builtin_amdgcn_readfirstlane(32u * unsigned(p.k_groups) * 4u);
    const unsigned slab_fill = __builtin_amdgcn_readfirstlane(lds_base + unsigned(A_SLAB) + unsigned(wave) * 2048u);
    const int first_block = n0 / 32;
    const int blocks = p.block_rows - first_block < 8 ? p.block_rows - first_block : 8;
    const unsigned skew = PACKED ? 0u : unsigned(__builtin_amdgcn_readfirstlane(unsigned(reinterpret_cast<uintptr_t>(weight_scale)) % 4u));
    const u32x4_t w_scale_resource =
        PACKED ? uniform_descriptor(weight_scale + size_t(n0) * p.k_groups * 4, unsigned(a_rows) * unsigned(p.k_groups) * 4u)
               : uniform_descriptor(weight_scale - skew + size_t(first_block) * p.k_groups * 4,
                                    unsigned(blocks) * unsigned(p.k_groups) * 4u + (skew ? 4u : 0u));
    const unsigned weight_slab_offset =
        PACKED ? (unsigned(wave * 32 + lane % 32) * unsigned(p.k_groups) + unsigned(lane / 32) * 4u) * 4u
               : (lane < 63 ? (unsigned(lane / 9) * unsigned(p.k_groups) + unsigned(lane % 9)) * 4u : 0x80000000u);
    const unsigned weight_slab_rows = __builtin_amdgcn_readfirstlane(128u * unsigned(p.k_groups) * 4u);
    const unsigned weight_slab_fill =
        __builtin_amdgcn_readfirstlane(lds_base + unsigned(W_SLAB) + (PACKED ? unsigned(wave) * 1024u : 0u));
    unsigned slab_k = 0; // byte offset of the next slab along a row of scale words
    unsigned middle_slabs = __builtin_amdgcn_readfirstlane(unsigned(p.k_groups / 8 - 2));

    // ---- reads. Lane l holds row l % 16 of a 16-row tile. Of the 128 K positions of a group an 8-bit
    // operand holds 16 c .. + 15 and 64 + 16 c .. + 15 with c = l / 16 (chunks c and 4 + c of its 128-byte
    // row), a 4-bit operand 32 c .. + 31 (chunk c of its 64-byte row); either way the lane supplies the scale
    // byte of inputs 32 c .. 32 c + 31: byte c of the row's word.
    const int frag_row = lane % 16, quarter = lane / 16;
    const int frag_swizzle = lds_swizzle<CH>(frag_row);
    const int wave_row = n0 + wn * NA * 16; // first weight row of the wavefront
    const unsigned a_row_bytes = unsigned(wn * NA * 16 + frag_row) * unsigned(A_ROW);
    const unsigned b_row_bytes = unsigned(A_BYTES) + unsigned(wm * NB * 16 + frag_row) * 128u;
    const unsigned read_a_lo =
        lds_base + a_row_bytes + unsigned(PACKED ? quarter ^ lds_swizzle<4>(frag_row) : quarter ^ frag_swizzle) * 16u;
    const unsigned read_a_hi = lds_base + a_row_bytes + unsigned((4 + quarter) ^ frag_swizzle) * 16u; // (E4M3 weights only)
    const unsigned read_b_lo = lds_base + b_row_bytes + unsigned(quarter ^ frag_swizzle) * 16u;
    const unsigned read_b_hi = lds_base + b_row_bytes + unsigned((4 + quarter) ^ frag_swizzle) * 16u;
    // (a wavefront's 128 tokens are four pieces of a slab, its 96 weight rows three)
    unsigned scale_address = lds_base + unsigned(A_SLAB) + unsigned(wm * 4) * 1024u + unsigned(frag_row) * 16u + unsigned(quarter);
    unsigned weight_scale_address =
        lds_base + unsigned(W_SLAB) + unsigned(quarter) +
        (PACKED ? unsigned(wn * 3) * 1024u + unsigned(frag_row) * 16u : unsigned(wave_row / 32 - first_block) * 36u + skew);

    // accumulator tile (i, j) (weight rows 16 i .., tokens 16 j ..) comes back as accs[8 i + j]
    f32x4_t accs[NA * NB];
    if constexpr (PACKED) {
#include "mx_wave4_loop_192x256_e2m1.inc"
    } else {
#include "mx_wave4_loop_192x256.inc"
    }

    // ---- epilogue. Register e of lane l in tile (i, j) is feature 16 i + 4 (l / 16) + e, token 16 j + l % 16.
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int m = m0 + wm * NB * 16 + j * 16 + frag_row;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const int n = wave_row + i * 16 + quarter * 4;
            const f32x4_t v = accs[NB * i + j];
            if (m < p.rows && n < p.n) // (tokens at or beyond a group's count multiplied zeros)
                *reinterpret_cast<u32x2_t *>(out + size_t(m) * p.out_pitch + n) =
                    u32x2_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
    }
}
} // namespace

// `outputs` weight rows from `weight` on (scale rows from weight_scale on), written at `out` with `out_pitch`
// elements between tokens. packed: E2M1 weights, two to a byte, a scale byte per row and 32 inputs.
// Grouped (metadata != nullptr, E4M3 weights only): `groups` groups of `rows` token rows each in input,
// input_scale and out (out_pitch = outputs); weights and their scales from table entry active[group].
hipError_t launch_mx_wave4(hipStream_t stream, bool packed, int rows, int outputs, int inner, const void *input,
                           const void *input_scale, const void *weight, const void *weight_scale, void *out, int out_pitch,
                           int groups, int weight_groups, const void *metadata, const void *active, const void *counts)
{
    const auto misaligned = [](const void *pointer, uintptr_t to) { return reinterpret_cast<uintptr_t>(pointer) % to != 0; };
    const bool grouped = metadata != nullptr;
    if (rows < 1 || outputs < 1 || outputs % 4 || out_pitch % 4 || inner % 1024 || inner < 2048 || misaligned(out, 8) ||
        misaligned(input, 16) || misaligned(input_scale, 16))
        return hipErrorInvalidValue;
    if (grouped ? packed || groups < 1 || weight_groups < 1 || !active || !counts || out_pitch != outputs
                : misaligned(weight, 16) || (packed && misaligned(weight_scale, 16)))
        return hipErrorInvalidValue;
    if (size_t(256) * size_t(inner) >= (size_t(1) << 32))
        return hipErrorInvalidValue;
    MxWave4Params p;
    p.w = static_cast<const unsigned char *>(weight);
    p.a = static_cast<const unsigned char *>(input);
    p.w_scale = static_cast<const unsigned char *>(weight_scale);
    p.a_scale = static_cast<const unsigned char *>(input_scale);
    p.out = static_cast<unsigned short *>(out);
    p.n = outputs;
    p.rows = rows;
    p.k = inner;
    p.k_groups = inner / 128;
    p.block_rows = (outputs + 31) / 32;
    p.out_pitch = out_pitch;
    p.tiles_n = (outputs + BN - 1) / BN;
    p.tiles_m = (rows + BM - 1) / BM;
    p.metadata = static_cast<const unsigned long long *>(metadata);
    p.active = static_cast<const int32_t *>(active);
    p.counts = static_cast<const int32_t *>(counts);
    p.weight_groups = weight_groups;
    p.groups = grouped ? groups : 1;
    const size_t grid = size_t(p.tiles_n) * size_t(p.tiles_m) * size_t(p.groups);
    if (grid > 0x7fffffffu)
        return hipErrorInvalidValue;
    if (grouped)
        mx_wave4_kernel<false, true><<<unsigned(grid), 256, 0, stream>>>(p);
    else if (packed)
        mx_wave4_kernel<true, false><<<unsigned(grid), 256, 0, stream>>>(p);
    else
        mx_wave4_kernel<false, false><<<unsigned(grid), 256, 0, stream>>>(p);
    return launch_status();
}
} // namespace camblas_hip
