// BF16 prefill linear y[M,N] = alpha * x[M,K] * W[N,K]^T + beta * y on four wavefronts per workgroup,
// one per SIMD: a (32*NA) x 256 x 64 tile (NA = 8: 256 weight rows, NA = 10: 320) in which every
// wavefront owns a (16*NA) x 128 block, i.e. NA x 8 tiles of v_mfma_f32_16x16x32_bf16 with 4*NA*8
// FP32 accumulators per lane. With the whole register file of its SIMD a wavefront reads each
// weight fragment once per eight and each token fragment once per NA matrix instructions (the
// eight-wavefront tiles of bgemm_dma.hip: once per four and per five), and nothing in the loop
// depends on how the hardware arbitrates between wavefronts of one SIMD.
//
// Such a kernel is not expressible in HIP source with this compiler (the allocator spreads the
// accumulators over both halves of the register file and spills), so the K loop is one
// inline-assembly statement with every register named, written by gen_wave4_loop.py into
// wave4_loop_*.inc; its header describes the schedule. Around it this file is ordinary HIP: tile
// numbering per XCD, the buffer descriptors and per-lane offsets of the direct-to-LDS fills, the
// XOR-swizzled LDS layout (both as in bgemm_dma.hip), and the epilogue.
// Shape requirements beyond launch_bgemm_dma's: K a multiple of 128 (an even number of steps per
// share of K).
// NN: the same product with the weights stored the other way round, W[K, N] with the outputs
// contiguous (x @ W with a row-major W; 'N','N' in the column-major terms of camblas_cuda_bgemm). The
// weight tile of a K step is copied into LDS as it lies (64 rows of 256 outputs, 1 KB pieces holding
// rows k and k + 4, pieces 1056 bytes apart) and a lane gathers the eight K values of its output with
// two transposing LDS reads (ds_read_b64_tr_b16; the generator's Layout describes the lane pattern),
// so no transposed copy of W is made first. 256 x 256 tile only; lda % 8 == 0.
// Contract: ref src/cuda/bfloat16.cuh:11-57 ('T','N' and 'N','N' calls of src/cuda/torch_bindings.cpp:155-199).
#include "bgemm_dma.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
template <int NA, bool NN>
__global__ __launch_bounds__(256) void bgemm_wave4_kernel(DmaParams p)
{
    constexpr int NB = 8, BN = 32 * NA, BM = 256, BK = 64, CH = 8, WAVES = 4, ROWS_PER_LOAD = 8;
    constexpr int NN_PIECE = 1056; // bytes from one 1 KB piece of an as-it-lies weight tile to the next
    static_assert(!NN || NA == 8, "a K row of 256 outputs is half a 1 KB load");
    constexpr int A_BYTES = NN ? (BK / 2) * NN_PIECE : BN * 128;
    constexpr int STAGE_SLOTS = (A_BYTES + BM * 128) / 16;
    __shared__ u32x4_t stages[2 * STAGE_SLOTS];

    int tile_n, tile_m;
    xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int first_step = int(blockIdx.y) * p.share_steps;
    const int k_tiles = p.k / BK - first_step < p.share_steps ? p.k / BK - first_step : p.share_steps;

    const int thread = threadIdx.x, lane = thread % 64;
    const int wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const int wn = wave % 2, wm = wave / 2;

    // ---- fills: wave instruction (it, wave) fills LDS slots [(it*4 + wave)*64, +64) of a stage with
    // rows (it*4 + wave)*8 + lane/8, 16-byte chunk lane%8 holding logical chunk (lane%8) ^ swizzle(row);
    // weight rows first, token rows behind them, so a wavefront's successive loads are 4 KB apart.
    const int load_row = wave * ROWS_PER_LOAD + lane / CH;
    const unsigned load_chunk = unsigned(((lane % CH) ^ lds_swizzle<CH>(load_row)) * 8);
    unsigned a_offset = (unsigned(load_row) * unsigned(p.lda) + load_chunk) * 2u + unsigned(first_step) * BK * 2;
    unsigned b_offset = (unsigned(load_row) * unsigned(p.ldb) + load_chunk) * 2u + unsigned(first_step) * BK * 2;
    unsigned a_row_step = __builtin_amdgcn_readfirstlane(unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.lda) * 2u);
    const unsigned b_row_step = __builtin_amdgcn_readfirstlane(unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.ldb) * 2u);
    // one descriptor per operand, covering exactly the rows of this tile that exist (the rest reads zero)
    const int a_rows = p.n - n0 < BN ? p.n - n0 : BN, b_rows = p.m - m0 < BM ? p.m - m0 : BM;
    u32x4_t a_resource =
        uniform_descriptor(p.w + size_t(n0) * p.lda, (unsigned(a_rows - 1) * unsigned(p.lda) + unsigned(p.k)) * 2u);
    const u32x4_t b_resource =
        uniform_descriptor(p.x + size_t(m0) * p.ldb, (unsigned(b_rows - 1) * unsigned(p.ldb) + unsigned(p.k)) * 2u);
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(stages));
    unsigned fill_base = __builtin_amdgcn_readfirstlane(lds_base + unsigned(wave) * 1024u);
    [[maybe_unused]] unsigned fill_base_b = 0, a_k_step = 0;
    if constexpr (NN) {
        // weights as they lie: load `it` of wavefront w is piece 4 it + w, rows 8 it + w (lanes 0..31) and
        // + 4 (lanes 32..63) of the K step, 16 bytes per lane along the outputs. Rows past K and bytes
        // past the end of the last row are outside the descriptor and read as zero; outputs past N
        // inside a row are whatever lies there and only reach accumulators that are never stored.
        a_offset = (unsigned(wave + 4 * (lane / 32) + first_step * BK) * unsigned(p.lda) + unsigned(lane % 32) * 8u) * 2u;
        a_row_step = __builtin_amdgcn_readfirstlane(8u * unsigned(p.lda) * 2u);
        a_k_step = __builtin_amdgcn_readfirstlane(unsigned(BK) * unsigned(p.lda) * 2u);
        a_resource = uniform_descriptor(p.w + n0, (unsigned(p.k - 1) * unsigned(p.lda) + unsigned(p.n - n0)) * 2u);
        fill_base = __builtin_amdgcn_readfirstlane(lds_base + unsigned(wave) * unsigned(NN_PIECE));
        fill_base_b = __builtin_amdgcn_readfirstlane(lds_base + unsigned(A_BYTES) + unsigned(wave) * 1024u);
    }

    // ---- fragment reads: lane l reads the 16 bytes of row l%16, K values 8*(l/16) .. +7 of a
    // 32-deep sub-step; sub-step 1 lies four chunks on, which the swizzle turns into bit 2 of the chunk
    const int frag_row = lane % 16, group = lane / 16;
    const int frag_swizzle = lds_swizzle<CH>(frag_row);
    const unsigned a_row_bytes = unsigned(wn * NA * 16 + frag_row) * 128u;
    const unsigned b_row_bytes = unsigned(A_BYTES) + unsigned(wm * NB * 16 + frag_row) * 128u;
    unsigned read_a0 = lds_base + a_row_bytes + unsigned(group ^ frag_swizzle) * 16u;
    const unsigned read_a1 = lds_base + a_row_bytes + unsigned((4 + group) ^ frag_swizzle) * 16u;
    const unsigned read_b0 = lds_base + b_row_bytes + unsigned(group ^ frag_swizzle) * 16u;
    const unsigned read_b1 = lds_base + b_row_bytes + unsigned((4 + group) ^ frag_swizzle) * 16u;
    if constexpr (NN) // lane s of a group of sixteen: row s / 4 of the group's four-row block, outputs 4 (s % 4) .. + 3
        read_a0 = lds_base + unsigned(4 * group + frag_row / 4) * unsigned(NN_PIECE) + unsigned(wn * 256 + (frag_row % 4) * 8);
    unsigned step_pairs = __builtin_amdgcn_readfirstlane(unsigned(k_tiles - 2) / 2u);

    // accumulator tile (i, j) (weight rows 16 i .., tokens 16 j ..) comes back as accs[8 i + j]
    f32x4_t accs[NA * NB];
    auto sum = [&](int i, int j, int e) { return accs[NB * i + j][e]; };
    if constexpr (NN) {
#include "wave4_loop_256x256_nn.inc"
    } else if constexpr (NA == 8) {
#include "wave4_loop_256x256.inc"
    } else {
#include "wave4_loop_320x256.inc"
    }

    // ---- epilogue. Register e of lane l in tile (i, j) is feature 16 i + 4 (l / 16) + e, token 16 j + l % 16.
    const int first_feature = n0 + wn * NA * 16 + group * 4;
    const int first_token = m0 + wm * NB * 16 + frag_row;
    if (gridDim.y > 1) { // a share of K: the plain sums, for the ordered sum over the shares
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                const int m = first_token + j * 16, n = first_feature + i * 16;
                if (m < p.m && n < p.n)
                    *reinterpret_cast<f32x4_t *>(p.partials + (size_t(blockIdx.y) * p.m + m) * p.n + n) =
                        f32x4_t{sum(i, j, 0), sum(i, j, 1), sum(i, j, 2), sum(i, j, 3)};
            }
        return;
    }
    auto store_tile = [&](int i, int j, u32x2_t old, bool with_beta) {
        const int m = first_token + j * 16, n = first_feature + i * 16;
        if (m < p.m && n < p.n) {
            float v0 = p.alpha * sum(i, j, 0), v1 = p.alpha * sum(i, j, 1);
            float v2 = p.alpha * sum(i, j, 2), v3 = p.alpha * sum(i, j, 3);
            if (with_beta) {
                v0 = fmaf(p.beta, __uint_as_float(old[0] << 16), v0);
                v1 = fmaf(p.beta, __uint_as_float(old[0] & 0xffff0000u), v1);
                v2 = fmaf(p.beta, __uint_as_float(old[1] << 16), v2);
                v3 = fmaf(p.beta, __uint_as_float(old[1] & 0xffff0000u), v3);
            }
            *reinterpret_cast<u32x2_t *>(p.y + size_t(m) * p.ldc + n) = u32x2_t{pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
        }
    };
    if (p.beta == 0.f) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NA; ++i)
                store_tile(i, j, u32x2_t{0u, 0u}, false);
        return;
    }
    // beta term: the addends of the next four tiles are fetched while four tiles are scaled and stored
    // (unconditional loads: a position outside the matrix reads a valid element instead and is not used)
    constexpr int TILES = NA * NB, AHEAD = 4;
    u32x2_t old[2][AHEAD];
    auto fetch = [&](int first, u32x2_t (&into)[AHEAD]) {
#pragma unroll
        for (int t = 0; t < AHEAD; ++t) {
            const int tile = first + t < TILES ? first + t : TILES - 1;
            int m = first_token + (tile / NA) * 16;
            m = m < p.m ? m : p.m - 1;
            const int n = first_feature + (tile % NA) * 16;
            into[t] = *reinterpret_cast<const u32x2_t *>(p.z + size_t(m) * p.ldz + (n < p.n ? n : 0));
        }
    };
    static_assert(TILES % AHEAD == 0, "whole groups of tiles");
    fetch(0, old[0]);
#pragma unroll
    for (int first = 0; first < TILES; first += AHEAD) {
        __builtin_amdgcn_sched_barrier(0);
        if (first + AHEAD < TILES)
            fetch(first + AHEAD, old[(first / AHEAD + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < AHEAD; ++t)
            store_tile((first + t) % NA, (first + t) / NA, old[(first / AHEAD) & 1][t], true);
    }
}

template <int NA, bool NN = false> hipError_t launch(hipStream_t stream, DmaParams p, int shares)
{
    constexpr int BN = 32 * NA, BM = 256, BK = 64;
    const int steps = p.k / BK;
    if (p.k % BK || shares < 1 || steps % 2)
        return hipErrorInvalidValue;
    // (as-it-lies weights: 16-byte pieces of rows, and the whole matrix inside one 32-bit descriptor)
    if (NN && (p.lda % 8 || size_t(p.k) * size_t(p.lda) * 2 >= (size_t(1) << 32)))
        return hipErrorInvalidValue;
    // shares of an even number of steps each, none empty
    p.share_steps = ((steps / 2 + shares - 1) / shares) * 2;
    shares = (steps + p.share_steps - 1) / p.share_steps;
    p.tiles_n = (p.n + BN - 1) / BN;
    p.tiles_m = (p.m + BM - 1) / BM;
    if (size_t(p.tiles_n) * size_t(p.tiles_m) > 0x7fffffffu)
        return hipErrorInvalidValue;
    const dim3 grid(unsigned(p.tiles_n) * unsigned(p.tiles_m), unsigned(shares));
    bgemm_wave4_kernel<NA, NN><<<grid, 256, 0, stream>>>(p);
    const hipError_t status = launch_status();
    if (shares == 1 || status != hipSuccess)
        return status;
    return launch_sum_shares(stream, p, shares);
}
} // namespace

hipError_t launch_bgemm_wave4(hipStream_t stream, int rows, DmaParams p, int shares, bool weights_as_they_lie)
{
    if (weights_as_they_lie)
        return rows == 256 ? launch<8, true>(stream, p, shares) : hipErrorInvalidValue;
    return rows == 320 ? launch<10>(stream, p, shares) : rows == 256 ? launch<8>(stream, p, shares) : hipErrorInvalidValue;
}
} // namespace camblas_hip
