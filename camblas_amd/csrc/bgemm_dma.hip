// Compute-bound BF16 prefill linear y[M,N] = alpha * x[M,K] * W[N,K]^T + beta * y: large MFMA
// tiles fed by direct global->LDS loads.
//
// A workgroup of four wavefronts (2 x 2) owns a (64*TN) x (64*TM) output tile; each wavefront
// accumulates a (32*TN) x (32*TM) block in TN*TM v_mfma_f32_32x32x16_bf16 accumulators (FP32).
// K advances 64 elements per step through two LDS stages. The next step's operands are fetched with
// global_load_lds_dwordx4: each lane names the 16-byte chunk of W or x that belongs in its LDS slot,
// so the data lands in the XOR-swizzled layout the MFMA-layout reads expect without passing through
// registers (no staging VGPRs, no ds_write). The two stages are separate LDS objects so the
// compiler can tell the in-flight stage from the one being read. Fragments of the next 16-deep
// step are read while the current step's MFMAs issue. Workgroups are renumbered per XCD so the
// tiles resident on one XCD share W and x panels through its L2.
// With few tokens the tiles of a projection leave compute units idle; the K steps of a tile can then
// be divided over gridDim.y workgroups, which leave FP32 planes that sum_shares_kernel adds in share
// order and finishes with alpha, beta and the addend.
// Shape requirements (the planner checks them): K % 64 == 0, N % 4 == 0, ldc % 4 == 0, 16-byte
// aligned operands, 8-byte aligned y.
// Contract: ref src/cuda/bfloat16.cuh:11-57 ('T','N' call of src/cuda/torch_bindings.cpp:155-199).
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"
#include "bgemm_dma.hpp"

namespace camblas_hip
{
namespace
{
// TN, TM: 32x32 MFMA tiles per wavefront along features / tokens; the workgroup has 2 x WM
// wavefronts and owns a (64*TN) x (32*WM*TM) tile; BK: K elements per step (32 or 64); STAGES: LDS
// stages (STAGES - 1 steps are in flight).
template <int TN, int TM, int WM, int BK, int STAGES>
__global__ __launch_bounds__(128 * WM) void bgemm_dma_kernel(DmaParams p)
{
    constexpr int WAVES = 2 * WM;
    constexpr int BN = 64 * TN, BM = 32 * WM * TM, CH = BK / 8;
    constexpr int ROWS_PER_LOAD = 64 / CH;               // rows one wave instruction fills
    constexpr int A_ITERS = BN / (WAVES * ROWS_PER_LOAD), B_ITERS = BM / (WAVES * ROWS_PER_LOAD);
    static_assert(BN % (WAVES * ROWS_PER_LOAD) == 0 && BM % (WAVES * ROWS_PER_LOAD) == 0 &&
                      (BK / 16) % 2 == 0,
                  "every wavefront issues whole loads; fragment buffers alternate evenly");
    constexpr int LOADS = A_ITERS + B_ITERS;             // direct loads per wavefront and step
    constexpr int SLOTS = (BN + BM) * CH;
    static_assert(STAGES >= 2 && STAGES <= 4 && (BK == 32 || BK == 64), "pipeline shape");
    static_assert(LOADS * (STAGES - 2) < 64, "vmcnt holds 6 bits");
    // One LDS object per stage so that reads of one stage and in-flight writes of another are
    // provably disjoint.
    __shared__ u32x4_t stage0[SLOTS];
    __shared__ u32x4_t stage1[SLOTS];
    __shared__ u32x4_t stage2[STAGES > 2 ? SLOTS : 1];
    __shared__ u32x4_t stage3[STAGES > 3 ? SLOTS : 1];

    int tile_n, tile_m;
    xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int first_step = int(blockIdx.y) * p.share_steps;
    const int k_tiles = p.k / BK - first_step < p.share_steps ? p.k / BK - first_step : p.share_steps;

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int wn = wave % 2, wm = wave / 2; // 2 x WM wavefront grid

    // ---- per-lane sources of the direct loads. Wave-instruction (it, wave) fills LDS slots
    // [(it*WAVES + wave)*64, +64): row = (it*WAVES + wave)*ROWS_PER_LOAD + lane/CH, chunk lane%CH,
    // which holds logical chunk (lane%CH) ^ swizzle(row). The address is the tile's buffer
    // resource plus a constant 32-bit per-lane byte offset plus a scalar offset that advances by
    // 2*BK per step: no vector arithmetic in the loop.
    // Successive loads of a thread are WAVES*ROWS_PER_LOAD rows apart, a multiple of 16, which
    // leaves the swizzle unchanged, so one lane offset per operand serves all of them and the row
    // advance goes into the scalar offset. Rows past the end of the matrix lie outside the buffer
    // resource and read as zero.
    static_assert((WAVES * ROWS_PER_LOAD) % 16 == 0, "row step keeps the swizzle");
    const int load_row = wave * ROWS_PER_LOAD + lane / CH;
    const unsigned load_chunk = unsigned(((lane % CH) ^ lds_swizzle<CH>(load_row)) * 8);
    const unsigned a_lane_off = (unsigned(load_row) * unsigned(p.lda) + load_chunk) * 2u;
    const unsigned b_lane_off = (unsigned(load_row) * unsigned(p.ldb) + load_chunk) * 2u;
    const unsigned a_row_step = unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.lda) * 2u;
    const unsigned b_row_step = unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.ldb) * 2u;
    // One resource per operand, covering exactly the rows of this tile that exist.
    const int a_rows = p.n - n0 < BN ? p.n - n0 : BN, b_rows = p.m - m0 < BM ? p.m - m0 : BM;
    const __amdgpu_buffer_rsrc_t a_resource = make_resource(
        p.w + size_t(n0) * p.lda, (unsigned(a_rows - 1) * unsigned(p.lda) + unsigned(p.k)) * 2u);
    const __amdgpu_buffer_rsrc_t b_resource = make_resource(
        p.x + size_t(m0) * p.ldb, (unsigned(b_rows - 1) * unsigned(p.ldb) + unsigned(p.k)) * 2u);
    unsigned k_bytes = unsigned(first_step) * BK * 2;
    // Load number `index` (0 .. LOADS-1) of the K block at k_bytes.
    auto issue_one = [&](u32x4_t *stage, int index) {
        if (index < A_ITERS)
            load_to_lds(a_resource, a_lane_off, k_bytes + unsigned(index) * a_row_step,
                        stage + (index * WAVES + wave) * 64);
        else
            load_to_lds(b_resource, b_lane_off, k_bytes + unsigned(index - A_ITERS) * b_row_step,
                        stage + BN * CH + ((index - A_ITERS) * WAVES + wave) * 64);
    };
    auto issue = [&](u32x4_t *stage) {
#pragma unroll
        for (int index = 0; index < LOADS; ++index)
            issue_one(stage, index);
        k_bytes += BK * 2;
    };

    // ---- MFMA-layout read positions
    const int frag_row = lane % 32, half = lane / 32;
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

    // Fragment registers are double-buffered across the 16-deep sub-steps: while the MFMAs of one
    // sub-step issue, the operands of the next are already on their way from LDS. The last
    // sub-step of a K step overlaps with the first fragment reads of the next stage, which become
    // legal once this wavefront's loads for that stage have landed and all wavefronts have met at
    // the barrier (which also tells everyone that the current stage may be overwritten).
    bf16x8_t a_frag[2][TN], b_frag[2][TM];
    auto read = [&](const u32x4_t *stage, int ks, bf16x8_t(&a)[TN], bf16x8_t(&b)[TM]) {
        const int column = (ks * 2 + half) ^ frag_swizzle;
#pragma unroll
        for (int i = 0; i < TN; ++i)
            a[i] = __builtin_bit_cast(bf16x8_t, stage[a_frag_base + i * 32 * CH + column]);
#pragma unroll
        for (int j = 0; j < TM; ++j)
            b[j] = __builtin_bit_cast(bf16x8_t, stage[b_frag_base + j * 32 * CH + column]);
    };
    auto mfma = [&](const bf16x8_t(&a)[TN], const bf16x8_t(&b)[TM]) {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
                acc[i][j] =
                    __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    };
    constexpr int KS = BK / 16;
    // One pipeline step: start the loads of step (tile + STAGES - 1) into the stage that was read
    // last, run the sub-steps of the current stage, and hand over to `next`. Loads are issued
    // unconditionally; steps past the end re-read the last K block into a stage nobody multiplies,
    // which keeps the outstanding-load count fixed.
    // sched_barrier(0) pins this order; left alone, the scheduler sinks the direct loads to the
    // end of the step and moves every fragment read next to its first use, which exposes both
    // latencies.
    auto step = [&](u32x4_t *fill, const u32x4_t *current, const u32x4_t *next) {
        // all fills of the step are issued up front: spreading them over the sub-steps measured
        // 8 % slower on the 320 x 256 tile
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int index = 0; index < LOADS; ++index)
            issue_one(fill, index);
#pragma unroll
        for (int ks = 0; ks + 1 < KS; ++ks) {
            __builtin_amdgcn_sched_barrier(0);
            read(current, ks + 1, a_frag[(ks + 1) & 1], b_frag[(ks + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            mfma(a_frag[ks & 1], b_frag[ks & 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        k_bytes += BK * 2;
        pipeline_barrier<LOADS *(STAGES - 2)>();
        read(next, 0, a_frag[0], b_frag[0]);
        __builtin_amdgcn_sched_barrier(0);
        mfma(a_frag[(KS - 1) & 1], b_frag[(KS - 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
    };
    const unsigned last_k_bytes = unsigned(first_step + k_tiles - 1) * BK * 2;
    auto clamp_k = [&]() { k_bytes = k_bytes < last_k_bytes ? k_bytes : last_k_bytes; };

    // prologue: STAGES - 1 steps in flight, the first one complete
    issue(stage0);
    clamp_k();
    if constexpr (STAGES > 2) {
        issue(stage1);
        clamp_k();
    }
    if constexpr (STAGES > 3) {
        issue(stage2);
        clamp_k();
    }
    pipeline_barrier<LOADS *(STAGES - 2)>();
    read(stage0, 0, a_frag[0], b_frag[0]);
    for (int tile = 0; tile < k_tiles; tile += STAGES) {
        if constexpr (STAGES == 2) {
            step(stage1, stage0, stage1);
            clamp_k();
            if (tile + 1 < k_tiles)
                step(stage0, stage1, stage0);
            clamp_k();
        } else if constexpr (STAGES == 3) {
            step(stage2, stage0, stage1);
            clamp_k();
            if (tile + 1 < k_tiles)
                step(stage0, stage1, stage2);
            clamp_k();
            if (tile + 2 < k_tiles)
                step(stage1, stage2, stage0);
            clamp_k();
        } else {
            step(stage3, stage0, stage1);
            clamp_k();
            if (tile + 1 < k_tiles)
                step(stage0, stage1, stage2);
            clamp_k();
            if (tile + 2 < k_tiles)
                step(stage1, stage2, stage3);
            clamp_k();
            if (tile + 3 < k_tiles)
                step(stage2, stage3, stage0);
            clamp_k();
        }
    }
    wait_loads<0>(); // drain the padding loads before the LDS is released

    // ---- epilogue. Accumulator register 4q+e of lane l is feature 8q + 4*(l/32) + e, token l%32.
    const int first_feature = n0 + wn * TN * 32 + half * 4;
    if (gridDim.y > 1) {
        // a share of K: the plain sums, for sum_shares_kernel
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                const int m = m0 + (wm * TM + j) * 32 + frag_row;
                float *row = p.partials + (size_t(blockIdx.y) * p.m + m) * p.n + first_feature;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int offset = i * 32 + q * 8;
                    if (m < p.m && first_feature + offset < p.n) {
                        const f32x4_t sums = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                                              acc[i][j][q * 4 + 3]};
                        *reinterpret_cast<f32x4_t *>(row + offset) = sums;
                    }
                }
            }
        return;
    }
    auto store_tile = [&](int i, int j, const u32x2_t (&old)[4], bool with_beta) {
        const int m = m0 + (wm * TM + j) * 32 + frag_row;
        unsigned short *row = p.y + size_t(m) * p.ldc + first_feature;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int offset = i * 32 + q * 8;
            if (m < p.m && first_feature + offset < p.n) {
                float v0 = p.alpha * acc[i][j][q * 4], v1 = p.alpha * acc[i][j][q * 4 + 1];
                float v2 = p.alpha * acc[i][j][q * 4 + 2], v3 = p.alpha * acc[i][j][q * 4 + 3];
                if (with_beta) {
                    v0 = fmaf(p.beta, __uint_as_float(old[q][0] << 16), v0);
                    v1 = fmaf(p.beta, __uint_as_float(old[q][0] & 0xffff0000u), v1);
                    v2 = fmaf(p.beta, __uint_as_float(old[q][1] << 16), v2);
                    v3 = fmaf(p.beta, __uint_as_float(old[q][1] & 0xffff0000u), v3);
                }
                u32x2_t packed = {pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
                *reinterpret_cast<u32x2_t *>(row + offset) = packed;
            }
        }
    };
    if (p.beta == 0.f) {
        const u32x2_t nothing[4] = {};
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                __builtin_amdgcn_sched_barrier(0); // keep one accumulator tile live at a time
                store_tile(i, j, nothing, false);
            }
        return;
    }
    // beta term: the addend of tile t + 1 is fetched while tile t is scaled and stored (one load
    // latency per tile would otherwise be exposed twenty times: measured +56 us on a 506 us product,
    // +29 us with the fetch one tile ahead, no better two tiles ahead). The loads are unconditional: a
    // position outside the matrix reads the first element of a valid row instead and is not used.
    constexpr int AHEAD = 1;
    u32x2_t old[AHEAD + 1][4];
    auto fetch_tile = [&](int t, u32x2_t (&into)[4]) {
        const int i = t % TN, j = t / TN;
        int m = m0 + (wm * TM + j) * 32 + frag_row;
        m = m < p.m ? m : p.m - 1;
        const unsigned short *source = p.z + size_t(m) * p.ldz;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int feature = first_feature + i * 32 + q * 8;
            into[q] = *reinterpret_cast<const u32x2_t *>(source + (feature < p.n ? feature : 0));
        }
    };
#pragma unroll
    for (int t = 0; t < AHEAD && t < TN * TM; ++t)
        fetch_tile(t, old[t]);
#pragma unroll
    for (int t = 0; t < TN * TM; ++t) {
        __builtin_amdgcn_sched_barrier(0);
        if (t + AHEAD < TN * TM)
            fetch_tile(t + AHEAD, old[(t + AHEAD) % (AHEAD + 1)]);
        __builtin_amdgcn_sched_barrier(0);
        store_tile(t % TN, t / TN, old[t % (AHEAD + 1)], true);
    }
}

// The same workgroup tile on v_mfma_f32_16x16x32_bf16. On operands with random bits the part sustains
// 2.19 PFLOP/s with this instruction against 1.83 with the 32 x 32 x 16 one (it holds a higher clock:
// measured with launches of nothing but matrix instructions), and the prefill kernel is limited by
// that clock. A wavefront's (32*TN) x (32*TM) block is 2TN x 2TM tiles of 16 x 16 with four accumulator
// registers each; a K step of 64 is two sub-steps of 32, in each of which every one of the 2TN
// weight fragments (16 rows x 32 K: lane l holds K values 8*(l/16) .. +7 of row l%16) meets all 2TM
// token fragments. The token fragments of a sub-step are read during the previous one, the weight
// fragments travel RING-1 fragments ahead of their use in a ring of registers; the barrier of a step
// lies RING-1 fragments before its end, so that the first fragments of the next stage are on their
// way while the last matrix instructions of this one issue.
template <int TN, int TM, int WM, int BK, int STAGES>
__global__ __launch_bounds__(128 * WM) void bgemm_dma16_kernel(DmaParams p)
{
    constexpr int WAVES = 2 * WM;
    constexpr int BN = 64 * TN, BM = 32 * WM * TM, CH = BK / 8;
    constexpr int ROWS_PER_LOAD = 64 / CH;
    constexpr int A_ITERS = BN / (WAVES * ROWS_PER_LOAD), B_ITERS = BM / (WAVES * ROWS_PER_LOAD);
    static_assert(BK == 64 && BN % (WAVES * ROWS_PER_LOAD) == 0 && BM % (WAVES * ROWS_PER_LOAD) == 0,
                  "every wavefront issues whole loads");
    constexpr int LOADS = A_ITERS + B_ITERS;
    constexpr int SLOTS = (BN + BM) * CH;
    static_assert(STAGES >= 2 && STAGES <= 3, "pipeline shape");
    __shared__ u32x4_t stage0[SLOTS];
    __shared__ u32x4_t stage1[SLOTS];
    __shared__ u32x4_t stage2[STAGES > 2 ? SLOTS : 1];

    int tile_n, tile_m;
    xcd_tile(int(blockIdx.x), p.tiles_n, p.tiles_m, tile_n, tile_m);
    const int n0 = tile_n * BN, m0 = tile_m * BM;
    const int first_step = int(blockIdx.y) * p.share_steps;
    const int k_tiles = p.k / BK - first_step < p.share_steps ? p.k / BK - first_step : p.share_steps;

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int wn = wave % 2, wm = wave / 2;

    // ---- fills: as in bgemm_dma_kernel
    static_assert((WAVES * ROWS_PER_LOAD) % 16 == 0, "row step keeps the swizzle");
    const int load_row = wave * ROWS_PER_LOAD + lane / CH;
    const unsigned load_chunk = unsigned(((lane % CH) ^ lds_swizzle<CH>(load_row)) * 8);
    const unsigned a_lane_off = (unsigned(load_row) * unsigned(p.lda) + load_chunk) * 2u;
    const unsigned b_lane_off = (unsigned(load_row) * unsigned(p.ldb) + load_chunk) * 2u;
    const unsigned a_row_step = unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.lda) * 2u;
    const unsigned b_row_step = unsigned(WAVES * ROWS_PER_LOAD) * unsigned(p.ldb) * 2u;
    const int a_rows = p.n - n0 < BN ? p.n - n0 : BN, b_rows = p.m - m0 < BM ? p.m - m0 : BM;
    const __amdgpu_buffer_rsrc_t a_resource = make_resource(
        p.w + size_t(n0) * p.lda, (unsigned(a_rows - 1) * unsigned(p.lda) + unsigned(p.k)) * 2u);
    const __amdgpu_buffer_rsrc_t b_resource = make_resource(
        p.x + size_t(m0) * p.ldb, (unsigned(b_rows - 1) * unsigned(p.ldb) + unsigned(p.k)) * 2u);
    unsigned k_bytes = unsigned(first_step) * BK * 2;
    const unsigned last_k_bytes = unsigned(first_step + k_tiles - 1) * BK * 2;
    auto issue = [&](u32x4_t *stage) {
#pragma unroll
        for (int index = 0; index < LOADS; ++index) {
            if (index < A_ITERS)
                load_to_lds(a_resource, a_lane_off, k_bytes + unsigned(index) * a_row_step,
                            stage + (index * WAVES + wave) * 64);
            else
                load_to_lds(b_resource, b_lane_off, k_bytes + unsigned(index - A_ITERS) * b_row_step,
                            stage + BN * CH + ((index - A_ITERS) * WAVES + wave) * 64);
        }
        // (steps past the end re-read the last K block into a stage nobody multiplies)
        k_bytes = k_bytes + BK * 2 < last_k_bytes ? k_bytes + BK * 2 : last_k_bytes;
    };

    // ---- fragments
    // (measured: the 256 x 256 tile is 3 % faster with a ring of two than of four, 5 % slower with eight; the
    // 320 x 256 tile is indifferent; the 128 x 128 tile of four wavefronts is 3 to 5 % faster when the
    // compiler is left to order fragment reads and matrix instructions inside a step, the 128 x 256 tile
    // 1 % slower and the larger ones 15 % slower)
    constexpr int NA = 2 * TN, NB = 2 * TM, KS = BK / 32, ITEMS = KS * NA, RING = TN == 4 && TM == 2 ? 2 : 4;
    constexpr bool FENCED = !(TN == 2 && WM == 2);
    static_assert(ITEMS % RING == 0 && KS % 2 == 0, "ring slots and token buffers line up from step to step");
    const int frag_row = lane % 16, group = lane / 16;
    const int frag_swizzle = lds_swizzle<CH>(frag_row);
    const int a_frag_base = (wn * TN * 32 + frag_row) * CH;
    const int b_frag_base = BN * CH + (wm * TM * 32 + frag_row) * CH;
    f32x4_t acc[NA][NB];
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
            acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    bf16x8_t a_ring[RING], b_buffer[2][NB];
    auto read_a = [&](const u32x4_t *stage, int item) { // item = sub-step * NA + weight tile
        const int ks = item / NA, i = item % NA;
        a_ring[item % RING] =
            __builtin_bit_cast(bf16x8_t, stage[a_frag_base + i * 16 * CH + ((ks * 4 + group) ^ frag_swizzle)]);
    };
    auto read_b = [&](const u32x4_t *stage, int ks) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
            b_buffer[ks & 1][j] =
                __builtin_bit_cast(bf16x8_t, stage[b_frag_base + j * 16 * CH + ((ks * 4 + group) ^ frag_swizzle)]);
    };
    auto step = [&](u32x4_t *fill, const u32x4_t *current, const u32x4_t *next) {
        __builtin_amdgcn_sched_barrier(0);
        issue(fill);
#pragma unroll
        for (int item = 0; item < ITEMS; ++item) {
            const int ks = item / NA, i = item % NA, ahead = item + RING - 1;
            if constexpr (FENCED)
                __builtin_amdgcn_sched_barrier(0);
            if (item == ITEMS - (RING - 1)) {
                pipeline_barrier<LOADS *(STAGES - 2)>();
                read_b(next, 0);
            }
            if (ahead < ITEMS)
                read_a(current, ahead);
            else
                read_a(next, ahead - ITEMS);
            if (i == 0 && ks + 1 < KS)
                read_b(current, ks + 1);
            if constexpr (FENCED)
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NB; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_ring[item % RING], b_buffer[ks & 1][j],
                                                                    acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    issue(stage0);
    if constexpr (STAGES > 2)
        issue(stage1);
    pipeline_barrier<LOADS *(STAGES - 2)>();
    read_b(stage0, 0);
#pragma unroll
    for (int item = 0; item < RING - 1; ++item)
        read_a(stage0, item);
    for (int tile = 0; tile < k_tiles; tile += STAGES) {
        if constexpr (STAGES == 2) {
            step(stage1, stage0, stage1);
            if (tile + 1 < k_tiles)
                step(stage0, stage1, stage0);
        } else {
            step(stage2, stage0, stage1);
            if (tile + 1 < k_tiles)
                step(stage0, stage1, stage2);
            if (tile + 2 < k_tiles)
                step(stage1, stage2, stage0);
        }
    }
    wait_loads<0>();

    // ---- epilogue. Register e of lane l in tile (i, j) is feature 16 i + 4 (l / 16) + e, token 16 j + l % 16.
    const int first_feature = n0 + wn * TN * 32 + group * 4;
    const int first_token = m0 + wm * TM * 32 + frag_row;
    if (gridDim.y > 1) { // a share of K: the plain sums, for sum_shares_kernel
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                const int m = first_token + j * 16, n = first_feature + i * 16;
                if (m < p.m && n < p.n)
                    *reinterpret_cast<f32x4_t *>(p.partials + (size_t(blockIdx.y) * p.m + m) * p.n + n) = acc[i][j];
            }
        return;
    }
    auto store_tile = [&](int i, int j, u32x2_t old, bool with_beta) {
        const int m = first_token + j * 16, n = first_feature + i * 16;
        if (m < p.m && n < p.n) {
            float v0 = p.alpha * acc[i][j][0], v1 = p.alpha * acc[i][j][1];
            float v2 = p.alpha * acc[i][j][2], v3 = p.alpha * acc[i][j][3];
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

// y = alpha * (plane 0 + plane 1 + ...) + beta * z over the shares of a divided K, four features per
// thread, the planes added in index order so that the result does not depend on scheduling.
__global__ __launch_bounds__(256) void sum_shares_kernel(DmaParams p, int shares)
{
    const size_t quad = size_t(blockIdx.x) * 256 + threadIdx.x, per_row = size_t(p.n / 4);
    if (quad >= per_row * size_t(p.m))
        return;
    const size_t m = quad / per_row, feature = quad % per_row * 4, plane = size_t(p.m) * p.n;
    const float *source = p.partials + m * p.n + feature;
    f32x4_t sum = *reinterpret_cast<const f32x4_t *>(source);
    for (int share = 1; share < shares; ++share) {
        const f32x4_t more = *reinterpret_cast<const f32x4_t *>(source + share * plane);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            sum[e] += more[e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
        sum[e] *= p.alpha;
    if (p.beta != 0.f) {
        const u32x2_t old = *reinterpret_cast<const u32x2_t *>(p.z + m * p.ldz + feature);
        sum[0] = fmaf(p.beta, __uint_as_float(old[0] << 16), sum[0]);
        sum[1] = fmaf(p.beta, __uint_as_float(old[0] & 0xffff0000u), sum[1]);
        sum[2] = fmaf(p.beta, __uint_as_float(old[1] << 16), sum[2]);
        sum[3] = fmaf(p.beta, __uint_as_float(old[1] & 0xffff0000u), sum[3]);
    }
    const u32x2_t packed = {pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3])};
    *reinterpret_cast<u32x2_t *>(p.y + m * p.ldc + feature) = packed;
}

template <int TN, int TM, int WM, int BK, int STAGES>
hipError_t launch_dma(hipStream_t stream, DmaParams p, int shares)
{
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    if (p.k % BK)
        return hipErrorInvalidValue;
    p.tiles_n = (p.n + BN - 1) / BN;
    p.tiles_m = (p.m + BM - 1) / BM;
    if (size_t(p.tiles_n) * size_t(p.tiles_m) > 0x7fffffffu)
        return hipErrorInvalidValue;
    const int steps = p.k / BK;
    p.share_steps = (steps + shares - 1) / shares;
    shares = (steps + p.share_steps - 1) / p.share_steps; // no empty share
    const dim3 grid(unsigned(p.tiles_n) * unsigned(p.tiles_m), unsigned(shares));
    bgemm_dma_kernel<TN, TM, WM, BK, STAGES><<<grid, 128 * WM, 0, stream>>>(p);
    const hipError_t status = launch_status();
    if (shares == 1 || status != hipSuccess)
        return status;
    const size_t quads = size_t(p.m) * size_t(p.n / 4);
    sum_shares_kernel<<<unsigned((quads + 255) / 256), 256, 0, stream>>>(p, shares);
    return launch_status();
}

template <int TN, int TM, int WM, int BK, int STAGES>
hipError_t launch_dma16(hipStream_t stream, DmaParams p, int shares)
{
    constexpr int BN = 64 * TN, BM = 32 * WM * TM;
    if (p.k % BK)
        return hipErrorInvalidValue;
    p.tiles_n = (p.n + BN - 1) / BN;
    p.tiles_m = (p.m + BM - 1) / BM;
    if (size_t(p.tiles_n) * size_t(p.tiles_m) > 0x7fffffffu)
        return hipErrorInvalidValue;
    const int steps = p.k / BK;
    p.share_steps = (steps + shares - 1) / shares;
    shares = (steps + p.share_steps - 1) / p.share_steps; // no empty share
    const dim3 grid(unsigned(p.tiles_n) * unsigned(p.tiles_m), unsigned(shares));
    bgemm_dma16_kernel<TN, TM, WM, BK, STAGES><<<grid, 128 * WM, 0, stream>>>(p);
    const hipError_t status = launch_status();
    if (shares == 1 || status != hipSuccess)
        return status;
    const size_t quads = size_t(p.m) * size_t(p.n / 4);
    sum_shares_kernel<<<unsigned((quads + 255) / 256), 256, 0, stream>>>(p, shares);
    return launch_status();
}

const TnVariant variants[] = {
    {"dma256x256x32s4w4", 256, 256, 32, 256}, {"dma256x128x64s3w4", 256, 128, 64, 256},
    {"dma128x128x64s2w4", 128, 128, 64, 256}, {"dma256x256x32s3w4", 256, 256, 32, 256},
    {"dma256x128x64s2w4", 256, 128, 64, 256}, {"dma128x128x64s3w4", 128, 128, 64, 256},
    {"dma256x256x64s2w8", 256, 256, 64, 512}, {"dma256x256x32s4w8", 256, 256, 32, 512},
    {"dma256x128x64s3w8", 256, 128, 64, 512}, {"dma128x256x64s3w8", 128, 256, 64, 512},
    {"dma320x256x64s2w8", 320, 256, 64, 512}, {"dma192x256x64s2w8", 192, 256, 64, 512},
    // the same tiles on the 16 x 16 x 32 matrix instruction
    {"dma16-320x256x64s2w8", 320, 256, 64, 512}, {"dma16-256x256x64s2w8", 256, 256, 64, 512},
    {"dma16-192x256x64s2w8", 192, 256, 64, 512}, {"dma16-128x256x64s3w8", 128, 256, 64, 512},
    {"dma16-256x128x64s3w8", 256, 128, 64, 512}, {"dma16-128x128x64s3w4", 128, 128, 64, 256},
    // four wavefronts, one per SIMD, K loop in assembly (bgemm_wave4.hip); K % 128 == 0
    {"wave4-256x256x64s2", 256, 256, 64, 256}, {"wave4-320x256x64s2", 320, 256, 64, 256},
    // the 256 x 256 tile for weights W[K, N] with the outputs contiguous ('N','N': w and lda describe W as it lies)
    {"wave4-256x256x64s2-weights-as-they-lie", 256, 256, 64, 256},
};
} // namespace

hipError_t launch_sum_shares(hipStream_t stream, const DmaParams &p, int shares)
{
    const size_t quads = size_t(p.m) * size_t(p.n / 4);
    sum_shares_kernel<<<unsigned((quads + 255) / 256), 256, 0, stream>>>(p, shares);
    return launch_status();
}

hipError_t launch_sum_shares(hipStream_t stream, const float *partials, int shares, int n_out, int m_rows,
                             float alpha, float beta, const void *z, int ldz, void *y, int ldc)
{
    if (n_out % 4 || ldc % 4 || ldz % 4 || reinterpret_cast<uintptr_t>(y) % 8 || reinterpret_cast<uintptr_t>(z) % 8 ||
        size_t(m_rows) * size_t(n_out / 4) > size_t(0x7fffffff) * 256)
        return hipErrorInvalidValue;
    DmaParams p = {};
    p.partials = const_cast<float *>(partials);
    p.n = n_out;
    p.m = m_rows;
    p.alpha = alpha;
    p.beta = beta;
    p.z = static_cast<const unsigned short *>(z);
    p.ldz = ldz;
    p.y = static_cast<unsigned short *>(y);
    p.ldc = ldc;
    const size_t quads = size_t(m_rows) * size_t(n_out / 4);
    sum_shares_kernel<<<unsigned((quads + 255) / 256), 256, 0, stream>>>(p, shares);
    return launch_status();
}

int dma_variant_count() { return int(sizeof(variants) / sizeof(variants[0])); }
const TnVariant &dma_variant(int index) { return variants[index]; }

hipError_t launch_bgemm_dma(hipStream_t stream, int variant, int n_out, int m_rows, int k,
                            float alpha, const void *w, int lda, const void *x, int ldb, float beta,
                            void *y, int ldc, const BetaSource &source, int shares, float *partials)
{
    if (k % 64 || n_out % 4 || ldc % 4 || reinterpret_cast<uintptr_t>(y) % 8)
        return hipErrorInvalidValue;
    if (shares < 1 || shares > 64 || (shares > 1 && !partials) ||
        size_t(m_rows) * size_t(n_out / 4) > size_t(0x7fffffff) * 256)
        return hipErrorInvalidValue;
    if (source.z && (source.ldz % 4 || reinterpret_cast<uintptr_t>(source.z) % 8))
        return hipErrorInvalidValue;
    // per-lane byte offsets are 32-bit: 256 rows of the widest operand plus the K extent must fit
    if ((size_t(256) * size_t(lda > ldb ? lda : ldb) + size_t(k)) * 2 >= (size_t(1) << 32))
        return hipErrorInvalidValue;
    DmaParams p;
    p.w = static_cast<const unsigned short *>(w);
    p.x = static_cast<const unsigned short *>(x);
    p.y = static_cast<unsigned short *>(y);
    p.lda = lda;
    p.ldb = ldb;
    p.ldc = ldc;
    p.z = source.z ? static_cast<const unsigned short *>(source.z) : p.y;
    p.ldz = source.z ? source.ldz : ldc;
    p.n = n_out;
    p.m = m_rows;
    p.k = k;
    p.alpha = alpha;
    p.beta = beta;
    p.tiles_n = p.tiles_m = 0;
    p.partials = partials;
    p.share_steps = 0;
    switch (variant) {
    case 0: return launch_dma<4, 4, 2, 32, 4>(stream, p, shares);
    case 1: return launch_dma<4, 2, 2, 64, 3>(stream, p, shares);
    case 2: return launch_dma<2, 2, 2, 64, 2>(stream, p, shares);
    case 3: return launch_dma<4, 4, 2, 32, 3>(stream, p, shares);
    case 4: return launch_dma<4, 2, 2, 64, 2>(stream, p, shares);
    case 5: return launch_dma<2, 2, 2, 64, 3>(stream, p, shares);
    case 6: return launch_dma<4, 2, 4, 64, 2>(stream, p, shares);
    case 7: return launch_dma<4, 2, 4, 32, 4>(stream, p, shares);
    case 8: return launch_dma<4, 1, 4, 64, 3>(stream, p, shares);
    case 9: return launch_dma<2, 2, 4, 64, 3>(stream, p, shares);
    case 10: return launch_dma<5, 2, 4, 64, 2>(stream, p, shares);
    case 11: return launch_dma<3, 2, 4, 64, 2>(stream, p, shares);
    case 12: return launch_dma16<5, 2, 4, 64, 2>(stream, p, shares);
    case 13: return launch_dma16<4, 2, 4, 64, 2>(stream, p, shares);
    case 14: return launch_dma16<3, 2, 4, 64, 2>(stream, p, shares);
    case 15: return launch_dma16<2, 2, 4, 64, 3>(stream, p, shares);
    case 16: return launch_dma16<4, 1, 4, 64, 3>(stream, p, shares);
    case 17: return launch_dma16<2, 2, 2, 64, 3>(stream, p, shares);
    case 18: return launch_bgemm_wave4(stream, 256, p, shares);
    case 19: return launch_bgemm_wave4(stream, 320, p, shares);
    case 20: return launch_bgemm_wave4(stream, 256, p, shares, true);
    default: return hipErrorInvalidValue;
    }
}
} // namespace camblas_hip
