// Bandwidth-bound BF16 decode linear y[M,N] = alpha * x[M,K] * W[N,K]^T + beta * y for small M.
//
// The whole cost is reading W once from HBM, so the kernel is organised around the weight stream:
// one workgroup owns 16*NT consecutive weight rows for the whole K extent (about one workgroup per
// compute unit for a Llama-sized projection) and marches along K in steps of KT 128-element
// blocks. Two K steps are in flight in registers per thread (128-bit loads, 256 contiguous bytes
// per row and block) while a third is multiplied, so a compute unit keeps 2 * 16*NT * KT * 256
// bytes outstanding; KT grows as NT shrinks (projections with few output rows) so that this stays
// near 64 KB, which is what it takes to cover the HBM latency at full bandwidth. Tiles are staged
// in LDS with a 16-way XOR swizzle (conflict-free 128-bit stores and MFMA-layout reads). The four
// wavefronts split each 128-element block four ways (v_mfma_f32_16x16x32_bf16, FP32 accumulate)
// and their partial sums are combined in wavefront order at the end, so results do not depend on
// scheduling. No split-K pass and no scratch.
// Contract: ref src/cuda/bfloat16.cuh:11-57 for the ('T','N') call of a linear
// (src/cuda/torch_bindings.cpp:146-199); the reference's own decode kernel class is
// src/cuda/decode_float.cuh:2-52 (FP32, one vector).
//
// This header holds the kernel and its launch templates; the instantiations are spread over several
// translation units that compile side by side (bgemv_stream.hip: one K block per step;
// bgemv_stream_deep.hip: two to eight; bgemv_stream_norm.hip and bgemv_stream_residual.hip: the fused
// halves; bgemv_stream_gated.hip: the gated form; bgemv_stream_many.hip: more than four token tiles), each
// behind one of the functions declared at the end.
#pragma once
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
struct StreamParams {
    const unsigned short *w;
    const unsigned short *w2; // gated form: the "up" weights (w holds the "gate" weights)
    const unsigned short *x;
    unsigned short *y;
    const unsigned short *z; // what beta multiplies: z[token * ldz + feature] (y and ldc by default)
    int lda, ldb, ldc, ldz;
    int n, m, k;
    float alpha, beta;
    int vector_store; // 8-byte accesses to y (and z) rows are aligned
    // K divided over gridDim.z workgroups per output tile: FP32 planes [gridDim.z, m, n] and one
    // arrival counter per (blockIdx.x, blockIdx.y), zero before and after every launch
    float *partials;
    unsigned *arrivals;
    // ---- the FUSE instantiations only
    // x is normalised while it is staged: round(round(x * scale[token]) * norm_weight[k]) with
    // scale = rsqrt(sum / k + epsilon), sum = ssq_in[0][token] + ssq_in[1][token] + ... in index order
    const unsigned short *norm_weight;
    const float *ssq_in;
    int ssq_count, ssq_ld;
    float epsilon;
    // y = round(round(alpha * x W^T) + residual[token * ld_residual + feature]), and workgroup
    // blockIdx.x leaves the sums of squares of its features of every row of y in
    // ssq_out[blockIdx.x * ssq_ld_out + token] (fixed order)
    const unsigned short *residual;
    int ld_residual;
    float *ssq_out;
    int ssq_ld_out;
};

namespace
{
constexpr int WAVES = 4, DEPTH = 2;
// passes in which the wavefronts' partial tiles (1 KB each) go through LDS at the end of a workgroup
constexpr int stream_combine_passes(int row_tiles, int token_tiles) { return WAVES * row_tiles * token_tiles > 144 ? 2 : 1; }

typedef float f32x2_round_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_round_t __attribute__((ext_vector_type(2)));
// two FP32 values rounded to nearest-even BF16 and packed, by the conversion instruction of gfx950
__device__ __forceinline__ unsigned round_pack_bf16x2(float lo, float hi)
{
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_round_t{lo, hi}, bf16x2_round_t));
}

// NT, MT: 16-row weight tiles and 16-token tiles per workgroup; a K step is KT blocks of 32*WAVES
// elements, each block split over the WAVES wavefronts; DEPTH K steps are in flight in registers.
//
// GATED: the gated-MLP front end in one pass. The workgroup's first NT/2 tiles are rows of the gate
// weights, the other NT/2 the SAME rows of the up weights, and the epilogue writes
// round(round(silu(g)) * u) for g = round(alpha * x Wg^T), u = round(alpha * x Wu^T): the two
// linears and the SiLU-multiply of the reference's gated MLP (src/cuda/torch_bindings.cpp:703-723,
// src/cuda/inference_fusion.cuh:19-28) with the same rounding points, without the two
// activations' round trip through memory and without two of the three launches.
//
// FUSE: the residual-add + RMSNorm that surrounds a decode linear (ref src/cuda/inference_fusion.cuh:136-191:
// added = round(x + r), scale = rsqrt(mean(added^2) + eps), out = round(round(added * scale) * w)) moved into
// the linears on either side of it. The linear before the norm adds the residual to its rounded result in
// the epilogue and leaves per-workgroup sums of squares; the linear after it adds those partial sums in
// index order, forms the row scales and normalises the tokens on their way from registers to LDS (every
// workgroup stages all of x anyway). Rounding points are the reference's; the sum of squares is taken
// in a different (but fixed) order than a row kernel's, so the scale may differ in its last bit.
// (FUSE: 0 none, 1 the normalised input, 2 the residual epilogue; compile-time, because a branch in
// the loop keeps the compiler from counting the loads in flight and makes every wait a wait for all)
//
// EXACT: K is whole K steps. Then every load is a buffer load whose lane offset never changes (row and
// chunk) with the K position in the scalar offset, and a step past the end reads through an empty
// descriptor (zeros, no memory request), so a K step costs no address arithmetic and no masks on the
// vector ALU. A workgroup has one wavefront per SIMD and its phases run one after another, so at three
// and four token tiles those instructions were part of the step time ([28672, 8192] x 64 tokens: 203
// vector-ALU instructions per wavefront and step, of which 28 are matrix instructions).
template <int NT, int MT, int KT, bool GATED, int FUSE = 0, bool EXACT = false>
__global__ __launch_bounds__(WAVES * 64) void bgemv_stream_kernel(StreamParams p)
{
    constexpr bool NORMALISE = FUSE == 1, RESIDUAL = FUSE == 2 && !GATED;
    static_assert(!GATED || NT % 2 == 0, "gate and up tiles come in pairs");
    constexpr int HALF = GATED ? NT / 2 : NT; // distinct 16-row blocks of output rows
    constexpr int ROWS = HALF * 16, XROWS = MT * 16, CH = 4 * WAVES, BK = 32 * WAVES;
    constexpr int BLOCK_SLOTS = (NT * 16 + XROWS) * CH, STAGE_SLOTS = BLOCK_SLOTS * KT;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];
    u32x4_t *lds = reinterpret_cast<u32x4_t *>(lds_bytes);

    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int chunk = thread % CH, pass_row = thread / CH; // CH lanes per row segment, 16 rows per pass
    const int n0 = blockIdx.x * ROWS, m0 = blockIdx.y * XROWS;
    // this workgroup's K steps: [first_tile, first_tile + k_tiles) of all_tiles (all of them unless
    // the launch divides K over blockIdx.z; the launcher leaves no share empty)
    const int all_tiles = (p.k + BK * KT - 1) / (BK * KT);
    const int share = (all_tiles + int(gridDim.z) - 1) / int(gridDim.z);
    const int first_tile = int(blockIdx.z) * share;
    const int k_tiles = all_tiles - first_tile < share ? all_tiles - first_tile : share;

    unsigned a_off[NT], b_off[MT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        int row = n0 + (i % HALF) * 16 + pass_row;
        row = row < p.n ? row : p.n - 1;
        a_off[i] = unsigned(row - n0) * unsigned(p.lda);
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) {
        // Byte offset inside the token descriptor below; a row past the end gets an offset outside it,
        // which reads as zero without a memory request. (Reading an existing row in its place costs:
        // a line that is requested again while its first request is in flight holds up the vector
        // cache; [28672, 8192] at 33 tokens in a 48-token tile 106 us with every such lane on the
        // last row, 96 us on distinct rows, 84 us with 48 real tokens.)
        const int row = j * 16 + pass_row;
        b_off[j] = m0 + row < p.m ? unsigned(row) * unsigned(p.ldb) * 2u : 0x80000000u;
    }
    const unsigned short *a_base = p.w + size_t(n0) * p.lda;
    const unsigned short *a2_base = GATED ? p.w2 + size_t(n0) * p.lda : a_base;
    // (the launcher keeps 64 rows of x within 2 GB)
    const int x_rows = p.m - m0 < XROWS ? p.m - m0 : XROWS;
    const unsigned x_bytes = (unsigned(x_rows - 1) * unsigned(p.ldb) + unsigned(p.k)) * 2u;
    const __amdgpu_buffer_rsrc_t x_resource = make_resource(p.x + size_t(m0) * p.ldb, x_bytes);
    // EXACT: the weight rows of the workgroup (the launcher keeps them within 4 GB) and every lane's fixed offsets
    const int w_rows = p.n - n0 < ROWS ? p.n - n0 : ROWS;
    const unsigned w_bytes = (unsigned(w_rows - 1) * unsigned(p.lda) + unsigned(p.k)) * 2u;
    unsigned a_lane[NT], b_lane[MT];
#pragma unroll
    for (int i = 0; i < NT; ++i)
        a_lane[i] = (a_off[i] + unsigned(chunk) * 8u) * 2u;
#pragma unroll
    for (int j = 0; j < MT; ++j)
        b_lane[j] = b_off[j] + unsigned(chunk) * 16u; // (a row past the end stays outside the descriptor)
    // LDS slot of this thread's chunk inside a 16-row pass; passes are 256 slots apart
    const int store_slot = pass_row * CH + (chunk ^ pass_row);
    static_assert(CH == 16 || CH == 32, "XOR swizzle covers the low four chunk bits");

    // Loads are unconditional and the loop below has no data-dependent control flow, so the
    // compiler can count outstanding loads exactly and wait only for the older of the two tiles in
    // flight. A K position past the end (the K tail, or the padding tile of an odd tile count) is
    // read from the last valid chunk instead and zeroed by a mask when it is stored to LDS.
    u32x4_t a_reg[DEPTH][KT][NT], b_reg[DEPTH][KT][MT];
    u32x4_t norm_reg[DEPTH][NORMALISE ? KT : 1]; // the norm weights of a step's K positions
    // Workgroups start at different K tiles and wrap around: if all of them swept K in lock step
    // the chip would read one column block of every row at a time, a pattern strided by the row
    // pitch that lands on few HBM channels; staggering spreads the requests over all of them.
    const int start = int(blockIdx.x % unsigned(k_tiles));
    auto rotated = [&](int step) {
        int tile = (step < k_tiles ? step : k_tiles - 1) + start;
        return first_tile + (tile < k_tiles ? tile : tile - k_tiles);
    };
    // W is read exactly once, so its loads are non-temporal: they bypass the cache allocation that
    // a 470 MB stream would otherwise keep evicting (measured: 5.7 -> 6.3 TB/s); x is re-read by
    // every workgroup and is loaded normally.
    auto fetch = [&](int step, u32x4_t(&a)[KT][NT], u32x4_t(&b)[KT][MT], u32x4_t(&norm)[NORMALISE ? KT : 1]) {
        if constexpr (EXACT) {
            const bool alive = step < k_tiles;
            const __amdgpu_buffer_rsrc_t gate_rows = make_resource(a_base, alive ? w_bytes : 0u);
            const __amdgpu_buffer_rsrc_t up_rows = make_resource(a2_base, alive ? w_bytes : 0u);
            const __amdgpu_buffer_rsrc_t token_rows = make_resource(p.x + size_t(m0) * p.ldb, alive ? x_bytes : 0u);
            const int step_bytes = rotated(step) * (BK * KT * 2);
#pragma unroll
            for (int t = 0; t < KT; ++t) {
#pragma unroll
                for (int i = 0; i < NT; ++i) // (cache policy 2: non-temporal, as below)
                    a[t][i] = __builtin_amdgcn_raw_buffer_load_b128(i < HALF ? gate_rows : up_rows, int(a_lane[i]),
                                                                    step_bytes + t * BK * 2, 2);
#pragma unroll
                for (int j = 0; j < MT; ++j)
                    b[t][j] = __builtin_amdgcn_raw_buffer_load_b128(token_rows, int(b_lane[j]), step_bytes + t * BK * 2, 0);
                if constexpr (NORMALISE)
                    norm[t] = *reinterpret_cast<const u32x4_t *>(
                        p.norm_weight + (alive ? rotated(step) * (BK * KT) + t * BK + chunk * 8 : 0));
            }
            return;
        }
        // padding steps past the end (their data is masked away) all read one cached line
        const unsigned live = step < k_tiles ? 0xffffffffu : 0u;
        const int tile_k = rotated(step) * (BK * KT) + chunk * 8;
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            int k0 = tile_k + t * BK;
            k0 = k0 < p.k ? k0 : p.k - 8;
            k0 &= int(live);
#pragma unroll
            for (int i = 0; i < NT; ++i)
                a[t][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(
                    (i < HALF ? a_base : a2_base) + k0 + (a_off[i] & live)));
#pragma unroll
            for (int j = 0; j < MT; ++j)
                b[t][j] = __builtin_amdgcn_raw_buffer_load_b128(x_resource, int((b_off[j] & live) + unsigned(k0) * 2u), 0, 0);
            if constexpr (NORMALISE)
                norm[t] = *reinterpret_cast<const u32x4_t *>(p.norm_weight + k0);
        }
    };
    float scale[MT] = {}; // NORMALISE: the row scales of this thread's tokens
    auto normalised = [&](u32x4_t values, float row_scale, const u32x4_t &weights) {
        u32x4_t result;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const unsigned rounded = round_pack_bf16x2(__fmul_rn(__uint_as_float(values[e] << 16), row_scale),
                                                       __fmul_rn(__uint_as_float(values[e] & 0xffff0000u), row_scale));
            result[e] = round_pack_bf16x2(
                __fmul_rn(__uint_as_float(rounded << 16), __uint_as_float(weights[e] << 16)),
                __fmul_rn(__uint_as_float(rounded & 0xffff0000u), __uint_as_float(weights[e] & 0xffff0000u)));
        }
        return result;
    };
    auto stash = [&](int stage, int step, const u32x4_t(&a)[KT][NT], const u32x4_t(&b)[KT][MT],
                     const u32x4_t(&norm)[NORMALISE ? KT : 1]) {
        const int tile_k = rotated(step) * (BK * KT) + chunk * 8;
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            // (EXACT: what lies past the end was read as zeros)
            const unsigned mask = EXACT || (step < k_tiles && tile_k + t * BK < p.k) ? 0xffffffffu : 0u;
            u32x4_t *base = lds + stage * STAGE_SLOTS + t * BLOCK_SLOTS + store_slot;
#pragma unroll
            for (int i = 0; i < NT; ++i)
                base[i * 16 * CH] = a[t][i] & mask;
#pragma unroll
            for (int j = 0; j < MT; ++j) {
                u32x4_t tokens = b[t][j];
                if constexpr (NORMALISE)
                    tokens = normalised(tokens, scale[j], norm[t]);
                base[(NT + j) * 16 * CH] = tokens & mask;
            }
        }
    };

    // MFMA 16x16x32 operand positions: lane -> row lane%16, 8 K values at (wave*4 + lane/16)*8
    const int frag_row = lane % 16;
    const int frag_slot = frag_row * CH + ((wave * 4 + lane / 16) ^ frag_row);
    f32x4_t acc[NT][MT];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
            acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](int stage) {
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const u32x4_t *base = lds + stage * STAGE_SLOTS + t * BLOCK_SLOTS + frag_slot;
            bf16x8_t b_frag[MT];
#pragma unroll
            for (int j = 0; j < MT; ++j)
                b_frag[j] = __builtin_bit_cast(bf16x8_t, base[(NT + j) * 16 * CH]);
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                bf16x8_t a_frag = __builtin_bit_cast(bf16x8_t, base[i * 16 * CH]);
#pragma unroll
                for (int j = 0; j < MT; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_frag, b_frag[j],
                                                                        acc[i][j], 0, 0, 0);
            }
        }
    };

    // sched_barrier(0) pins the phase order (also between the prologue fetches): if the scheduler
    // interleaves loads of different tiles, the wait before a store to LDS degenerates to "all
    // loads" and only one tile stays in flight.
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        fetch(d, a_reg[d], b_reg[d], norm_reg[d]);
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (NORMALISE) {
        {
            // Row scales, with the first weight loads already on their way: the workgroup's tokens go
            // round its threads, PARTS threads per token, each adding a contiguous range of the partial
            // sums in index order; then the PARTS ranges in order. Fixed for a given count.
            constexpr int PARTS = WAVES * 64 / XROWS;
            float *table = reinterpret_cast<float *>(lds_bytes);
            const int token = thread % XROWS, part = thread / XROWS;
            const int row = m0 + token < p.m ? m0 + token : p.m - 1;
            const int per = (p.ssq_count + PARTS - 1) / PARTS;
            const int last = (part + 1) * per < p.ssq_count ? (part + 1) * per : p.ssq_count;
            float sum = 0.f;
            for (int q = part * per; q < last; ++q)
                sum = __fadd_rn(sum, p.ssq_in[size_t(q) * p.ssq_ld + row]);
            table[part * XROWS + token] = sum;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < MT; ++j) {
                float total = table[j * 16 + pass_row];
                for (int q = 1; q < PARTS; ++q)
                    total = __fadd_rn(total, table[q * XROWS + j * 16 + pass_row]);
                scale[j] = rsqrtf(__fadd_rn(total / float(p.k), p.epsilon));
            }
            __syncthreads(); // the table lies where the first stage is stashed
        }
    }
    int stage = 0;
    for (int step = 0; step < k_tiles; step += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            __builtin_amdgcn_sched_barrier(0);
            stash(stage, step + d, a_reg[d], b_reg[d], norm_reg[d]);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + d + DEPTH, a_reg[d], b_reg[d], norm_reg[d]);
            __builtin_amdgcn_sched_barrier(0);
            multiply(stage);
            stage ^= 1;
        }
    }

    // ---- combine the K partitions of the wavefronts: each parks its partial sums in a region of
    // its own, and after one barrier tile t is summed in wavefront order 0, 1, 2, 3 by wavefront t % 4.
    // The sums of more than 36 tiles do not fit the LDS at once: they go in two passes of half the tiles.
    // (the launcher sizes the dynamic LDS for the larger of the two uses)
    constexpr int PASSES = stream_combine_passes(NT, MT), PASS_TILES = (NT * MT + PASSES - 1) / PASSES;
    static_assert(PASSES == 1 || (!GATED && FUSE == 0), "passes of the plain form");
    f32x4_t *combine = reinterpret_cast<f32x4_t *>(lds_bytes);
    auto park = [&](int pass) {
        __syncthreads(); // (every wavefront is done with the stages, or with the previous pass)
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int j = 0; j < MT; ++j)
                if ((i * MT + j) / PASS_TILES == pass)
                    combine[(wave * PASS_TILES + (i * MT + j) % PASS_TILES) * 64 + lane] = acc[i][j];
        __syncthreads();
    };
    // ---- epilogue: wavefront w writes tiles w, w+4, ...; register r of lane l is feature
    // 4*(l/16) + r and token l%16 inside the 16x16 tile
    auto summed = [&](int index) { // (of the pass that is parked)
        f32x4_t sum = combine[(index % PASS_TILES) * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            sum = sum + combine[(w * PASS_TILES + index % PASS_TILES) * 64 + lane];
        return sum;
    };
    // ---- K divided over several workgroups: every workgroup parks its sums in its own FP32 plane;
    // the one that arrives last (a counter per output tile) adds the planes in index order, so the
    // result does not depend on which workgroup that was, and writes the output.
    const bool divided = !GATED && gridDim.z > 1;
    // a plane holds, per output tile of a workgroup, 64 lanes x 4 sums in the accumulator's own
    // layout: whole wavefronts store and load 1 KB runs
    constexpr unsigned TILE_BYTES = 64 * 16, GROUP_BYTES = unsigned(HALF * MT) * TILE_BYTES;
    const size_t plane_bytes = size_t(gridDim.x) * gridDim.y * GROUP_BYTES;
    const char *group = reinterpret_cast<const char *>(p.partials) +
                        (size_t(blockIdx.y) * gridDim.x + blockIdx.x) * GROUP_BYTES;
    if (divided) {
        const __amdgpu_buffer_rsrc_t mine = make_resource(group + blockIdx.z * plane_bytes, GROUP_BYTES);
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            park(pass);
#pragma unroll
            for (int index = pass * PASS_TILES; index < (pass + 1) * PASS_TILES && index < NT * MT; ++index) {
                if (index % WAVES != wave)
                    continue;
                const f32x4_t sum = summed(index);
                store_device_scope(mine, unsigned(index) * TILE_BYTES + unsigned(lane) * 16, sum);
            }
        }
        // The planes are written and read with device-scope accesses, which go to the point where
        // all XCDs agree instead of staying in one XCD's L2, so no cache has to be written back or
        // invalidated (a device-scope fence per workgroup was measured at +20 us on a 70 us
        // launch). Order, written out: every wavefront waits until its own plane stores have been
        // acknowledged at device scope (vmcnt counts a store until its acknowledgement returns),
        // then the barrier collects all four wavefronts, and only then does thread 0 count the
        // arrival; a barrier alone promises nothing about global stores still in flight. On the
        // reading side the last arriver's plane loads are issued after the atomic has returned
        // its value (the branch on it below depends on the returned value) and are device-scope
        // too, so they cannot be served from a stale XCD-local line.
        wait_loads<0>();
        __syncthreads(); // (also: every wavefront is done with `combine`)
        unsigned *flag = reinterpret_cast<unsigned *>(lds_bytes);
        if (thread == 0) {
            unsigned *counter = p.arrivals + size_t(blockIdx.y) * gridDim.x + blockIdx.x;
            const unsigned before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned last = before + 1 == gridDim.z ? 1u : 0u;
            if (last) // nobody else touches it any more: ready for the next launch
                __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = last;
        }
        __syncthreads();
        if (*flag == 0)
            return;
    }
    // (residual epilogue: per tile and lane, the squares of the four outputs the lane wrote; behind
    // the region the wavefronts' sums were parked in, which the launcher sizes for)
    float *square_table = reinterpret_cast<float *>(lds_bytes + size_t(WAVES) * NT * MT * 64 * 16);
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
    if (!divided) // (a divided product parked its sums above and reads the planes here)
        park(pass);
#pragma unroll
    for (int index = pass * PASS_TILES; index < (pass + 1) * PASS_TILES && index < HALF * MT; ++index) {
        if (index % WAVES != wave)
            continue;
        const int i = index / MT, j = index % MT;
        const int m = m0 + j * 16 + lane % 16;
        const int n = n0 + i * 16 + (lane / 16) * 4;
        f32x4_t sum;
        if (divided) { // (before the bounds check: the loads are whole-wavefront)
            sum = f32x4_t{0.f, 0.f, 0.f, 0.f};
            for (unsigned z = 0; z < gridDim.z; ++z)
                sum = sum + load_device_scope(make_resource(group + z * plane_bytes, GROUP_BYTES),
                                              unsigned(index) * TILE_BYTES + unsigned(lane) * 16);
        } else {
            sum = summed(index);
        }
        if constexpr (RESIDUAL) {
            {
                // added = round(round(alpha * product) + residual), and this lane's share of the sums of
                // squares of the rows of `added` (zero where the tile leaves the matrix)
                float added[4] = {0.f, 0.f, 0.f, 0.f};
                if (m < p.m && n < p.n) {
                    const unsigned short *carried = p.residual + size_t(m) * p.ld_residual + n;
                    unsigned short *out = p.y + size_t(m) * p.ldc + n;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < p.n) {
                            const float product = bf16_bits_to_float(float_to_bf16_bits(p.alpha * sum[e]));
                            const unsigned short bits = float_to_bf16_bits(__fadd_rn(product, bf16_bits_to_float(carried[e])));
                            out[e] = bits;
                            added[e] = bf16_bits_to_float(bits);
                        }
                }
                float squares = __fmul_rn(added[0], added[0]);
#pragma unroll
                for (int e = 1; e < 4; ++e)
                    squares = __fadd_rn(squares, __fmul_rn(added[e], added[e]));
                square_table[index * 64 + lane] = squares;
                continue;
            }
        }
        if (m >= p.m || n >= p.n)
            continue;
        float v[4] = {sum[0], sum[1], sum[2], sum[3]};
        unsigned short *out = p.y + size_t(m) * p.ldc + n;
        if constexpr (GATED) {
            const f32x4_t raised = summed((i + HALF) * MT + j);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float g = bf16_bits_to_float(float_to_bf16_bits(p.alpha * v[e]));
                const float u = bf16_bits_to_float(float_to_bf16_bits(p.alpha * raised[e]));
                const float activated = bf16_bits_to_float(float_to_bf16_bits(g / (1.f + expf(-g))));
                v[e] = __fmul_rn(activated, u);
            }
            if (n + 3 < p.n && p.vector_store) {
                *reinterpret_cast<u32x2_t *>(out) = u32x2_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < p.n)
                        out[e] = float_to_bf16_bits(v[e]);
            }
            continue;
        }
        const unsigned short *source = p.z + size_t(m) * p.ldz + n;
        if (n + 3 < p.n && p.vector_store) {
            if (p.beta != 0.f) {
                u32x2_t old = *reinterpret_cast<const u32x2_t *>(source);
                v[0] = fmaf(p.beta, __uint_as_float(old[0] << 16), p.alpha * v[0]);
                v[1] = fmaf(p.beta, __uint_as_float(old[0] & 0xffff0000u), p.alpha * v[1]);
                v[2] = fmaf(p.beta, __uint_as_float(old[1] << 16), p.alpha * v[2]);
                v[3] = fmaf(p.beta, __uint_as_float(old[1] & 0xffff0000u), p.alpha * v[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    v[e] *= p.alpha;
            }
            u32x2_t packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2_t *>(out) = packed;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e >= p.n)
                    break;
                float value = p.alpha * v[e];
                if (p.beta != 0.f)
                    value = fmaf(p.beta, bf16_bits_to_float(source[e]), value);
                out[e] = float_to_bf16_bits(value);
            }
        }
    }
    } // passes
    if constexpr (RESIDUAL) {
        {
            // one thread per token adds the table's entries of that token in a fixed order: feature
            // tiles ascending, inside a tile the four lane groups (features 0-3, 4-7, ...) ascending
            __syncthreads();
            if (thread < XROWS && m0 + thread < p.m) {
                float total = 0.f;
#pragma unroll
                for (int i = 0; i < HALF; ++i)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        total = __fadd_rn(total, square_table[(i * MT + thread / 16) * 64 + g * 16 + thread % 16]);
                p.ssq_out[size_t(blockIdx.x) * p.ssq_ld_out + m0 + thread] = total;
            }
        }
    }
}

template <int NT, int MT, int KT, bool GATED = false, int FUSE = 0>
hipError_t launch_one(hipStream_t stream, const StreamParams &p, int shares = 1)
{
    constexpr size_t stage_bytes = size_t(2) * KT * (NT + MT) * 16 * (64 * WAVES);
    // partial sums at the end (residual epilogue: and the table of squares behind them)
    constexpr size_t parked_bytes = size_t(WAVES) * ((NT * MT + stream_combine_passes(NT, MT) - 1) / stream_combine_passes(NT, MT)) * 64 * 16 +
                                    (FUSE == 2 && !GATED ? size_t(NT) * MT * 64 * 4 : 0);
    constexpr size_t lds_bytes = stage_bytes > parked_bytes ? stage_bytes : parked_bytes;
    // combined limits: the tiles in flight fit the register file, a stage pair fits the LDS
    if constexpr (NT * KT > 8 || lds_bytes > 160 * 1024) {
        return hipErrorInvalidValue;
    } else {
        // whole K steps and a workgroup's weight rows within one 4 GB descriptor: the variant without
        // address arithmetic and masks in its K loop
        const bool exact = p.k % (32 * WAVES * KT) == 0 && (size_t(NT * 16 - 1) * size_t(p.lda) + size_t(p.k)) * 2 < (size_t(1) << 32);
        auto kernel = exact ? bgemv_stream_kernel<NT, MT, KT, GATED, FUSE, true> : bgemv_stream_kernel<NT, MT, KT, GATED, FUSE, false>;
        static LdsLimitFlags limits[2]; // (one per instantiation)
        const hipError_t status = raise_lds_limit(limits[exact ? 1 : 0], reinterpret_cast<const void *>(kernel), lds_bytes);
        if (status != hipSuccess)
            return status;
        constexpr int rows = (GATED ? NT / 2 : NT) * 16;
        // every share of a divided K holds at least one K step
        const int all_tiles = (p.k + 32 * WAVES * KT - 1) / (32 * WAVES * KT);
        const int share = (all_tiles + shares - 1) / shares;
        shares = (all_tiles + share - 1) / share;
        dim3 grid(unsigned((p.n + rows - 1) / rows), unsigned((p.m + MT * 16 - 1) / (MT * 16)), unsigned(shares));
        if (shares > 1 && (GATED || !p.partials || !p.arrivals || size_t(grid.x) * grid.y > STREAM_ARRIVAL_SLOTS))
            return hipErrorInvalidValue;
        kernel<<<grid, WAVES * 64, lds_bytes, stream>>>(p);
        return launch_status();
    }
}

template <int MT, int KT, int FUSE>
hipError_t launch_rows(hipStream_t stream, int row_tiles, const StreamParams &p, int shares)
{
    switch (row_tiles) {
    case 1: return launch_one<1, MT, KT, false, FUSE>(stream, p, shares);
    case 2: return launch_one<2, MT, KT, false, FUSE>(stream, p, shares);
    case 3: return launch_one<3, MT, KT, false, FUSE>(stream, p, shares);
    case 4: return launch_one<4, MT, KT, false, FUSE>(stream, p, shares);
    case 5: return launch_one<5, MT, KT, false, FUSE>(stream, p, shares);
    case 6: return launch_one<6, MT, KT, false, FUSE>(stream, p, shares);
    case 7: return launch_one<7, MT, KT, false, FUSE>(stream, p, shares);
    case 8: return launch_one<8, MT, KT, false, FUSE>(stream, p, shares);
    default: return hipErrorInvalidValue;
    }
}

template <int KT, int FUSE = 0>
hipError_t launch_tokens(hipStream_t stream, int row_tiles, int token_tiles, const StreamParams &p, int shares)
{
    switch (token_tiles) {
    case 1: return launch_rows<1, KT, FUSE>(stream, row_tiles, p, shares);
    case 2: return launch_rows<2, KT, FUSE>(stream, row_tiles, p, shares);
    case 3: // (33 to 48 tokens; the fused forms keep to 1, 2 and 4 tiles)
        if constexpr (FUSE == 0)
            return launch_rows<3, KT, FUSE>(stream, row_tiles, p, shares);
        else
            return hipErrorInvalidValue;
    case 4: return launch_rows<4, KT, FUSE>(stream, row_tiles, p, shares);
    default: return hipErrorInvalidValue;
    }
}
} // namespace

// One per translation unit. depth_log2: log2 of the K blocks per step.
hipError_t stream_plain_single(hipStream_t stream, int row_tiles, int token_tiles, const StreamParams &p, int shares);
hipError_t stream_plain_deep(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, const StreamParams &p, int shares);
hipError_t stream_normalising(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, const StreamParams &p, int shares);
hipError_t stream_residual(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, const StreamParams &p, int shares);
hipError_t stream_gated(hipStream_t stream, int pair_tiles, int token_tiles, bool normalising, const StreamParams &p);
// five to eight token tiles (65 to 128 tokens): the plain form with one K block per step
hipError_t stream_many_tokens(hipStream_t stream, int row_tiles, int token_tiles, const StreamParams &p, int shares);
} // namespace camblas_hip
