// GEMM planner: a pure host function from (dtype, layout, shape, leading dimensions, alignment)
// to a kernel family, a tile variant and a split-K factor. It replaces the reference's run-time
// plan cache and timing autotune (src/cuda/backend.cu:553-784) with a closed-form decision: no
// device access, no stream synchronisation, identical answers for identical inputs, so a shape
// planned during warm-up replays unchanged under graph capture.
#include "common.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace camblas_hip
{
namespace
{
int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Work partition for the bandwidth-bound decode tiles: enough workgroups to keep about four per
// compute unit in flight, never fewer than four K tiles per partition.
int decode_split(int tiles, int k_tiles, int compute_units)
{
    int wanted = ceil_div(4 * compute_units, std::max(1, tiles));
    int limit = std::max(1, k_tiles / 4);
    return std::max(1, std::min(wanted, limit));
}

// Weight rows per workgroup (in units of 16) for the streaming decode kernel: the choice that
// spreads the row tiles most evenly over the compute units; ties go to the larger block, which
// keeps more bytes in flight per workgroup.
int stream_row_tiles(int outputs, int compute_units)
{
    const int tiles = ceil_div(outputs, 16);
    int best = 1;
    double best_score = -1;
    for (int candidate = 1; candidate <= 8; ++candidate) {
        int groups = ceil_div(tiles, candidate);
        double busiest = double(ceil_div(groups, compute_units)) * candidate;
        double score = (double(tiles) / compute_units) / busiest;
        if (groups < compute_units)
            score = std::min(score, double(groups) / compute_units);
        if (score >= best_score - 1e-9) {
            best_score = score;
            best = candidate;
        }
    }
    return best;
}

// Weight rows per workgroup (in units of 16) for the FP8 streaming kernel. Several of its
// workgroups can share a compute unit, so the time follows the busiest compute unit's share of the
// traffic: workgroups per compute unit times the bytes one workgroup moves, the weight rows from
// HBM plus the token tiles, which every workgroup re-reads through L2 (counted at half weight).
int fp8_stream_row_tiles(int outputs, int token_tiles, int compute_units, int limit)
{
    const int tiles = ceil_div(outputs, 16);
    int best = 1;
    double best_cost = 1e300;
    for (int candidate = 1; candidate <= limit; ++candidate) {
        int groups = ceil_div(tiles, candidate);
        double cost = double(ceil_div(groups, compute_units)) * (candidate + 0.5 * token_tiles);
        if (cost <= best_cost + 1e-9) {
            best_cost = cost;
            best = candidate;
        }
    }
    return best;
}

// 128-element K blocks per step of the streaming kernel, as a power of two. Workgroups with few
// weight rows (projections with few outputs) take two blocks per step so that enough bytes are in
// flight per compute unit; measured on 8192- and 10240-row projections, two blocks beat one by
// 10-20 % up to three row tiles, and four blocks or more lose again.
// 33..64 tokens on a projection too narrow for one workgroup per compute unit: the number of workgroups
// K is divided over so that each takes 64 to 128 weight rows, if K is long enough for that many shares
// (0: none is)
int narrow_stream_shares(int outputs, int k, int compute_units)
{
    for (const int shares : {2, 4}) {
        const int row_tiles = ceil_div(shares * ceil_div(outputs, 16), compute_units);
        if (row_tiles >= 4 && row_tiles <= 8 && k >= (shares == 2 ? 8192 : 14336))
            return shares;
    }
    return 0;
}

int stream_depth_log2(int row_tiles, int token_tiles, int k)
{
    return row_tiles <= 3 && (row_tiles + token_tiles) * 2 <= 16 && k >= 2048 ? 1 : 0;
}

// Fraction of the machine a tiling keeps busy: useful tiles over whole rounds of resident
// workgroups, times the fraction of each tile that is inside the matrix.
double occupancy_score(int n, int m, int block_n, int block_m, int resident, int compute_units)
{
    double tiles = double(ceil_div(n, block_n)) * ceil_div(m, block_m);
    double slots = double(resident) * compute_units;
    double rounds = std::ceil(tiles / slots);
    double fill = (double(n) * m) / (tiles * block_n * block_m);
    return tiles / (rounds * slots) * fill;
}

// Estimated microseconds of one launch of a direct-to-LDS BF16 tile over `outputs` weight rows with
// K divided over `shares` workgroups per tile, fitted to sweeps of six tiles and 1..8 shares over
// ten projection shapes at 65..1536 tokens (the choice by this estimate is within 2 % of the best
// measured kernel in the geometric mean, 20 % at worst). The longer of two terms: rounds of
// workgroups times steps times the tile's time per 64-deep step; and the weights streamed at what
// the workgroups in flight can draw (each keeps the stages it is not reading in flight for 2.6 us,
// together at most 5.2 TB/s; a partly filled last round draws less). A divided K adds the second
// kernel and the traffic of the FP32 planes.
struct DmaPrice {
    int variant;
    double step_us, kilobytes_in_flight;
};
const DmaPrice dma_prices[] = {{5, 0.557, 64}, {9, 0.849, 96}, {6, 1.632, 64},
                               {8, 0.943, 96}, {10, 1.878, 72}, {11, 1.281, 56}};
double dma_launch_us(const DmaPrice &price, int outputs, int tokens, int k, int shares, int compute_units)
{
    const TnVariant &v = dma_variant(price.variant);
    const double workgroups = double(ceil_div(outputs, v.block_n)) * ceil_div(tokens, v.block_m) * shares;
    const double rounds = std::ceil(workgroups / compute_units);
    const double steps = ceil_div(ceil_div(k, 64), shares);
    const double bytes_per_us =
        std::min(5.183e6, std::min(workgroups, double(compute_units)) * price.kilobytes_in_flight * 1024 / 2.601);
    double stream_us = double(outputs) * k * 2 / bytes_per_us;
    if (workgroups > compute_units)
        stream_us *= rounds * compute_units / workgroups;
    double us = 0.8 + std::max(rounds * steps * price.step_us, stream_us);
    if (shares > 1)
        us += 1.553 + 2.0 * shares * double(tokens) * outputs * 4 / 4.517e6;
    return us;
}
} // namespace

Plan make_plan(int dtype, int algorithm, bool trans_a, bool trans_b, int m, int n, int k, int lda,
               int ldb, int ldc, bool aligned16, int compute_units)
{
        Plan plan;
    if (compute_units < 1)
        compute_units = 256;
    if (dtype == 0) {
        // FP32: the single-vector shortcut exists only under AUTO (ref: src/cuda/backend.cu:810-815)
        if (algorithm == CAMBLAS_CUDA_AUTO && n == 1 && trans_a && !trans_b && m >= 1024 &&
            k >= 4096 && k % 4 == 0 && lda % 4 == 0 && aligned16) {
            plan.family = FAMILY_GEMV_F32;
            plan.counter = 0;
            return plan;
        }
        // matrix-core tiles unless the product is a sliver: 128 x 128 per workgroup once that gives
        // every compute unit two or more workgroups, else 128 x 64 (measured: 2048^3 189 vs 202 us,
        // 4096^3 1420 vs 1287 us; the 64 x 64 vector-ALU tiles are 2-3 times slower at every size)
        if (m >= 32 && n >= 32 && k >= 16) {
            plan.family = FAMILY_MFMA_F32;
            plan.kernel = double(ceil_div(m, 128)) * ceil_div(n, 128) >= 2.0 * compute_units ? 0 : 1;
        } else if (algorithm != CAMBLAS_CUDA_CLASSICAL && m >= 256 && k >= 512) {
            // a handful of columns against a large A (a linear layer at 2 to 31 tokens): the
            // matrix-core tiles, mostly empty, still beat the vector-ALU kernel several times over
            plan.family = FAMILY_MFMA_F32;
            plan.kernel = 1;
        } else {
            plan.family = FAMILY_GENERIC;
        }
        // Few tiles and a long K (up to a few hundred tokens against a weight matrix): K divided
        // over workgroups, about two per compute unit, FP32 planes summed in share order
        // ([8192, 8192] x 16 tokens: 980 us on the vector-ALU kernel, 420 us at 32 tokens undivided).
        if (plan.family == FAMILY_MFMA_F32 && plan.kernel == 1 && algorithm != CAMBLAS_CUDA_CLASSICAL && k >= 512) {
            // (up to 32 columns: tiles of 128 x 32, kernel 2, and four workgroups per compute unit:
            // [8192, 8192] x 16 tokens 100 us on the 64-column tiles)
            const bool narrow = n <= 32;
            const int tiles = ceil_div(m, 128) * ceil_div(n, narrow ? 32 : 64);
            const int counts[] = {32, 16, 8, 4, 2};
            for (const int shares : counts)
                if (tiles * shares <= (narrow ? 4 : 2) * compute_units && k % shares == 0 && k / shares >= 256 &&
                    double(shares) * m * n * 4 <= double(1 << 28)) {
                    plan.split_k = shares;
                    plan.kernel = narrow ? 2 : 1;
                    break;
                }
        }
        plan.counter = algorithm == CAMBLAS_CUDA_LT || algorithm == CAMBLAS_CUDA_AUTO ? 4 : 0;
        return plan;
    }
    if (dtype == 2) {
        const int limit = 1 << 23;
        bool matrix_path = algorithm != CAMBLAS_CUDA_CLASSICAL && trans_a && !trans_b &&
                           k % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && aligned16 && lda < limit &&
                           ldb < limit;
        // x @ W with a row-major W ('N','N') and up to 512 tokens: one pass over W per 256 tokens with
        // its outputs contiguous (the layout-agnostic tiles below re-read operands through LDS in
        // 32-deep steps and are 3 to 4 times slower at these sizes; below 32 tokens the product went
        // to the vector-ALU kernel: [8192, 28672] x 16 tokens 1660 us). K divided over workgroups
        // when the 128-output tiles leave compute units idle.
        if (algorithm != CAMBLAS_CUDA_CLASSICAL && !trans_a && !trans_b && n <= 512 && k % 64 == 0 && k >= 64 &&
            m % 4 == 0 && lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 && aligned16 &&
            double(k) * lda * 2 < 4294967296.0 && (256.0 * ldb + k) * 2 < 4294967296.0) {
            plan.family = FAMILY_NN;
            plan.counter = 4;
            const int tiles = ceil_div(m, 128) * ceil_div(n, 256);
            const int resident = n <= 64 ? 2 : 1; // workgroups a compute unit holds (LDS of three stages)
            const int counts[] = {8, 6, 4, 3, 2};
            for (const int shares : counts)
                if (tiles * shares <= resident * compute_units && k / shares >= 512) {
                    plan.split_k = shares;
                    break;
                }
            return plan;
        }
        // x @ W with a row-major W and many tokens: the four-wavefront 256 x 256 tile that copies W into
        // LDS as it lies and transposes on the way to the registers, where its tiles fill at least nine
        // tenths of the rounds of workgroups they make; other shapes are better served by a transposed
        // copy of W and the tile the 'T','N' planner picks for it (measured, this kernel against the copy
        // route: 8192^3 757 against 799 us, 8192 x 4096 x 4096 200 against 217, 4096^3 125 against 129;
        // 4096 x 8192 x 10240, 2.5 rounds, 511 against 503 with the 320-row tile).
        if (algorithm != CAMBLAS_CUDA_CLASSICAL && !trans_a && !trans_b && k % 128 == 0 && k >= 256 && m % 4 == 0 &&
            lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 && aligned16 && double(k) * lda * 2 < 4294967296.0 &&
            (256.0 * ldb + k) * 2 < 4294967296.0) {
            const int tiles = ceil_div(m, 256) * ceil_div(n, 256);
            if (tiles * 10 >= ceil_div(tiles, compute_units) * compute_units * 9) {
                plan.family = FAMILY_DMA;
                plan.kernel = 20;
                plan.counter = 4;
                return plan;
            }
        }
        if (!matrix_path) {
            // the other layouts (and 'T','N' operands the K-contiguous kernels cannot take): the
            // layout-agnostic matrix-core kernel unless the product is a sliver, tiles chosen as for
            // FP32 (the reference sends every transpose pair to tensor-core GEMMs)
            if (algorithm != CAMBLAS_CUDA_CLASSICAL && m >= 32 && n >= 32 && k >= 16) {
                plan.family = FAMILY_MFMA_BF16;
                plan.kernel = double(ceil_div(m, 128)) * ceil_div(n, 128) >= 2.0 * compute_units ? 0 : 1;
                plan.counter = 4;
                return plan;
            }
            plan.family = FAMILY_GENERIC;
            plan.counter = 0;
            return plan;
        }
        plan.family = FAMILY_MFMA_TN;
        plan.counter = 4;
        const int outputs = m, tokens = n;
        // narrow projection: its 128-row tiles occupy at most half of the compute units
        const bool narrow = ceil_div(outputs, 128) * 2 <= compute_units;
        if (tokens <= 32 || (tokens <= 128 && !narrow)) {
            // decode: bandwidth-bound on W, one streaming pass, no split-K
            plan.family = FAMILY_STREAM;
            plan.kernel = undivided_stream_kernel(outputs, tokens, k, compute_units);
            plan.split_k = 1;
            // Few output rows and a long K (a down projection): one workgroup per compute unit
            // would own 32-48 weight rows and re-read as many token rows through L2. Two
            // workgroups per output tile, each with half of K and twice the rows, keep the same
            // number of workgroups with half the token traffic (measured at 32 tokens:
            // [8192, 28672] 77 against 85-90 us, [10240, 8192] 30.5 against 33, [8192, 8192] even;
            // up to 16 tokens the token rows are half as many and only K beyond 12288 gains).
            const int row_tiles = plan.kernel / 10 % 10, token_tiles = plan.kernel % 10;
            const int wider = std::min(8, ceil_div(2 * ceil_div(outputs, 16), compute_units));
            const bool long_enough = token_tiles >= 2 ? k >= 8192 : k >= 12288;
            if (row_tiles <= 3 && long_enough && wider > row_tiles && wider + token_tiles <= 16) {
                plan.kernel = 10 * wider + token_tiles;
                plan.split_k = 2;
            }
        } else if (tokens <= 64 && k >= 8192 &&
                   ceil_div(2 * ceil_div(outputs, 16), compute_units) >= 5) {
            // 33..64 tokens on a projection of 10240 to 16384 rows: the streaming kernel with K
            // divided over two workgroups per tile and 80 to 128 rows each (one workgroup per
            // compute unit) beats the register-staged tiles below by 15-25 % from 12288 rows on
            // (measured: [12288, 8192] 46-48 vs 55-58 us, [16384, 8192] 58-59 vs 71-74,
            // [12288, 16384] 79-81 vs 100-106; [10240, 8192] 32 vs 41 at 33 tokens, 34.5 at 64)
            plan.family = FAMILY_STREAM;
            plan.kernel = 10 * std::min(8, ceil_div(2 * ceil_div(outputs, 16), compute_units)) + (tokens <= 48 ? 3 : 4);
            plan.split_k = 2;
        } else if (const int shares = narrow_stream_shares(outputs, k, compute_units); tokens <= 64 && shares) {
            // 33..64 tokens on a narrow projection with a long K: the streaming kernel again, K divided over
            // two or four workgroups of 64 to 128 rows each, about one workgroup per compute unit (the
            // token rows a workgroup re-reads through L2 are what costs here, and that traffic falls
            // with the rows per workgroup). Measured against the register-staged tiles of the branch
            // below at 33 / 48 / 64 tokens: [8192, 8192] 27 / 28 / 31 against 32 / 33 / 35 us,
            // [8192, 28672] 78 / 83 / 95 against 88 / 92 / 97, [4096, 14336] 26 / 27 / 31 against 30 / 31 / 32.
            plan.family = FAMILY_STREAM;
            plan.kernel = 10 * ceil_div(shares * ceil_div(outputs, 16), compute_units) + (tokens <= 48 ? 3 : 4);
            plan.split_k = shares;
        } else if (tokens <= 64) {
            // 33..64 tokens on a narrow projection: the undivided streaming kernel would have 32-48
            // weight rows per workgroup and re-read as many token rows through L2; 128 x 64
            // register-staged tiles with K divided over up to 2.5 workgroups per compute unit are
            // 15-30 % faster (measured: [8192, 28672] 89-98 vs 118-137 us, [8192, 8192] 29-32 vs 36-40 us)
            plan.kernel = 3;
            const int tiles = ceil_div(outputs, 128);
            plan.split_k = 1;
            while (plan.split_k < 16 && tiles * plan.split_k * 2 * 2 <= 5 * compute_units &&
                   k / (plan.split_k * 2) >= 512)
                plan.split_k *= 2;
        } else if (tokens <= 1536 && k % 64 == 0 && k >= 512 && outputs % 4 == 0 && ldc % 4 == 0 &&
                   lda < (1 << 22) && ldb < (1 << 22)) {
            // 65..1536 tokens: the direct-to-LDS tile, the number of workgroups K is divided over
            // and, where a tile would end in a partly filled round, the tile of a second launch
            // over the last outputs, all by estimated time. (Measured against the rules below,
            // which this replaced: [8192, 8192] x 256 tokens 58 -> 47 us, [10240, 8192] x 256
            // 77 -> 56, [4096, 14336] x 384 79 -> 59, [8192, 28672] x 384 305 -> 234.)
            plan.family = FAMILY_DMA;
            double best = 1e300;
            const int shares[] = {1, 2, 3, 4, 6, 8};
            for (const DmaPrice &price : dma_prices)
                for (const int count : shares) {
                    const TnVariant &v = dma_variant(price.variant);
                    const double workgroups = double(ceil_div(outputs, v.block_n)) * ceil_div(tokens, v.block_m) * count;
                    if (count > 1 && (k / count < 512 || workgroups > 2.0 * compute_units ||
                                      double(count) * tokens * outputs * 4 > double(1 << 28)))
                        continue;
                    const double us = dma_launch_us(price, outputs, tokens, k, count, compute_units);
                    if (us < best) {
                        best = us;
                        plan.kernel = price.variant;
                        plan.split_k = count;
                    }
                }
            for (const DmaPrice &main : dma_prices) {
                const TnVariant &v = dma_variant(main.variant);
                const int token_tiles = ceil_div(tokens, v.block_m);
                const int whole = ceil_div(outputs, v.block_n) * token_tiles / compute_units;
                const int main_outputs = whole * compute_units / token_tiles * v.block_n;
                if (whole < 1 || main_outputs < 1 || main_outputs >= outputs)
                    continue;
                const double main_us = dma_launch_us(main, main_outputs, tokens, k, 1, compute_units);
                for (const DmaPrice &tail : dma_prices) {
                    const double us =
                        main_us + dma_launch_us(tail, outputs - main_outputs, tokens, k, 1, compute_units) + 3.0;
                    if (us < 0.97 * best) {
                        best = us / 0.97;
                        plan.kernel = main.variant;
                        plan.split_k = 1;
                        plan.tail_kernel = tail.variant;
                        plan.tail_outputs = outputs - main_outputs;
                    }
                }
            }
        } else if (ceil_div(outputs, 128) * ceil_div(tokens, 128) * 2 <= compute_units) {
            // few output tiles (a narrow projection, a small batch): 128 x 128 register-staged
            // tiles with K divided over workgroups, the largest power-of-two split that keeps the
            // grid within two workgroups per compute unit and at least 512 of K per partition
            // (measured against the direct-to-LDS tiles: [8192, 28672] x 128 tokens 120 vs 314 us,
            // x 256 tokens 181 vs 313 us; [8192, 8192] x 128 tokens 42 vs 71 us)
            plan.kernel = 2;
            const int tiles = ceil_div(outputs, 128) * ceil_div(tokens, 128);
            plan.split_k = 1;
            while (plan.split_k < 16 && tiles * plan.split_k * 2 <= 2 * compute_units &&
                   k / (plan.split_k * 2) >= 512)
                plan.split_k *= 2;
        } else {
            // prefill: larger tiles reuse more per byte; prefer them unless a smaller tile fills
            // the compute units noticeably better
            const bool direct = k % 64 == 0 && outputs % 4 == 0 && ldc % 4 == 0 &&
                                lda < (1 << 22) && ldb < (1 << 22);
            double best = -1;
            if (direct) {
                // direct-to-LDS tiles: {variant, resident workgroups per CU, relative efficiency}
                // (with K a multiple of 128 the two largest tiles run on four wavefronts with the K loop
                // in assembly, 5 % faster tile for tile, so the smaller tiles weigh a little less; per
                // round of workgroups at 8192 tokens: 320 x 256 230 us, 256 x 256 189 us)
                struct Candidate {
                    int variant, resident;
                    double weight;
                };
                const bool four_wavefronts = k % 128 == 0 && k <= 16384;
                const Candidate eight[] = {{10, 1, 1.0}, {6, 1, 0.96}, {11, 1, 0.88}, {9, 1, 0.85}, {5, 1, 0.83}};
                const Candidate four[] = {{10, 1, 1.0}, {6, 1, 0.96}, {11, 1, 0.84}, {9, 1, 0.81}, {5, 1, 0.79}};
                const Candidate(&candidates)[5] = four_wavefronts ? four : eight;
                plan.family = FAMILY_DMA;
                for (const auto &candidate : candidates) {
                    const TnVariant &v = dma_variant(candidate.variant);
                    double score = candidate.weight * occupancy_score(outputs, tokens, v.block_n,
                                                                      v.block_m, candidate.resident,
                                                                      compute_units);
                    if (score > best) {
                        best = score;
                        plan.kernel = candidate.variant;
                    }
                }
                // Two launches: whole rounds of one tile over the first outputs, then the outputs
                // that would have made a partly filled last round on the tile that covers them
                // cheapest. Costs in tile area per unit of efficiency; a second launch is priced
                // like 5 us of a compute unit's work (0.38 ps per element of tile area and of K).
                auto rounds_cost = [&](int rows, int variant, double weight) {
                    const TnVariant &v = dma_variant(variant);
                    const double tiles = double(ceil_div(rows, v.block_n)) * ceil_div(tokens, v.block_m);
                    return std::ceil(tiles / compute_units) * v.block_n * v.block_m / weight;
                };
                double single = 1e300;
                for (const auto &candidate : candidates)
                    single = std::min(single, rounds_cost(outputs, candidate.variant, candidate.weight));
                const double launch_cost = 5.0 / (3.8e-7 * k);
                for (const auto &candidate : candidates) {
                    const TnVariant &v = dma_variant(candidate.variant);
                    const int token_tiles = ceil_div(tokens, v.block_m);
                    const int whole = ceil_div(outputs, v.block_n) * token_tiles / compute_units;
                    const int main_outputs = whole * compute_units / token_tiles * v.block_n;
                    if (whole < 1 || main_outputs < 1 || main_outputs >= outputs)
                        continue;
                    const double main_cost = rounds_cost(main_outputs, candidate.variant, candidate.weight);
                    for (const auto &tail : candidates) {
                        const double cost =
                            main_cost + rounds_cost(outputs - main_outputs, tail.variant, tail.weight) + launch_cost;
                        if (cost < 0.97 * single) {
                            single = cost / 0.97;
                            plan.kernel = candidate.variant;
                            plan.tail_kernel = tail.variant;
                            plan.tail_outputs = outputs - main_outputs;
                        }
                    }
                }
            } else {
                const int candidates[3] = {0, 1, 2};
                const int resident[3] = {1, 1, 2};
                const double weight[3] = {0.5, 0.95, 1.0};
                for (int i = 0; i < 3; ++i) {
                    const TnVariant &v = tn_variant(candidates[i]);
                    double score = weight[i] * occupancy_score(outputs, tokens, v.block_n,
                                                               v.block_m, resident[i],
                                                               compute_units);
                    if (score > best) {
                        best = score;
                        plan.kernel = candidates[i];
                    }
                }
            }
            plan.split_k = 1;
        }
        if (plan.family == FAMILY_DMA) {
            // every tile above exists on the 16 x 16 x 32 matrix instruction as well, which the part
            // runs at a higher clock on real data: 3 to 11 % faster tile for tile (measured:
            // 4096 x 10240 x 8192 534 -> 481 us, 8192^3 on 256 x 256 tiles 862 -> 807)
            // (the 320 x 256 and 256 x 256 tiles: on four wavefronts, one per SIMD, when K allows)
            // (measured round-robin on one box: 4096 x 10240 x 8192 478 -> 457 us, 8192^3 806 -> 757,
            // 2048 x 8192 x 8192 204 -> 194; at K = 28672 the eight-wavefront tiles stay 3 % ahead)
            const bool four_wavefronts = k % 128 == 0 && k <= 16384 && plan.split_k == 1;
            const auto narrow = [four_wavefronts](int variant) {
                switch (variant) {
                case 10: return four_wavefronts ? 19 : 12;
                case 6: return four_wavefronts ? 18 : 13;
                case 11: return 14;
                case 9: return 15;
                case 8: return 16;
                case 5: return 17;
                default: return variant;
                }
            };
            plan.kernel = narrow(plan.kernel);
            plan.tail_kernel = narrow(plan.tail_kernel);
        }
        return plan;
    }
    // FP8 block-scaled: rows = n (tokens), outputs = m, always K-contiguous
    plan.counter = 4;
    const bool tiles_apply = m % 4 == 0 && k < (1 << 24); // what the direct-to-LDS tiles need
    // (the streaming kernel holds a row of K / 128 scales per token in LDS: K up to 24576; 33 to 64
    // tokens go to the tiles when K is long enough to divide: measured at K = 1536 and 2048 the
    // streaming kernel is 35 % faster there, at 7168 and 18432 the tiles are 10 to 35 % faster)
    const bool streamable = k / 128 <= STREAM_SCALE_GROUPS;
    // (up to 8 tokens: only when the 16-row tiles alone fill the compute units; narrower projections
    // keep the small tiles with divided K below. [18432, 7168] at 1 token: 24.2 us in this one launch
    // against 24.5 in the two launches of the divided product, at 8 tokens 25.1 against 25.5 to 26.6)
    const bool enough_rows = n > 8 || ceil_div(m, 16) >= compute_units;
    if (enough_rows && streamable && (n <= 32 || (n <= 64 && (!tiles_apply || k < 4096)))) {
        // decode batches: one streaming pass over the weights, whole K per workgroup; the row
        // tiles are limited by the operand registers (row_tiles * token_tiles <= 16, sum <= 10).
        // From 33 tokens on the 64-token tiles below with divided K are faster, but for the wide
        // projections of the rule that follows this one.
        const int token_tiles = n <= 16 ? 1 : n <= 32 ? 2 : 4;
        const int limit = std::min(16 / token_tiles, 10 - token_tiles);
        plan.family = FAMILY_FP8_STREAM;
        plan.kernel =
            10 * fp8_stream_row_tiles(m, token_tiles, compute_units, std::min(8, limit)) + token_tiles;
        return plan;
    }
    if (n > 32 && n <= 64 && streamable && enough_rows) {
        // 33 to 64 tokens on a projection whose 16-row tiles come to about one workgroup of five or six per
        // compute unit: the streaming kernel again, with three token tiles up to 48 tokens, four above
        // ([18432, 7168] in 231 workgroups of 80 rows: 27.0 / 28.2 / 32.2 us at 33 / 48 / 64 tokens against
        // 30.6 / 31.5 / 33.6 on the tiles with K divided; with fewer rows per workgroup, or a number of
        // workgroups just above the compute units, the tiles stay ahead: [7168, 18432] 32 against 46 to 63)
        const int token_tiles = n <= 48 ? 3 : 4;
        const int row_tiles = ceil_div(ceil_div(m, 16), compute_units);
        const int workgroups = ceil_div(ceil_div(m, 16), row_tiles);
        if (row_tiles >= 5 && row_tiles * token_tiles <= 20 && row_tiles + token_tiles <= 10 &&
            workgroups * 100 >= compute_units * 85) {
            plan.family = FAMILY_FP8_STREAM;
            plan.kernel = 10 * row_tiles + token_tiles;
            return plan;
        }
    }
    if (n <= 8) {
        // a handful of tokens: small tiles with split-K put the most workgroups on the weight stream
        plan.family = FAMILY_FP8_BLOCK;
        plan.kernel = 3; // 64 x 32 tiles, split-K: the most workgroups in flight for the weight stream
        const TnVariant &v = fp8_variant(plan.kernel);
        plan.split_k = decode_split(ceil_div(m, v.block_n), ceil_div(k, v.block_k), compute_units);
        return plan;
    }
    if (!tiles_apply) {
        plan.family = FAMILY_FP8_BLOCK;
        plan.kernel = 0;
        return plan;
    }
    plan.family = FAMILY_FP8_DMA;
    // {256, 192} x {256, 128, 64} tiles, one workgroup per compute unit, the K groups of a tile
    // divided over up to eight workgroups when the tiles alone leave compute units empty (FP32
    // planes summed in share order by a second launch). Each choice is priced in microseconds:
    // rounds of workgroups x K groups per workgroup x the measured time of one group of that tile
    // with the machine full (18432 x 7168 at 4096 tokens), plus what dividing costs. Checked
    // against sweeps of every tile and split on [18432, 7168], [7168, 18432], [4096, 7168],
    // [2048, 7168], [7168, 2048] and [24576, 1536] from 72 to 4096 tokens: the choice is the
    // measured best or within a few per cent of it (e.g. [7168, 18432] at 256 tokens 60 us with
    // 256 x 128 tiles in four shares against 98 undivided; [4096, 7168] at 256 tokens 24 against 38).
    // (The 64-token tiles are priced as measured with weights that come from memory, not from the
    // last-level cache: every further token tile re-reads the weight rows.)
    const struct {
        int variant;
        double group_us;
    } candidates[] = {{0, 1.88}, {8, 1.55}, {4, 1.12}, {7, 0.90}, {6, 0.90}, {9, 0.72}};
    const int groups = k / 128;
    double best = 1e30;
    for (const auto &candidate : candidates) {
        const TnVariant &v = fp8_dma_variant(candidate.variant);
        const int tiles = ceil_div(m, v.block_n) * ceil_div(n, v.block_m);
        // shares: as many as keep the grid within one round, at least six groups each
        const int limit = std::max(1, std::min({8, groups / 6, compute_units / std::max(1, tiles)}));
        for (int shares = 1; shares <= limit; ++shares) {
            const int steps = ceil_div(groups, shares);
            if (shares > 1 && ceil_div(groups, steps) != shares)
                continue; // (the launcher would use fewer)
            const double rounds = double(ceil_div(tiles * shares, compute_units));
            double cost = rounds * steps * candidate.group_us;
            if (shares > 1) // a second launch, and the planes written and read once
                cost += 5.0 + 2.0 * shares * double(m) * n * 4.0 / 4.0e6;
            if (cost < best) {
                best = cost;
                plan.kernel = candidate.variant;
                plan.split_k = shares;
            }
        }
    }
    // Two launches: whole rounds of one tile over the first outputs, and the outputs that would
    // have made a partly filled last round on whichever tile covers them cheapest (18432 outputs
    // by 4096 tokens are 4.5 rounds of 256 x 256 tiles: four rounds over 16384 outputs, then the
    // last 2048 outputs as exactly one round of 256 x 128 tiles; measured 489 against 521 us).
    for (const auto &candidate : candidates) {
        const TnVariant &v = fp8_dma_variant(candidate.variant);
        const int token_tiles = ceil_div(n, v.block_m);
        const int whole_rounds = ceil_div(m, v.block_n) * token_tiles / compute_units;
        int main_row_tiles = whole_rounds * compute_units / token_tiles;
        if (v.block_n % 128 != 0)
            main_row_tiles -= main_row_tiles % 2; // (192-row tiles: the tail starts at a multiple of 128)
        const int main_outputs = main_row_tiles * v.block_n;
        if (whole_rounds < 1 || main_row_tiles < 1 || main_outputs >= m)
            continue;
        const double main_cost =
            double(ceil_div(main_row_tiles * token_tiles, compute_units)) * groups * candidate.group_us;
        for (const auto &tail : candidates) {
            const TnVariant &t = fp8_dma_variant(tail.variant);
            const int tail_tiles = ceil_div(m - main_outputs, t.block_n) * ceil_div(n, t.block_m);
            const double cost =
                main_cost + double(ceil_div(tail_tiles, compute_units)) * groups * tail.group_us + 5.0;
            if (cost < 0.97 * best) {
                best = cost / 0.97;
                plan.kernel = candidate.variant;
                plan.split_k = 1;
                plan.tail_kernel = tail.variant;
                plan.tail_outputs = m - main_outputs;
            }
        }
    }
    // The 128-token and 256-token tiles also exist on the 16 x 16 x 128 matrix instruction, which the
    // part runs at a higher clock on real data; that pays where the launch is bound by arithmetic
    // (measured tile for tile: 256 x 256 at 4096 tokens 534 -> 509 us, 192 x 128 from 256 tokens on
    // 2 to 6 % faster, 192 x 256 1 to 6 %; with fewer tokens, and on the 64-token tiles, the four
    // times as many instructions per group cost more than the clock gives).
    const auto narrow = [&](int variant) {
        if (variant == 0 && n >= 2048)
            return 10;
        if (variant == 7 && n >= 256)
            return 13;
        if (variant == 8 && n >= 256)
            return 14;
        return variant;
    };
    plan.kernel = narrow(plan.kernel);
    if (plan.tail_outputs)
        plan.tail_kernel = narrow(plan.tail_kernel);
    return plan;
}

// The streaming kernel's variant code when every workgroup takes the whole K extent.
int undivided_stream_kernel(int outputs, int tokens, int k, int compute_units)
{
    const int row_tiles = stream_row_tiles(outputs, compute_units);
    // (65 to 128 tokens on a wide projection: as many token tiles as the tokens need, one K block per step;
    // [28672, 8192] at 80 / 96 / 128 tokens 82 / 90 / 107 us against 115 / 114 / 122 on the direct-to-LDS tiles.
    // Narrow projections keep the tiles there: a divided K and the token rows every workgroup re-reads cost more.)
    const int token_tiles = tokens <= 16 ? 1 : tokens <= 32 ? 2 : tokens <= 48 ? 3 : tokens <= 64 ? 4 : ceil_div(tokens, 16);
    if (token_tiles > 4)
        return 10 * row_tiles + token_tiles;
    return 100 * stream_depth_log2(row_tiles, token_tiles, k) + 10 * row_tiles + token_tiles;
}

void describe_plan(const Plan &plan, int dtype, char *text, size_t bytes)
{
    if (!text || !bytes)
        return;
    const char *type = dtype == 0 ? "f32" : dtype == 2 ? "bf16" : "fp8-block128";
    switch (plan.family) {
    case FAMILY_GEMV_F32:
        std::snprintf(text, bytes, "%s gemv wave-per-row", type);
        break;
    case FAMILY_MFMA_F32:
        if (plan.split_k > 1)
            std::snprintf(text, bytes, "%s mfma %s split_k=%d", type, plan.kernel == 2 ? "128x32x32" : "128x64x32",
                          plan.split_k);
        else
            std::snprintf(text, bytes, "%s mfma %s", type, plan.kernel == 0 ? "128x128x32" : "128x64x32");
        break;
    case FAMILY_MFMA_BF16:
        std::snprintf(text, bytes, "%s mfma any-layout %s", type, plan.kernel == 0 ? "128x128x32" : "128x64x32");
        break;
    case FAMILY_MFMA_TN:
        std::snprintf(text, bytes, "%s %s split_k=%d", type, tn_variant(plan.kernel).name,
                      plan.split_k);
        break;
    case FAMILY_FP8_BLOCK:
        std::snprintf(text, bytes, "%s %s split_k=%d", type, fp8_variant(plan.kernel).name,
                      plan.split_k);
        break;
    case FAMILY_FP8_DMA:
        if (plan.tail_outputs)
            std::snprintf(text, bytes, "%s %s split_k=%d, last %d outputs %s", type,
                          fp8_dma_variant(plan.kernel).name, plan.split_k, plan.tail_outputs,
                          fp8_dma_variant(plan.tail_kernel).name);
        else
            std::snprintf(text, bytes, "%s %s split_k=%d", type, fp8_dma_variant(plan.kernel).name, plan.split_k);
        break;
    case FAMILY_FP8_STREAM:
        std::snprintf(text, bytes, "%s stream rows=%d tokens=%d", type, 16 * (plan.kernel / 10),
                      16 * (plan.kernel % 10));
        break;
    case FAMILY_DMA:
        if (plan.tail_outputs)
            std::snprintf(text, bytes, "%s %s, last %d outputs %s", type, dma_variant(plan.kernel).name,
                          plan.tail_outputs, dma_variant(plan.tail_kernel).name);
        else if (plan.split_k > 1)
            std::snprintf(text, bytes, "%s %s split_k=%d", type, dma_variant(plan.kernel).name, plan.split_k);
        else
            std::snprintf(text, bytes, "%s %s", type, dma_variant(plan.kernel).name);
        break;
    case FAMILY_NN:
        std::snprintf(text, bytes, "%s outputs-contiguous stream 128x64 split_k=%d", type, plan.split_k);
        break;
    case FAMILY_STREAM:
        std::snprintf(text, bytes, "%s stream rows=%d tokens=%d k_step=%d k_shares=%d", type,
                      16 * (plan.kernel / 10 % 10), 16 * (plan.kernel % 10),
                      128 << (plan.kernel / 100), plan.split_k);
        break;
    default:
        std::snprintf(text, bytes, "%s generic 64x64x16", type);
    }
}
} // namespace camblas_hip
