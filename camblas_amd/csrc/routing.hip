// Mixture-of-experts routing helpers (contract: ref include/camblas_cuda.h:168-185,
// src/cuda/backend.cu:1306-1361, src/cuda/routing.cuh:1-56).
//
// route_groups: expert IDs [tokens, choices] (int64) -> for every local group (active[g] is the
// local expert ID it serves, the first group wins for duplicates) the list of (token, choice)
// slots routed to it, `rows` at most, and for every slot its position in that list. The reference
// hands rows out with an atomic counter, so its row order inside a group depends on scheduling;
// here a group's rows are assigned in ascending slot order (one workgroup per group, ballot
// prefix sums), which is one of the orders the contract allows and makes the result reproducible.
// counts[g] is the number of slots routed to the group, including those beyond `rows`.
//
// reduce_groups: out[token, :] = sum over the token's choices, in ascending (expert ID, choice)
// order, of the BF16 row reverse[token, choice] of the grouped matrix, accumulated in FP32.
#include "common.hpp"
#include "device.hpp"

#include <climits>

namespace camblas_hip
{
namespace
{
constexpr int THREADS = 256;

__global__ __launch_bounds__(THREADS) void route_fill_kernel(int groups, size_t slot_cells,
                                                             size_t reverse_cells, int32_t *counts,
                                                             int32_t *slots, int32_t *reverse)
{
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    const size_t first = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    for (size_t index = first; index < size_t(groups); index += stride)
        counts[index] = 0;
    for (size_t index = first; index < slot_cells; index += stride)
        slots[index] = -1;
    for (size_t index = first; index < reverse_cells; index += stride)
        reverse[index] = -1;
}

// One workgroup of sixteen wavefronts per group. The slots are divided into sixteen contiguous
// ranges, one per wavefront; a first pass counts each range's matches, one barrier turns the counts
// into the row at which each range starts, and a second pass hands out the rows in ascending slot
// order. (A workgroup-wide prefix sum per 256 slots, two barriers each, took 92 us for 65536 slots.)
constexpr int ROUTE_THREADS = 1024;
__global__ __launch_bounds__(ROUTE_THREADS) void route_assign_kernel(int slot_count, int first_expert,
                                                                     int rows, const int64_t *experts,
                                                                     const int32_t *active, int32_t *counts,
                                                                     int32_t *slots, int32_t *reverse)
{
    constexpr int WAVES = ROUTE_THREADS / 64;
    __shared__ int wave_total[WAVES];
    __shared__ int earlier;
    const int group = blockIdx.x, thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int local = active[group];
    // duplicate active IDs select their first group: a later one receives nothing
    if (thread == 0)
        earlier = 0;
    __syncthreads();
    for (int other = thread; other < group; other += ROUTE_THREADS)
        if (active[other] == local)
            earlier = 1;
    __syncthreads();
    if (earlier)
        return; // counts[group] stays 0, slots stay -1
    const int range = ((slot_count + WAVES - 1) / WAVES + 63) / 64 * 64;
    const int begin = wave * range < slot_count ? wave * range : slot_count;
    const int end = begin + range < slot_count ? begin + range : slot_count;
    auto matches = [&](int slot) {
        if (slot >= end)
            return false;
        const int64_t expert = experts[slot];
        return expert >= first_expert && expert < INT_MAX && int(expert) - first_expert == local;
    };
    int found = 0;
    for (int base = begin; base < end; base += 64)
        found += __popcll(__ballot(matches(base + lane)));
    if (lane == 0)
        wave_total[wave] = found;
    __syncthreads();
    int row = 0, total = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        if (w < wave)
            row += wave_total[w];
        total += wave_total[w];
    }
    for (int base = begin; base < end; base += 64) {
        const int slot = base + lane;
        const bool mine = matches(slot);
        const unsigned long long ballot = __ballot(mine);
        const int mine_row = row + __popcll(ballot & ((1ull << lane) - 1ull));
        if (mine && mine_row < rows) {
            slots[size_t(group) * rows + mine_row] = slot;
            reverse[slot] = group * rows + mine_row;
        }
        row += __popcll(ballot);
    }
    if (thread == 0)
        counts[group] = total;
}

// One workgroup per token: the choices are ranked by (expert ID, choice) once, then every thread
// sums its columns in that order.
__global__ __launch_bounds__(THREADS) void reduce_groups_kernel(int choices, int width,
                                                                int grouped_rows,
                                                                const int64_t *experts,
                                                                const int32_t *reverse,
                                                                const unsigned short *input,
                                                                float *output)
{
    __shared__ int ordered_row[64];
    __shared__ int ordered_count;
    const int token = blockIdx.x, thread = threadIdx.x;
    const int64_t *mine = experts + size_t(token) * choices;
    if (thread < 64)
        ordered_row[thread] = -1;
    __syncthreads();
    if (thread < choices) {
        const int64_t expert = mine[thread];
        const bool valid = expert >= 0 && expert < INT_MAX;
        int rank = 0, valid_total = 0;
        for (int other = 0; other < choices; ++other) {
            const int64_t theirs = mine[other];
            const bool theirs_valid = theirs >= 0 && theirs < INT_MAX;
            valid_total += theirs_valid;
            rank += theirs_valid && (theirs < expert || (theirs == expert && other < thread));
        }
        if (valid) {
            const int row = reverse[size_t(token) * choices + thread];
            ordered_row[rank] = row >= 0 && row < grouped_rows ? row : -1;
        }
        if (thread == 0)
            ordered_count = valid_total;
    }
    __syncthreads();
    const int count = ordered_count;
    for (int column = thread; column < width; column += THREADS) {
        float sum = 0.f;
        for (int step = 0; step < count; ++step) {
            const int row = ordered_row[step];
            if (row >= 0)
                sum = __fadd_rn(sum, bf16_bits_to_float(input[size_t(row) * width + column]));
        }
        output[size_t(token) * width + column] = sum;
    }
}
// The same with eight columns per thread (16-byte loads, all rows of a step's eight choices requested
// before the first is added) and the columns of a token spread over gridDim.y workgroups: a token
// summed one column and one choice at a time is a chain of 28 x 8 dependent 2-byte loads (36 us for
// one token of 7168 columns; 2.2 TB/s at 8192 tokens).
__global__ __launch_bounds__(THREADS) void reduce_groups_wide_kernel(int choices, int vectors, int grouped_rows,
                                                                     const int64_t *experts, const int32_t *reverse,
                                                                     const u32x4_t *input, f32x4_t *output)
{
    __shared__ int ordered_row[64];
    __shared__ int ordered_count;
    const int token = blockIdx.x, thread = threadIdx.x;
    const int64_t *mine = experts + size_t(token) * choices;
    if (thread < 64)
        ordered_row[thread] = -1;
    __syncthreads();
    if (thread < choices) {
        const int64_t expert = mine[thread];
        const bool valid = expert >= 0 && expert < INT_MAX;
        int rank = 0, valid_total = 0;
        for (int other = 0; other < choices; ++other) {
            const int64_t theirs = mine[other];
            const bool theirs_valid = theirs >= 0 && theirs < INT_MAX;
            valid_total += theirs_valid;
            rank += theirs_valid && (theirs < expert || (theirs == expert && other < thread));
        }
        if (valid) {
            const int row = reverse[size_t(token) * choices + thread];
            ordered_row[rank] = row >= 0 && row < grouped_rows ? row : -1;
        }
        if (thread == 0)
            ordered_count = valid_total;
    }
    __syncthreads();
    const int count = ordered_count;
    for (int vector = int(blockIdx.y) * THREADS + thread; vector < vectors; vector += int(gridDim.y) * THREADS) {
        float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int first = 0; first < count; first += 8) {
            u32x4_t part[8];
            bool present[8];
#pragma unroll
            for (int step = 0; step < 8; ++step) {
                const int row = first + step < count ? ordered_row[first + step] : -1;
                present[step] = row >= 0;
                part[step] = input[size_t(present[step] ? row : 0) * vectors + vector];
            }
#pragma unroll
            for (int step = 0; step < 8; ++step)
                if (present[step]) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        sum[2 * e] = __fadd_rn(sum[2 * e], __uint_as_float(part[step][e] << 16));
                        sum[2 * e + 1] = __fadd_rn(sum[2 * e + 1], __uint_as_float(part[step][e] & 0xffff0000u));
                    }
                }
        }
        f32x4_t *out = output + (size_t(token) * vectors + vector) * 2;
        out[0] = f32x4_t{sum[0], sum[1], sum[2], sum[3]};
        out[1] = f32x4_t{sum[4], sum[5], sum[6], sum[7]};
    }
}
} // namespace

hipError_t launch_route_groups(hipStream_t stream, int tokens, int choices, int first_expert,
                               int groups, int rows, const void *experts, const void *active,
                               void *counts, void *slots, void *reverse)
{
    const size_t slot_cells = size_t(groups) * rows, reverse_cells = size_t(tokens) * choices;
    const size_t cells = slot_cells > reverse_cells ? slot_cells : reverse_cells;
    const unsigned blocks = unsigned(std::min<size_t>((cells + THREADS - 1) / THREADS + 1, 4096));
    // a fill kernel rather than memset nodes, so that the call can be captured in a graph
    route_fill_kernel<<<blocks, THREADS, 0, stream>>>(groups, slot_cells, reverse_cells,
                                                      static_cast<int32_t *>(counts),
                                                      static_cast<int32_t *>(slots),
                                                      static_cast<int32_t *>(reverse));
    hipError_t status = launch_status();
    if (status != hipSuccess || !tokens)
        return status;
    route_assign_kernel<<<unsigned(groups), ROUTE_THREADS, 0, stream>>>(
        tokens * choices, first_expert, rows, static_cast<const int64_t *>(experts),
        static_cast<const int32_t *>(active), static_cast<int32_t *>(counts),
        static_cast<int32_t *>(slots), static_cast<int32_t *>(reverse));
    return launch_status();
}

hipError_t launch_reduce_groups(hipStream_t stream, int tokens, int choices, int width,
                                int grouped_rows, const void *experts, const void *reverse,
                                const void *input, void *output)
{
    if (width % 8 == 0 && grouped_rows > 0 && reinterpret_cast<uintptr_t>(input) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(output) % 16 == 0) {
        const int vectors = width / 8;
        const int chunks = (vectors + THREADS - 1) / THREADS;
        const dim3 grid(unsigned(tokens), unsigned(chunks < 8 ? chunks : 8));
        reduce_groups_wide_kernel<<<grid, THREADS, 0, stream>>>(
            choices, vectors, grouped_rows, static_cast<const int64_t *>(experts), static_cast<const int32_t *>(reverse),
            static_cast<const u32x4_t *>(input), static_cast<f32x4_t *>(output));
        return launch_status();
    }
    reduce_groups_kernel<<<unsigned(tokens), THREADS, 0, stream>>>(
        choices, width, grouped_rows, static_cast<const int64_t *>(experts),
        static_cast<const int32_t *>(reverse), static_cast<const unsigned short *>(input),
        static_cast<float *>(output));
    return launch_status();
}
} // namespace camblas_hip
