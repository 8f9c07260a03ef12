// Grouped-query decode attention: one query token per sequence against a BF16 KV cache
// [batch, context, kv_heads, 128], split over the context so that a batch of 32 sequences fills
// 256 compute units, then an ordered combine. The reference has no counterpart (its
// src/cuda/fusion.cuh:95-157 is dense single-head FP32/FP64 with a materialised score matrix); the
// arithmetic is the textbook softmax(scale * q k^T) v with FP32 accumulation and an online-softmax
// merge of the context partitions.
//
// Partition kernel, one workgroup per (256 positions, kv head, sequence); each of its 4 wavefronts
// owns 64 positions and runs both products on the matrix cores (v_mfma_f32_16x16x32_bf16), with the
// query heads of the group padded to 16:
//   scores  S[position, head] = K[position, :] . Q[head, :]    A = K rows (16-byte loads), B = Q
//   output  O[head, dim]      = P[head, position] . V[position, dim]
// The score tile leaves the first product with lane l holding head l%16 and four positions, which
// is already the A-operand layout of the second product once the K index of that product is
// *defined* as the position order the lane holds; V has to follow the same order. V is read with
// 16-byte loads (a lane takes dims 8m..8m+7 of its eight positions, 16 lanes cover one 256-byte
// row) and transposed in registers with byte permutes into eight B operands, one per dim offset
// w, so that output column m of product w is dim 8m + w.
// All K, V and Q loads of a wavefront are issued before the first product, which keeps about
// 32 KB per wavefront in flight. The wavefronts' partial (max, sum, O) are merged through LDS in
// wavefront order. The kernel is bound by the cache read (2 * context * 256 bytes per kv head
// and sequence).
#include "common.hpp"
#include "device.hpp"

#include <atomic>

namespace camblas_hip
{
namespace
{
constexpr int DIM = 128, CHUNK = 256, WAVES = 4, WAVE_POSITIONS = CHUNK / WAVES, HEADS = 16;

// Partials of the allocation-free entry point: one fixed array in the library's device image, so
// every GPU that loads the library holds its own 16 MiB copy until the process ends. The name is
// a host-side stand-in, not a device address: host code only ever uses the per-device address
// that hipGetSymbolAddress returned (resident_partials below).
constexpr size_t RESIDENT_BYTES = size_t(16) << 20;
constexpr int MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[RESIDENT_BYTES];
std::atomic<void *> resident_address[MAX_DEVICES] = {};

__device__ __forceinline__ float swap_lanes(float value, int mask)
{
    return __shfl_xor(value, mask, 64);
}

// What the FRESH form of the partition kernel adds: the step's new token arrives un-rotated in a
// fused activation row [q heads | k heads | v heads] per sequence and is rotated here (q in
// registers, for every partition; k by the one wavefront whose positions hold the token's cache
// slot), that wavefront takes the new K and V rows from the activation instead of the cache, and
// writes them to the cache. This replaces a launch of the rotary-embedding + cache-append kernel.
struct FreshToken {
    const int32_t *positions; // cache slot of the new token per sequence; the sequence then has positions + 1 entries
    float theta;
    const unsigned short *k_new, *v_new; // rows of the activation, token_stride apart per sequence, head-major
    int token_stride;
    unsigned short *k_cache, *v_cache;
    // optional: sines [batch][64] then cosines of the positions' angles, made once per decode step for all
    // layers (rope_table_kernel); without it every workgroup works the angles out itself
    const float *table;
};

// positions the attention covers: lengths[b], or, in the FRESH form, positions[b] + 1
__device__ __forceinline__ int live_length(const int32_t *lengths, const int32_t *positions, int b, int context_length)
{
    if (positions)
        return min(max(positions[b] + 1, 0), context_length);
    return lengths ? min(max(lengths[b], 0), context_length) : context_length;
}

// rotates the pair (lo, hi) of packed BF16 vectors: element e of lo pairs with element e of hi; the
// eight sines and cosines are read from LDS where they are used, so that they do not occupy registers
// across the kernel
__device__ __forceinline__ void rotate_vectors(const float *sines, const float *cosines, u32x4_t &lo, u32x4_t &hi)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        unsigned short l0, h0, l1, h1;
        rotate_by(sines[2 * e], cosines[2 * e], __uint_as_float(lo[e] << 16), __uint_as_float(hi[e] << 16), l0, h0);
        rotate_by(sines[2 * e + 1], cosines[2 * e + 1], __uint_as_float(lo[e] & 0xffff0000u),
                  __uint_as_float(hi[e] & 0xffff0000u), l1, h1);
        lo[e] = unsigned(l0) | (unsigned(l1) << 16);
        hi[e] = unsigned(h0) | (unsigned(h1) << 16);
    }
}

template <bool FRESH>
__device__ __forceinline__ void gqa_partition(
    int q_heads, int kv_heads, int context_length, const int32_t *lengths, float scale,
    const unsigned short *q, int q_stride, const unsigned short *k_cache,
    const unsigned short *v_cache, float *part_o, float *part_m, float *part_l, int splits,
    int group, const FreshToken &fresh)
{
    __shared__ __attribute__((aligned(16))) float wave_o[WAVES][HEADS][DIM];
    __shared__ float wave_m[WAVES][HEADS], wave_l[WAVES][HEADS];
    __shared__ float trig[2][FRESH ? DIM / 2 : 1]; // FRESH: sines and cosines of the new token's position
    // Consecutive workgroups go to consecutive XCDs, so with the partition as the fast grid index
    // and a partition count that is a multiple of eight, partition s of every sequence and head
    // would run on XCD s % 8: sequences much shorter than the cache would keep one or two XCDs
    // busy and leave the rest idle. The partition index is rotated by the (head, sequence) number.
    const int kvh = blockIdx.y, b = blockIdx.z;
    const int split = int((blockIdx.x + blockIdx.y + blockIdx.z * gridDim.y) % gridDim.x);
    const int thread = threadIdx.x, lane = thread % 64, wave = thread / 64;
    const int m = lane % 16, j = lane / 16;
    const int length = live_length(lengths, FRESH ? fresh.positions : nullptr, b, context_length);
    if (split * CHUNK >= length)
        return; // past the sequence: the combine never reads this partition (uniform, before any barrier)
    const int begin = split * CHUNK + wave * WAVE_POSITIONS;
    const int count = min(WAVE_POSITIONS, length - begin); // may be <= 0: nothing for this wave
    const size_t row_stride = size_t(kv_heads) * DIM;
    const unsigned short *k_base =
        k_cache + (size_t(b) * context_length + begin) * row_stride + size_t(kvh) * DIM;
    const unsigned short *v_base =
        v_cache + (size_t(b) * context_length + begin) * row_stride + size_t(kvh) * DIM;

    f32x4_t acc[8];
#pragma unroll
    for (int w = 0; w < 8; ++w)
        acc[w] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float top = -INFINITY, total = 0.f;
    bf16x8_t q_frag[4], k_frag[4][4];
    u32x4_t v_rows[2][8];
    // FRESH: the new token's slot relative to this wavefront's first position (outside
    // [0, count) when another wavefront or partition holds it, or when it lies outside the cache)
    const int token = FRESH ? fresh.positions[b] : -1;
    // (in scalar registers: the branches on it below are then branches, not predication, which keeps the
    // rare path's loads and temporaries out of the common path's register allocation)
    const int slot = __builtin_amdgcn_readfirstlane(FRESH && token >= 0 && token < context_length ? token - begin : -1);
    const int wave_count = __builtin_amdgcn_readfirstlane(count);
    const bool holds_token = slot >= 0 && slot < wave_count; // uniform over the wavefront
    if (count > 0) { // uniform over the wavefront
        // ---- loads: Q (head m, dims 32s + 8j ..), K (position 16t + m, same dims),
        // V (position 32u + 16(e/4) + 4j + e%4, dims 8m ..); rows past the end repeat the last one
        const int head = kvh * group + (m < group ? m : group - 1);
        const unsigned short *q_row = q + size_t(b) * q_stride + size_t(head) * DIM + 8 * j;
#pragma unroll
        for (int s = 0; s < 4; ++s)
            q_frag[s] = *reinterpret_cast<const bf16x8_t *>(q_row + 32 * s);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int position = 16 * t + m;
            position = position < count ? position : count - 1;
            const unsigned short *row = k_base + size_t(position) * row_stride + 8 * j;
#pragma unroll
            for (int s = 0; s < 4; ++s)
                k_frag[t][s] = *reinterpret_cast<const bf16x8_t *>(row + 32 * s);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                int position = 32 * u + 16 * (e / 4) + 4 * j + e % 4;
                position = position < count ? position : count - 1;
                // a V row is consumed whole by one load (16 lanes x 16 bytes) and read once: it
                // bypasses cache allocation; a K row is covered by four loads and stays cacheable
                v_rows[u][e] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(
                    v_base + size_t(position) * row_stride + 8 * m));
            }
    }
    if constexpr (FRESH) {
        // the sixty-four angles of the token's position, once per workgroup, while the loads travel
        // (every lane working out its own sixteen doubled the kernel's time)
        if (thread < DIM / 2) {
            if (fresh.table) {
                trig[0][thread] = fresh.table[(size_t(b) * 2) * (DIM / 2) + thread];
                trig[1][thread] = fresh.table[(size_t(b) * 2 + 1) * (DIM / 2) + thread];
            } else {
                pair_sincos(float(token), thread, DIM, fresh.theta, trig[0][thread], trig[1][thread]);
            }
        }
        __syncthreads();
    }
    if (count > 0) {
        if constexpr (FRESH) {
            // this lane's sixteen pair indices: dims 32 s + 8 j + e for s = 0, 1 pair with 64 + the same
            // (fragments s and s + 2), for the queries and for the new K row alike
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                u32x4_t lo = __builtin_bit_cast(u32x4_t, q_frag[s]), hi = __builtin_bit_cast(u32x4_t, q_frag[s + 2]);
                rotate_vectors(&trig[0][32 * s + 8 * j], &trig[1][32 * s + 8 * j], lo, hi);
                q_frag[s] = __builtin_bit_cast(bf16x8_t, lo);
                q_frag[s + 2] = __builtin_bit_cast(bf16x8_t, hi);
            }
            if (holds_token) {
                const unsigned short *k_new = fresh.k_new + size_t(b) * fresh.token_stride + size_t(kvh) * DIM;
                const unsigned short *v_new = fresh.v_new + size_t(b) * fresh.token_stride + size_t(kvh) * DIM;
                unsigned short *k_slot = fresh.k_cache + (size_t(b) * context_length + begin + slot) * row_stride +
                                         size_t(kvh) * DIM;
                unsigned short *v_slot = fresh.v_cache + (size_t(b) * context_length + begin + slot) * row_stride +
                                         size_t(kvh) * DIM;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    // (uniform: tile t holds the slot, or repeats it as the sequence's last row)
                    if (!((slot >= 16 * t && slot < 16 * t + 16) || (slot == wave_count - 1 && 16 * t + 15 > slot)))
                        continue;
                    int position = 16 * t + m;
                    position = position < count ? position : count - 1;
                    if (position == slot) {
                        // the token's cache slot is not written yet: what was loaded from it is replaced by
                        // the activation's row, rotated (a second, dependent load, in this one wavefront only)
#pragma unroll
                        for (int s = 0; s < 4; ++s)
                            k_frag[t][s] = *reinterpret_cast<const bf16x8_t *>(k_new + 32 * s + 8 * j);
#pragma unroll
                        for (int s = 0; s < 2; ++s) {
                            u32x4_t lo = __builtin_bit_cast(u32x4_t, k_frag[t][s]);
                            u32x4_t hi = __builtin_bit_cast(u32x4_t, k_frag[t][s + 2]);
                            rotate_vectors(&trig[0][32 * s + 8 * j], &trig[1][32 * s + 8 * j], lo, hi);
                            k_frag[t][s] = __builtin_bit_cast(bf16x8_t, lo);
                            k_frag[t][s + 2] = __builtin_bit_cast(bf16x8_t, hi);
                        }
                        if (16 * t + m == slot) // the lanes that hold the row itself (not a repeat of it) append it
#pragma unroll
                            for (int s = 0; s < 4; ++s)
                                *reinterpret_cast<bf16x8_t *>(k_slot + 32 * s + 8 * j) = k_frag[t][s];
                    }
                }
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        // (uniform: some lane of this register holds the slot or repeats it)
                        const int first = 32 * u + 16 * (e / 4) + e % 4, last = first + 12;
                        if (!((slot >= first && slot <= last) || (slot == wave_count - 1 && last > slot)))
                            continue;
                        int position = 32 * u + 16 * (e / 4) + 4 * j + e % 4;
                        const bool row_itself = position == slot;
                        position = position < count ? position : count - 1;
                        if (position == slot) // (also the lanes that repeat the last row: they must not keep stale data)
                            v_rows[u][e] = *reinterpret_cast<const u32x4_t *>(v_new + 8 * m);
                        if (row_itself)
                            *reinterpret_cast<u32x4_t *>(v_slot + 8 * m) = v_rows[u][e];
                    }
            }
        }

        // ---- scores: register r of tile t is position 16t + 4j + r, head m
        f32x4_t score[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            score[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s)
                score[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag[t][s], q_frag[s], score[t],
                                                                   0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float value = 16 * t + 4 * j + r < count ? score[t][r] * scale : -INFINITY;
                score[t][r] = value;
                top = fmaxf(top, value);
            }
        // the four lanes m, m+16, m+32, m+48 share a head; position 0 is always valid, so the
        // maximum is finite
        top = fmaxf(top, swap_lanes(top, 16));
        top = fmaxf(top, swap_lanes(top, 32));
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float e = __expf(score[t][r] - top);
                score[t][r] = e;
                total += e;
            }
        total += swap_lanes(total, 16);
        total += swap_lanes(total, 32);

        // ---- output: K index 8j + e of product u is position 32u + 16(e/4) + 4j + e%4
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            u32x4_t weights = {pack_bf16x2(score[2 * u][0], score[2 * u][1]),
                               pack_bf16x2(score[2 * u][2], score[2 * u][3]),
                               pack_bf16x2(score[2 * u + 1][0], score[2 * u + 1][1]),
                               pack_bf16x2(score[2 * u + 1][2], score[2 * u + 1][3])};
            bf16x8_t p_frag = __builtin_bit_cast(bf16x8_t, weights);
#pragma unroll
            for (int pair = 0; pair < 4; ++pair) {
                u32x4_t even, odd; // dims 8m + 2 pair and 8m + 2 pair + 1 of the eight positions
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    unsigned lo = v_rows[u][2 * c][pair], hi = v_rows[u][2 * c + 1][pair];
                    even[c] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                    odd[c] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
                }
                acc[2 * pair] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    p_frag, __builtin_bit_cast(bf16x8_t, even), acc[2 * pair], 0, 0, 0);
                acc[2 * pair + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    p_frag, __builtin_bit_cast(bf16x8_t, odd), acc[2 * pair + 1], 0, 0, 0);
            }
        }
    }

    // ---- merge the wavefronts: register r of acc[w] is head 4j + r, dim 8m + w
    if (j == 0) {
        wave_m[wave][m] = top;
        wave_l[wave][m] = total;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float *row = &wave_o[wave][4 * j + r][8 * m];
        *reinterpret_cast<f32x4_t *>(row) = f32x4_t{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
        *reinterpret_cast<f32x4_t *>(row + 4) = f32x4_t{acc[4][r], acc[5][r], acc[6][r], acc[7][r]};
    }
    __syncthreads();
    for (int index = thread; index < group * DIM; index += WAVES * 64) {
        const int h = index / DIM, d = index % DIM;
        float best = wave_m[0][h];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            best = fmaxf(best, wave_m[w][h]);
        float numerator = 0.f, denominator = 0.f;
        if (best > -INFINITY) {
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                float factor = __expf(wave_m[w][h] - best); // 0 for a wavefront without positions
                numerator = fmaf(factor, wave_o[w][h][d], numerator);
                denominator = fmaf(factor, wave_l[w][h], denominator);
            }
        }
        const size_t row = (size_t(b) * q_heads + kvh * group + h) * splits + split;
        part_o[row * DIM + d] = numerator;
        if (d == 0) {
            part_m[row] = best;
            part_l[row] = denominator;
        }
    }
}

// table[b][0][i] = sin, table[b][1][i] = cos of positions[b] * theta^(-2i/dim), i < dim / 2: the angles of a
// decode step, the same for every layer of a model
__global__ void rope_table_kernel(int batch, int dim, float theta, const int32_t *positions, float *table)
{
    const int half = dim / 2, index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= batch * half)
        return;
    const int b = index / half, i = index % half;
    pair_sincos(float(positions[b]), i, dim, theta, table[(size_t(b) * 2) * half + i], table[(size_t(b) * 2 + 1) * half + i]);
}

__global__ __launch_bounds__(WAVES * 64) void gqa_partition_kernel(
    int q_heads, int kv_heads, int context_length, const int32_t *lengths, float scale,
    const unsigned short *q, int q_stride, const unsigned short *k_cache,
    const unsigned short *v_cache, float *part_o, float *part_m, float *part_l, int splits, int group)
{
    gqa_partition<false>(q_heads, kv_heads, context_length, lengths, scale, q, q_stride, k_cache, v_cache, part_o,
                         part_m, part_l, splits, group, FreshToken{});
}

// (two wavefronts per SIMD, i.e. at most 256 registers, as the plain form has: two workgroups per
// compute unit keep twice the cache rows in flight; left alone this form allocated 268 registers and
// ran at half the rate)
__global__ __launch_bounds__(WAVES * 64, 2) void gqa_fresh_partition_kernel(
    int q_heads, int kv_heads, int context_length, float scale, const unsigned short *q, int q_stride,
    const unsigned short *k_cache, const unsigned short *v_cache, float *part_o, float *part_m, float *part_l,
    int splits, int group, FreshToken fresh)
{
    gqa_partition<true>(q_heads, kv_heads, context_length, nullptr, scale, q, q_stride, k_cache, v_cache, part_o,
                        part_m, part_l, splits, group, fresh);
}

// out[b, head, :] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s, partitions in index order.
// Only the partitions that hold positions of the sequence are read: the others were never written.
__global__ __launch_bounds__(DIM) void gqa_combine_kernel(int partitions, int q_heads, int context_length,
                                                          const int32_t *lengths, const int32_t *positions,
                                                          const float *part_o, const float *part_m,
                                                          const float *part_l, unsigned short *out)
{
    const size_t row = blockIdx.x; // b * q_heads + head
    const int d = threadIdx.x;
    const int b = int(row / q_heads);
    const int length = live_length(lengths, positions, b, context_length);
    const int splits = min(partitions, (length + CHUNK - 1) / CHUNK);
    // Partitions are taken eight at a time with all loads of a batch issued before any is used
    // (a loop of dependent scalar loads would pay the memory latency once per partition); indices
    // past the end are clamped and masked. The order of the sums is the partition order.
    constexpr int BATCH = 8;
    const float *row_m = part_m + row * partitions, *row_l = part_l + row * partitions;
    const float *row_o = part_o + row * partitions * DIM + d;
    float top = -INFINITY;
    for (int s0 = 0; s0 < splits; s0 += BATCH) {
        float l[BATCH], m[BATCH];
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
            const int s = s0 + i < splits ? s0 + i : splits - 1;
            l[i] = row_l[s];
            m[i] = row_m[s];
        }
#pragma unroll
        for (int i = 0; i < BATCH; ++i)
            if (s0 + i < splits && l[i] > 0.f)
                top = fmaxf(top, m[i]);
    }
    float numerator = 0.f, denominator = 0.f;
    for (int s0 = 0; s0 < splits; s0 += BATCH) {
        float l[BATCH], m[BATCH], o[BATCH];
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
            const int s = s0 + i < splits ? s0 + i : splits - 1;
            l[i] = row_l[s];
            m[i] = row_m[s];
            o[i] = row_o[size_t(s) * DIM];
        }
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
            if (s0 + i < splits && l[i] > 0.f) {
                const float factor = __expf(m[i] - top);
                numerator = fmaf(factor, o[i], numerator);
                denominator = fmaf(factor, l[i], denominator);
            }
        }
    }
    out[row * DIM + d] = float_to_bf16_bits(denominator > 0.f ? numerator / denominator : 0.f);
}
} // namespace

size_t gqa_decode_scratch_bytes(int batch, int q_heads, int dim, int context_length, int *splits)
{
    int count = (context_length + CHUNK - 1) / CHUNK;
    if (splits)
        *splits = count;
    size_t rows = size_t(batch) * q_heads * count;
    return rows * (size_t(dim) + 2) * sizeof(float);
}

hipError_t launch_rope_table(hipStream_t stream, int batch, int dim, float theta, const int32_t *positions, float *table)
{
    const int count = batch * (dim / 2);
    rope_table_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(batch, dim, theta, positions, table);
    return launch_status();
}

size_t gqa_resident_scratch_bytes() { return RESIDENT_BYTES; }

// Address of this device's copy of the fixed partials array. `device` must be the current device
// (every entry point runs under the context's device scope). Resolved once per device; later
// calls are one atomic load and touch no runtime API.
hipError_t gqa_resident_scratch(int device, void **address)
{
    *address = nullptr;
    if (device < 0 || device >= MAX_DEVICES)
        return hipErrorInvalidDevice;
    void *known = resident_address[device].load(std::memory_order_acquire);
    if (!known) {
        hipError_t status = hipGetSymbolAddress(&known, HIP_SYMBOL(scratch));
        if (status != hipSuccess) {
            (void)hipGetLastError();
            return status;
        }
        if (!known)
            return hipErrorInvalidSymbol;
        resident_address[device].store(known, std::memory_order_release);
    }
    *address = known;
    return hipSuccess;
}

hipError_t launch_gqa_decode(hipStream_t stream, int batch, int q_heads, int kv_heads, int dim,
                             int context_length, const int32_t *lengths, float scale, const void *q,
                             int q_stride, const void *k, const void *v, void *out, void *partials,
                             int splits, const int32_t *positions, float theta, const void *k_new,
                             const void *v_new, const float *table)
{
    const int group = kv_heads > 0 ? q_heads / kv_heads : 0;
    if (dim != DIM || splits > 65535 || kv_heads > 65535 || batch > 65535 || group < 1 ||
        group > HEADS)
        return hipErrorInvalidValue;
    size_t rows = size_t(batch) * q_heads * splits;
    float *part_o = static_cast<float *>(partials);
    float *part_m = part_o + rows * DIM;
    float *part_l = part_m + rows;
    dim3 grid(splits, kv_heads, batch);
    const unsigned short *qp = static_cast<const unsigned short *>(q);
    const unsigned short *kp = static_cast<const unsigned short *>(k);
    const unsigned short *vp = static_cast<const unsigned short *>(v);
    if (positions) {
        // the new token's rows come with the queries (token stride q_stride) and go into the caches
        const FreshToken fresh = {positions, theta, static_cast<const unsigned short *>(k_new),
                                  static_cast<const unsigned short *>(v_new), q_stride,
                                  const_cast<unsigned short *>(kp), const_cast<unsigned short *>(vp), table};
        gqa_fresh_partition_kernel<<<grid, WAVES * 64, 0, stream>>>(q_heads, kv_heads, context_length, scale, qp,
                                                                    q_stride, kp, vp, part_o, part_m, part_l, splits,
                                                                    group, fresh);
    } else {
        gqa_partition_kernel<<<grid, WAVES * 64, 0, stream>>>(q_heads, kv_heads, context_length, lengths, scale, qp,
                                                              q_stride, kp, vp, part_o, part_m, part_l, splits, group);
    }
    hipError_t status = launch_status();
    if (status != hipSuccess)
        return status;
    gqa_combine_kernel<<<unsigned(size_t(batch) * q_heads), DIM, 0, stream>>>(
        splits, q_heads, context_length, positions ? nullptr : lengths, positions, part_o, part_m, part_l,
        static_cast<unsigned short *>(out));
    return launch_status();
}
} // namespace camblas_hip
