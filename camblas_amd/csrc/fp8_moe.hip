// One token through a block-scaled FP8 mixture-of-experts layer: for every chosen expert the gate/up
// product, the clipped SiLU-multiply, the down product, and the routed sum over the experts.
// Arithmetic rule (ref: camblas/_hopper.py:13-126 `_products`, :129-182 `_reduce`, :267-326
// `_combine`, :329-401 `fused`):
//   x is quantised per 128 inputs (scale = max(|x|, 1e-10) / 448, values clamped to +-448, E4M3);
//   up[c][n]  = bf16( sum_g fma(dot_g, x_scale[g] * w1_scale[e_c][n/128][g], .) ), dot_g the unscaled
//               FP32 dot product of one 128-input group on the matrix cores;
//   act[c][i] = bf16( silu(min(gate, 10)) * clamp(up, -10, 10) ), gate = up[c][i], up = up[c][H + i];
//   act is quantised per 128 like x, per expert choice;
//   down[c][n] = sum_g fma(dot_g, act_scale[c][g] * w2_scale[e_c][n/128][g], .);
//   out[n] = bf16( factor * sum_c f32(bf16(down[c][n] * routing[c])) ), c ascending.
//
// Two launches. The matrix instruction (v_mfma_scale_f32_16x16x128_f8f6f4 with unit scales) takes
// 16 weight rows against the token's group in every column; a lane group c = lane/16 supplies K
// positions 16c..16c+15 and 64+16c..64+16c+15 of the group for both operands. A group's 128 values
// are activated and quantised two per lane (one wavefront reduction for the maximum), written as
// 128 bytes to a patch of LDS private to the wavefront and read back in the operand layout (LDS
// operations of one wavefront execute in order: no barrier). Kernel one: a workgroup owns eight
// gate rows of one choice and the up rows of the same indices, its eight wavefronts take the K
// groups in turn (each quantises the groups it multiplies), their partial sums are added in
// wavefront order and the activation is applied once per value. Kernel two: a workgroup owns 16
// output rows for all choices; the (choice, group) pairs go round the wavefronts, each quantising
// the pair's 128 activated values itself, and 16 lanes then do the ordered scaling, routing and
// summing.
#include "common.hpp"
#include "device.hpp"
#include "dma.hpp"

namespace camblas_hip
{
namespace
{
// (eight wavefronts: a call is short and bound by memory latency, so every wavefront should have
// all its loads in flight at once: 32 groups / 8 = 4 for the reference's gate/up shape, 36 pairs / 8 <= 5)
constexpr int MOE_THREADS = 512, MOE_WAVES = 8, MOE_ROWS = 16, UP_DEPTH = 4, DOWN_DEPTH = 5;
constexpr int UNIT_SCALE = 0x7f7f7f7f;

struct MoeParams {
    const unsigned short *x;  // [hidden] BF16
    const unsigned char *w1;  // [experts, 2 * width, hidden] E4M3
    const float *s1;          // [experts, 2 * width / 128, hidden / 128]
    const unsigned char *w2;  // [experts, hidden_out, width] E4M3
    const float *s2;          // [experts, ceil(hidden_out / 128), width / 128]
    const int32_t *ids;       // [choices]
    const float *routing;     // [choices]
    unsigned short *act;      // [choices, width] BF16, activated (scratch between the launches)
    unsigned short *out;      // [hidden_out] BF16
    int experts, choices, hidden, width, hidden_out;
    float factor;
};

// A wavefront's step is 16 weight rows x 128 bytes. Loading them straight in the operand layout
// (lane -> row lane%16) would touch every 128-byte line from four quarter-wave passes; instead
// eight lanes read one whole line (rows lane/8 and 8 + lane/8), and the tile is transposed to the
// operand layout through a swizzled LDS tile private to the wavefront.
__device__ __forceinline__ void load_weight_lines(const unsigned char *rows, size_t pitch, int lane,
                                                  u32x4_t (&w)[2])
{
    const unsigned char *source = rows + size_t(lane / 8) * pitch + (lane % 8) * 16;
    w[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(source));
    w[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(source + 8 * pitch));
}

// tile: 16 rows x 8 chunks of 16 bytes; returns the operand of lane (row lane%16, lane group
// `piece`): chunks piece and 4 + piece of its row
__device__ __forceinline__ i32x8_t transpose_weights(const u32x4_t (&w)[2], u32x4_t *tile, int lane, int piece)
{
    const int load_row = lane / 8, chunk = lane % 8, row = lane % 16;
    tile[load_row * 8 + (chunk ^ lds_swizzle<8>(load_row))] = w[0];
    tile[(load_row + 8) * 8 + (chunk ^ lds_swizzle<8>(load_row + 8))] = w[1];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const u32x4_t lo = tile[row * 8 + (piece ^ lds_swizzle<8>(row))];
    const u32x4_t hi = tile[row * 8 + ((4 + piece) ^ lds_swizzle<8>(row))];
    // the tile is overwritten by the next step: order these reads before that store
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]), int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
}

__device__ __forceinline__ i32x8_t operand(const u32x4_t &lo, const u32x4_t &hi)
{
    return i32x8_t{int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]), int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
}

// Quantise one 128-value group, lane l holding values 2l and 2l+1, and return the group as the
// instruction's token operand (the same in every column) together with its scale
// (ref: camblas/_hopper.py:82-98). `patch` is 128 bytes of LDS private to the wavefront.
__device__ __forceinline__ i32x8_t quantise_group(float v0, float v1, unsigned char *patch, int lane,
                                                  int piece, float &scale)
{
    const float amax = wave_max(fmaxf(1e-10f, fmaxf(fabsf(v0), fabsf(v1))));
    const float inv = 448.0f / amax;
    const unsigned codes = f32x2_to_e4m3_sat(v0 * inv, v1 * inv);
    reinterpret_cast<unsigned short *>(patch)[lane] = static_cast<unsigned short>(codes);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const u32x4_t lo = *reinterpret_cast<const u32x4_t *>(patch + piece * 16);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t *>(patch + 64 + piece * 16);
    // the patch is overwritten by the next group: order these reads before that store
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    scale = amax * (1.0f / 448.0f);
    return operand(lo, hi);
}

__device__ __forceinline__ int chosen_expert(const MoeParams &p, int choice)
{
    const int expert = p.ids[choice];
    return expert < 0 ? 0 : expert >= p.experts ? p.experts - 1 : expert; // (validated by the caller's router)
}

// Everything one group's step needs from memory, requested a few steps ahead. Steps past a
// wavefront's last group repeat that group with a zero scale, so that no load sits under a branch.
struct UpAhead {
    u32x4_t weight[2];
    unsigned pair;
    float gate_scale, up_scale;
};

// act[c][i0 .. i0+7] for choice c = blockIdx.y: the workgroup's 16 rows are gate rows i0..i0+7 and
// the up rows of the same indices, so the clipped SiLU-multiply is applied here, once per value
__global__ __launch_bounds__(MOE_THREADS) void moe_up_kernel(MoeParams p)
{
    __shared__ float parked[MOE_WAVES][MOE_ROWS];
    __shared__ __attribute__((aligned(16))) unsigned char patches[MOE_WAVES][128];
    __shared__ u32x4_t tiles[MOE_WAVES][MOE_ROWS * 8];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int row = lane % 16, piece = lane / 16;
    const int i0 = blockIdx.x * (MOE_ROWS / 2), choice = blockIdx.y;
    const int groups = p.hidden / 128;
    const int expert = chosen_expert(p, choice);
    // rows lane/8 of the first load are gate rows, of the second load the matching up rows
    const unsigned char *weights = p.w1 + (size_t(expert) * 2 * p.width + i0) * p.hidden;
    const size_t up_rows = size_t(p.width) * p.hidden;
    const float *gate_scale = p.s1 + (size_t(expert) * (2 * p.width / 128) + i0 / 128) * groups;
    const float *up_scale = gate_scale + size_t(p.width / 128) * groups;

    // this wavefront's groups: wave, wave + 8, ...
    const int mine = (groups - wave + MOE_WAVES - 1) / MOE_WAVES;
    auto fetch = [&](int ordinal, UpAhead &slot) {
        const int clamped = ordinal < mine ? ordinal : (mine > 0 ? mine - 1 : 0);
        int g = wave + MOE_WAVES * clamped;
        g = g < groups ? g : 0;
        const unsigned char *source = weights + size_t(lane / 8) * p.hidden + size_t(g) * 128 + (lane % 8) * 16;
        slot.weight[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(source));
        slot.weight[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(source + up_rows));
        slot.pair = reinterpret_cast<const unsigned *>(p.x + size_t(g) * 128)[lane];
        slot.gate_scale = gate_scale[g];
        slot.up_scale = up_scale[g];
    };
    UpAhead ahead[UP_DEPTH];
#pragma unroll
    for (int d = 0; d < UP_DEPTH; ++d)
        fetch(d, ahead[d]);
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int step = 0; step < mine; step += UP_DEPTH) {
#pragma unroll
        for (int d = 0; d < UP_DEPTH; ++d) {
            const UpAhead &now = ahead[d];
            float scale;
            const i32x8_t b = quantise_group(__uint_as_float(now.pair << 16), __uint_as_float(now.pair & 0xffff0000u),
                                             patches[wave], lane, piece, scale);
            f32x4_t dot = {0.f, 0.f, 0.f, 0.f};
            const i32x8_t a = transpose_weights(now.weight, tiles[wave], lane, piece);
            dot = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, dot, 0, 0, 0, UNIT_SCALE, 0, UNIT_SCALE);
            // accumulator rows 0..7 (lane groups 0 and 1) are gate rows, 8..15 up rows
            const float block = piece < 2 ? now.gate_scale : now.up_scale;
            const float s = step + d < mine ? __fmul_rn(scale, block) : 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                acc[r] = fmaf(dot[r], s, acc[r]);
            // the slot is refilled only after its last use, so that the loads can land in the same
            // registers (loads hoisted above the uses would need copies at the end of the loop,
            // and the copies would wait for every load in flight)
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + d + UP_DEPTH, ahead[d]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // accumulator element r of lane l is row 4*(l/16) + r (every column holds the same token)
    if (row == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            parked[wave][4 * piece + r] = acc[r];
    }
    __syncthreads();
    if (threadIdx.x < MOE_ROWS / 2) {
        float gate = 0.f, up = 0.f;
#pragma unroll
        for (int w = 0; w < MOE_WAVES; ++w) {
            gate += parked[w][threadIdx.x];
            up += parked[w][MOE_ROWS / 2 + threadIdx.x];
        }
        // both products are rounded to BF16, then the clipped SiLU-multiply, rounded to BF16
        // (ref: camblas/_hopper.py:65-80 and :183)
        gate = fminf(bf16_bits_to_float(float_to_bf16_bits(gate)), 10.0f);
        up = fminf(fmaxf(bf16_bits_to_float(float_to_bf16_bits(up)), -10.0f), 10.0f);
        p.act[size_t(choice) * p.width + i0 + threadIdx.x] =
            float_to_bf16_bits(gate / (1.0f + __expf(-gate)) * up);
    }
}

struct DownAhead {
    u32x4_t weight[2];
    unsigned pair;
    float block_scale;
};

// out[n0 .. n0+15]: the down products of every choice, routed and summed
__global__ __launch_bounds__(MOE_THREADS) void moe_down_kernel(MoeParams p)
{
    extern __shared__ float terms[]; // [pairs][16] unscaled dots, then [pairs] scale products
    __shared__ __attribute__((aligned(16))) unsigned char patches[MOE_WAVES][128];
    __shared__ u32x4_t tiles[MOE_WAVES][MOE_ROWS * 8];
    __shared__ int expert_of[16];
    __shared__ float routing_of[16];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int row = lane % 16, piece = lane / 16;
    const int n0 = blockIdx.x * MOE_ROWS;
    const int groups = p.width / 128, pairs = p.choices * groups;
    float *scales = terms + size_t(pairs) * MOE_ROWS;
    const int block_rows = (p.hidden_out + 127) / 128;
    if (threadIdx.x < 16) {
        const int choice = threadIdx.x < p.choices ? threadIdx.x : 0;
        expert_of[threadIdx.x] = chosen_expert(p, choice);
        routing_of[threadIdx.x] = p.routing[choice];
    }
    __syncthreads();

    // this wavefront's (choice, group) pairs: wave, wave + 8, ...; the activated values of pair
    // (c, g) are act[c * width + g * 128 ..), i.e. pair * 128 onwards
    const int mine = (pairs - wave + MOE_WAVES - 1) / MOE_WAVES;
    auto pair_of = [&](int ordinal) {
        const int clamped = ordinal < mine ? ordinal : (mine > 0 ? mine - 1 : 0);
        const int pair = wave + MOE_WAVES * clamped;
        return pair < pairs ? pair : 0;
    };
    auto fetch = [&](int ordinal, DownAhead &slot) {
        const int pair = pair_of(ordinal), choice = pair / groups, g = pair - choice * groups;
        const int expert = expert_of[choice];
        load_weight_lines(p.w2 + (size_t(expert) * p.hidden_out + n0) * p.width + size_t(g) * 128,
                          size_t(p.width), lane, slot.weight);
        slot.pair = reinterpret_cast<const unsigned *>(p.act + size_t(pair) * 128)[lane];
        slot.block_scale = p.s2[(size_t(expert) * block_rows + n0 / 128) * groups + g];
    };
    DownAhead ahead[DOWN_DEPTH];
#pragma unroll
    for (int d = 0; d < DOWN_DEPTH; ++d)
        fetch(d, ahead[d]);
    for (int step = 0; step < mine; step += DOWN_DEPTH) {
#pragma unroll
        for (int d = 0; d < DOWN_DEPTH; ++d) {
            const DownAhead &now = ahead[d];
            const int pair = pair_of(step + d);
            float scale;
            const i32x8_t b = quantise_group(__uint_as_float(now.pair << 16), __uint_as_float(now.pair & 0xffff0000u),
                                             patches[wave], lane, piece, scale);
            f32x4_t dot = {0.f, 0.f, 0.f, 0.f};
            const i32x8_t a = transpose_weights(now.weight, tiles[wave], lane, piece);
            dot = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, dot, 0, 0, 0, UNIT_SCALE, 0, UNIT_SCALE);
            // (a repeated last pair writes the same values again)
            if (row == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    terms[size_t(pair) * MOE_ROWS + 4 * piece + r] = dot[r];
                if (piece == 0)
                    scales[pair] = __fmul_rn(scale, now.block_scale);
            }
            __builtin_amdgcn_sched_barrier(0); // (refill after the last use, as above)
            fetch(step + d + DOWN_DEPTH, ahead[d]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();
    if (threadIdx.x < MOE_ROWS) {
        float total = 0.f;
        for (int choice = 0; choice < p.choices; ++choice) {
            float acc = 0.f;
            for (int g = 0; g < groups; ++g) {
                const int pair = choice * groups + g;
                acc = fmaf(terms[size_t(pair) * MOE_ROWS + threadIdx.x], scales[pair], acc);
            }
            total += bf16_bits_to_float(float_to_bf16_bits(acc * routing_of[choice]));
        }
        p.out[n0 + threadIdx.x] = float_to_bf16_bits(total * p.factor);
    }
}
} // namespace

size_t fp8_moe_decode_scratch_bytes(int choices, int width) { return size_t(choices) * width * 2; }

// hidden and width multiples of 128, hidden_out of 16, choices 1..16, 16-byte aligned x, w1, w2;
// scratch holds choices * width BF16 values.
hipError_t launch_fp8_moe_decode(hipStream_t stream, int experts, int choices, int hidden, int width,
                                 int hidden_out, const void *x, const void *w1, const float *s1,
                                 const void *w2, const float *s2, const int32_t *ids,
                                 const float *routing, float factor, void *scratch, void *out)
{
    if (experts < 1 || choices < 1 || choices > 16 || hidden < 128 || hidden % 128 || width < 128 ||
        width % 128 || hidden_out < 16 || hidden_out % 16)
        return hipErrorInvalidValue;
    MoeParams p;
    p.x = static_cast<const unsigned short *>(x);
    p.w1 = static_cast<const unsigned char *>(w1);
    p.s1 = s1;
    p.w2 = static_cast<const unsigned char *>(w2);
    p.s2 = s2;
    p.ids = ids;
    p.routing = routing;
    p.act = static_cast<unsigned short *>(scratch);
    p.out = static_cast<unsigned short *>(out);
    p.experts = experts;
    p.choices = choices;
    p.hidden = hidden;
    p.width = width;
    p.hidden_out = hidden_out;
    p.factor = factor;
    dim3 up_grid(unsigned(width / (MOE_ROWS / 2)), unsigned(choices));
    moe_up_kernel<<<up_grid, MOE_THREADS, 0, stream>>>(p);
    hipError_t error = launch_status();
    if (error != hipSuccess)
        return error;
    const int pairs = choices * (width / 128);
    // dynamic LDS beside 18 KB of static LDS, inside the 64 KB a launch gets without asking for more
    const size_t lds = size_t(pairs) * (MOE_ROWS + 1) * sizeof(float);
    if (pairs > 512)
        return hipErrorInvalidValue;
    moe_down_kernel<<<unsigned(hidden_out / MOE_ROWS), MOE_THREADS, lds, stream>>>(p);
    return launch_status();
}
} // namespace camblas_hip
