// Calibration launch for the matrix cores: every wavefront issues independent matrix instructions
// back to back, with no memory traffic, so the launch's duration gives the rate the part sustains
// for that instruction (its clock under matrix load included). No counterpart in the reference.
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int PROBE_THREADS = 512, PROBE_ACCUMULATORS = 8;

// Per-lane operand words: the value 1 in every element (constant), or a multiplicative hash shaped
// into finite values of either sign with random mantissas and eight different exponents: BF16 and
// FP32 magnitudes in [2^-7, 2), E4M3 below 2 (which also covers every E2M1 nibble). The sustained
// rate depends on how many operand bits toggle, so the hash stands in for real activations.
template <int KIND> __device__ __forceinline__ unsigned operand_word(int index, bool constant)
{
    const unsigned hash = (threadIdx.x * 2654435761u + unsigned(index) * 0x9E3779B9u) >> 5;
    if (KIND == 0)
        return constant ? 0x3f803f80u : (hash & 0x83ff83ffu) | 0x3c003c00u;
    if (KIND == 3)
        return constant ? 0x3f800000u : (hash & 0x83ffffffu) | 0x3c000000u;
    return constant ? 0x38383838u : hash & 0xbfbfbfbfu;
}

// KIND: 0 BF16 32x32x16, 1 E4M3 x E4M3 scaled 32x32x64, 2 E2M1 x E4M3 scaled 32x32x64, 3 FP32 32x32x2
template <int KIND> __global__ __launch_bounds__(PROBE_THREADS) void matrix_probe_kernel(int rounds, int constant, float *sink)
{
    f32x16_t acc[PROBE_ACCUMULATORS];
#pragma unroll
    for (int t = 0; t < PROBE_ACCUMULATORS; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[t][r] = 0.f;
    unsigned a_words[8], b_words[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a_words[i] = operand_word<KIND>(i, constant != 0);
        b_words[i] = operand_word<KIND>(i + 8, constant != 0);
    }
    for (int round = 0; round < rounds; ++round) {
#pragma unroll
        for (int t = 0; t < PROBE_ACCUMULATORS; ++t) {
            if constexpr (KIND == 0) {
                const bf16x8_t a = __builtin_bit_cast(bf16x8_t, u32x4_t{a_words[0], a_words[1], a_words[2], a_words[3]});
                const bf16x8_t b = __builtin_bit_cast(bf16x8_t, u32x4_t{b_words[0], b_words[1], b_words[2], b_words[3]});
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
            } else if constexpr (KIND == 3) {
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a_words[0]),
                                                              __builtin_bit_cast(float, b_words[0]), acc[t], 0, 0, 0);
            } else {
                const i32x8_t a = {int(a_words[0]), int(a_words[1]), int(a_words[2]), int(a_words[3]),
                                   int(a_words[4]), int(a_words[5]), int(a_words[6]), int(a_words[7])};
                const i32x8_t b = {int(b_words[0]), int(b_words[1]), int(b_words[2]), int(b_words[3]),
                                   int(b_words[4]), int(b_words[5]), int(b_words[6]), int(b_words[7])};
                acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[t], KIND == 2 ? 4 : 0, 0, 0, 127,
                                                                        0, 127);
            }
        }
    }
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < PROBE_ACCUMULATORS; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            sum += acc[t][r];
    sink[blockIdx.x * PROBE_THREADS + threadIdx.x] = sum;
}
} // namespace

// One workgroup of eight wavefronts per compute unit; each wavefront issues rounds * 8 instructions.
// sink receives workgroups * 512 floats. Returns the floating-point operations of the launch in
// *flops (0 for an unknown kind).
hipError_t launch_matrix_probe(hipStream_t stream, int kind, int workgroups, int rounds, int constant,
                               float *sink, double *flops)
{
    const double per_instruction[] = {2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 64, 2.0 * 32 * 32 * 64, 2.0 * 32 * 32 * 2};
    *flops = 0;
    switch (kind) {
    case 0: matrix_probe_kernel<0><<<workgroups, PROBE_THREADS, 0, stream>>>(rounds, constant, sink); break;
    case 1: matrix_probe_kernel<1><<<workgroups, PROBE_THREADS, 0, stream>>>(rounds, constant, sink); break;
    case 2: matrix_probe_kernel<2><<<workgroups, PROBE_THREADS, 0, stream>>>(rounds, constant, sink); break;
    case 3: matrix_probe_kernel<3><<<workgroups, PROBE_THREADS, 0, stream>>>(rounds, constant, sink); break;
    default: return hipErrorInvalidValue;
    }
    *flops = per_instruction[kind] * double(workgroups) * (PROBE_THREADS / 64) * double(rounds) * PROBE_ACCUMULATORS;
    return launch_status();
}
} // namespace camblas_hip
