// Bench equipment, built as libcamblas_probes.so beside the product library and loaded by bench.py
// only: nothing here is part of libcamblas_hip.so.
//
// Calibration launch for the matrix cores: every wavefront issues independent matrix instructions
// back to back, with no memory traffic, so the launch's duration gives the rate the part sustains
// for that instruction (its clock under matrix load included). No counterpart in the reference.
#include "device.hpp"

#include <hip/hip_runtime.h>

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

// KIND: 0 BF16 32x32x16, 1 E4M3 x E4M3 scaled 32x32x64, 2 E2M1 x E4M3 scaled 32x32x64, 3 FP32 32x32x2;
// 4 BF16 16x16x32, 5 E4M3 x E4M3 scaled 16x16x128, 6 E2M1 x E4M3 scaled 16x16x128 (narrow_probe_kernel)
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

// The 16 x 16 forms of the same instructions (four accumulator registers each): sixteen independent
// accumulators per wavefront, so that an instruction never waits for the previous one's result.
constexpr int NARROW_ACCUMULATORS = 16;
template <int KIND> __global__ __launch_bounds__(PROBE_THREADS) void narrow_probe_kernel(int rounds, int constant, float *sink)
{
    f32x4_t acc[NARROW_ACCUMULATORS];
#pragma unroll
    for (int t = 0; t < NARROW_ACCUMULATORS; ++t)
        acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    unsigned a_words[8], b_words[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a_words[i] = operand_word<KIND == 4 ? 0 : 1>(i, constant != 0);
        b_words[i] = operand_word<KIND == 4 ? 0 : 1>(i + 8, constant != 0);
    }
    for (int round = 0; round < rounds; ++round) {
#pragma unroll
        for (int t = 0; t < NARROW_ACCUMULATORS; ++t) {
            if constexpr (KIND == 4) {
                const bf16x8_t a = __builtin_bit_cast(bf16x8_t, u32x4_t{a_words[0], a_words[1], a_words[2], a_words[3]});
                const bf16x8_t b = __builtin_bit_cast(bf16x8_t, u32x4_t{b_words[0], b_words[1], b_words[2], b_words[3]});
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
            } else {
                const i32x8_t a = {int(a_words[0]), int(a_words[1]), int(a_words[2]), int(a_words[3]),
                                   int(a_words[4]), int(a_words[5]), int(a_words[6]), int(a_words[7])};
                const i32x8_t b = {int(b_words[0]), int(b_words[1]), int(b_words[2]), int(b_words[3]),
                                   int(b_words[4]), int(b_words[5]), int(b_words[6]), int(b_words[7])};
                acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[t], KIND == 6 ? 4 : 0, 0, 0, 127,
                                                                         0, 127);
            }
        }
    }
    f32x4_t sum = acc[0];
#pragma unroll
    for (int t = 1; t < NARROW_ACCUMULATORS; ++t)
        sum = sum + acc[t];
    sink[blockIdx.x * PROBE_THREADS + threadIdx.x] = sum[0] + sum[1] + sum[2] + sum[3];
}
} // namespace

// One workgroup of `threads` / 64 wavefronts per compute unit (512: two wavefronts per SIMD, 256: one);
// each wavefront issues rounds * 8 (kinds 0 to 3) or rounds * 16 (kinds 4 to 6) instructions.
// sink receives workgroups * 512 floats. Returns the floating-point operations of the launch in
// *flops (0 for an unknown kind).
hipError_t launch_matrix_probe(hipStream_t stream, int kind, int workgroups, int rounds, int constant,
                               float *sink, double *flops, int threads)
{
    const double per_instruction[] = {2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 64, 2.0 * 32 * 32 * 64, 2.0 * 32 * 32 * 2,
                                      2.0 * 16 * 16 * 32, 2.0 * 16 * 16 * 128, 2.0 * 16 * 16 * 128};
    *flops = 0;
    switch (kind) {
    case 0: matrix_probe_kernel<0><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    case 1: matrix_probe_kernel<1><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    case 2: matrix_probe_kernel<2><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    case 3: matrix_probe_kernel<3><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    case 4: narrow_probe_kernel<4><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    case 5: narrow_probe_kernel<5><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    case 6: narrow_probe_kernel<6><<<workgroups, threads, 0, stream>>>(rounds, constant, sink); break;
    default: return hipErrorInvalidValue;
    }
    *flops = per_instruction[kind] * double(workgroups) * (threads / 64) * double(rounds) *
             (kind >= 4 ? NARROW_ACCUMULATORS : PROBE_ACCUMULATORS);
    return hipGetLastError();
}

// Plain 16-byte-per-thread copy: a launch of known HBM traffic (bytes read + bytes written)
// against which the hardware byte counters are calibrated.
namespace
{
__global__ void copy_probe_kernel(size_t vectors, const u32x4_t *source, u32x4_t *destination)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < vectors;
         index += size_t(gridDim.x) * blockDim.x)
        destination[index] = source[index];
}
} // namespace
} // namespace camblas_hip

// stream: a raw hipStream_t. Both return 0 or a negative hipError_t.
extern "C" int camblas_probe_copy(void *stream, size_t bytes, const void *source, void *destination)
{
    using namespace camblas_hip;
    if (bytes % 16 || !source || !destination || reinterpret_cast<uintptr_t>(source) % 16 ||
        reinterpret_cast<uintptr_t>(destination) % 16)
        return -int(hipErrorInvalidValue);
    if (!bytes)
        return 0;
    copy_probe_kernel<<<2048, 256, 0, static_cast<hipStream_t>(stream)>>>(
        bytes / 16, static_cast<const u32x4_t *>(source), static_cast<u32x4_t *>(destination));
    return -int(hipGetLastError());
}

// kind 0 BF16 32x32x16, 1 E4M3 x E4M3 and 2 E2M1 x E4M3 scaled 32x32x64, 3 FP32 32x32x2, 4 BF16
// 16x16x32, 5 E4M3 x E4M3 and 6 E2M1 x E4M3 scaled 16x16x128; one workgroup of eight wavefronts per
// entry of `workgroups`, each wavefront issuing rounds * 8 (kinds 4 to 6: rounds * 16) independent
// matrix instructions. sink (device) receives workgroups * 512 floats; *flops (host) the
// floating-point operations of the launch.
extern "C" int camblas_probe_matrix(void *stream, int kind, int workgroups, int rounds, int constant_operands,
                                    void *sink, size_t sink_bytes, double *flops)
{
    if (kind < 0 || kind > 6 || workgroups < 1 || rounds < 1 || !sink || !flops ||
        reinterpret_cast<uintptr_t>(sink) % 4 || sink_bytes < size_t(workgroups) * 512 * sizeof(float))
        return -int(hipErrorInvalidValue);
    return -int(camblas_hip::launch_matrix_probe(static_cast<hipStream_t>(stream), kind, workgroups, rounds,
                                                 constant_operands != 0, static_cast<float *>(sink), flops, 512));
}

// The same with four wavefronts per workgroup: one wavefront per SIMD, the occupancy of the
// four-wavefront prefill tiles.
extern "C" int camblas_probe_matrix_single(void *stream, int kind, int workgroups, int rounds, int constant_operands,
                                           void *sink, size_t sink_bytes, double *flops)
{
    if (kind < 0 || kind > 6 || workgroups < 1 || rounds < 1 || !sink || !flops ||
        reinterpret_cast<uintptr_t>(sink) % 4 || sink_bytes < size_t(workgroups) * 512 * sizeof(float))
        return -int(hipErrorInvalidValue);
    return -int(camblas_hip::launch_matrix_probe(static_cast<hipStream_t>(stream), kind, workgroups, rounds,
                                                 constant_operands != 0, static_cast<float *>(sink), flops, 256));
}
