// Device-side helpers shared by the gfx950 kernels: vector types, BF16/E4M3 conversion, wave-64
// reductions.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace camblas_hip
{
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_bits_to_float(unsigned short bits)
{
    return __uint_as_float(unsigned(bits) << 16);
}

// Round-to-nearest-even FP32 -> BF16 bit pattern; NaN stays a quiet NaN.
__device__ __forceinline__ unsigned short float_to_bf16_bits(float value)
{
    unsigned bits = __float_as_uint(value);
    if ((bits & 0x7fffffffu) > 0x7f800000u)
        return (unsigned short)((bits >> 16) | 0x0040u);
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (unsigned short)(bits >> 16);
}

__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi)
{
    return unsigned(float_to_bf16_bits(lo)) | (unsigned(float_to_bf16_bits(hi)) << 16);
}

// Storage traits: T is float, double or bf16_storage (a 16-bit wrapper).
struct bf16_storage {
    unsigned short bits;
};

template <typename T> struct storage;
template <> struct storage<float> {
    using accumulator = float;
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
    static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct storage<double> {
    using accumulator = double;
    static __device__ __forceinline__ double load(const double *p) { return *p; }
    static __device__ __forceinline__ void store(double *p, double v) { *p = v; }
    static __device__ __forceinline__ double round(double v) { return v; }
};
template <> struct storage<bf16_storage> {
    using accumulator = float;
    static __device__ __forceinline__ float load(const bf16_storage *p)
    {
        return bf16_bits_to_float(p->bits);
    }
    static __device__ __forceinline__ void store(bf16_storage *p, float v)
    {
        p->bits = float_to_bf16_bits(v);
    }
    static __device__ __forceinline__ float round(float v)
    {
        return bf16_bits_to_float(float_to_bf16_bits(v));
    }
};

// Sum across the 64 lanes of a wavefront in a fixed order; every lane receives the total.
__device__ __forceinline__ float wave_sum(float value)
{
#pragma unroll
    for (int offset = 32; offset; offset >>= 1)
        value += __shfl_xor(value, offset, 64);
    return value;
}

__device__ __forceinline__ float wave_max(float value)
{
#pragma unroll
    for (int offset = 32; offset; offset >>= 1)
        value = fmaxf(value, __shfl_xor(value, offset, 64));
    return value;
}
} // namespace camblas_hip
