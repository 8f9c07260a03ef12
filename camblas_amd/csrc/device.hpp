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

// FP32 -> E4M3fn, round-to-nearest-even, saturating at +-448, NaN -> 0x7f: the conversion
// instruction of gfx950 (OCP formats) after a clamp; the comparisons of the clamp keep NaN.
__device__ __forceinline__ unsigned f32_to_e4m3_sat(float value)
{
    const float clamped = value > 448.f ? 448.f : value < -448.f ? -448.f : value;
    const unsigned code = unsigned(__builtin_amdgcn_cvt_pk_fp8_f32(clamped, clamped, 0, false)) & 0xffu;
    return (code & 0x7fu) == 0x7fu ? 0x7fu : code;
}

// two values at once: low byte from `first`, next byte from `second`
__device__ __forceinline__ unsigned f32x2_to_e4m3_sat(float first, float second)
{
    const float a = first > 448.f ? 448.f : first < -448.f ? -448.f : first;
    const float b = second > 448.f ? 448.f : second < -448.f ? -448.f : second;
    unsigned codes = unsigned(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false)) & 0xffffu;
    if ((codes & 0x7fu) == 0x7fu)
        codes &= 0xff7fu;
    if ((codes & 0x7f00u) == 0x7f00u)
        codes &= 0x7fffu;
    return codes;
}

// Rotary embedding, rotate-half pairing (i, i + dim/2): angle = position * theta^(-2i/dim) with FP32
// sine and cosine, one BF16 rounding per element. Shared by every kernel that rotates, so that they
// agree bit for bit.
__device__ __forceinline__ void pair_sincos(float position, int i, int dim, float theta, float &s, float &c)
{
    float frequency = exp2f(-2.f * float(i) / float(dim) * log2f(theta));
    float angle = position * frequency;
    sincosf(angle, &s, &c);
}
__device__ __forceinline__ void rotate_by(float s, float c, float lo, float hi, unsigned short &out_lo,
                                          unsigned short &out_hi)
{
    // (written out so that every kernel rounds in the same places whatever the compiler would contract;
    // the two roundings to BF16 are one conversion instruction of gfx950, round to nearest even)
    typedef float pair_f32 __attribute__((ext_vector_type(2)));
    typedef __bf16 pair_bf16 __attribute__((ext_vector_type(2)));
    const pair_f32 rotated = {__fmaf_rn(lo, c, -__fmul_rn(hi, s)), __fmaf_rn(hi, c, __fmul_rn(lo, s))};
    const unsigned packed = __builtin_bit_cast(unsigned, __builtin_convertvector(rotated, pair_bf16));
    out_lo = (unsigned short)(packed & 0xffffu);
    out_hi = (unsigned short)(packed >> 16);
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

// Cross-lane moves inside the vector ALU (DPP), no LDS traffic. CONTROL: 0xB1 swaps neighbours
// (lane ^ 1), 0x4E swaps pairs (lane ^ 2), 0x141 mirrors each group of 8, 0x140 mirrors each row of
// 16 lanes.
template <int CONTROL> __device__ __forceinline__ float dpp_move(float value)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), CONTROL, 0xf, 0xf, true));
}

// Sum over each aligned group of 16 lanes; every lane of the group receives the total. Fixed order:
// neighbours, pairs, then the two mirrored halves.
__device__ __forceinline__ float row16_sum(float value)
{
    value += dpp_move<0xB1>(value);
    value += dpp_move<0x4E>(value);
    value += dpp_move<0x141>(value);
    value += dpp_move<0x140>(value);
    return value;
}

__device__ __forceinline__ float row16_max(float value)
{
    value = fmaxf(value, dpp_move<0xB1>(value));
    value = fmaxf(value, dpp_move<0x4E>(value));
    value = fmaxf(value, dpp_move<0x141>(value));
    value = fmaxf(value, dpp_move<0x140>(value));
    return value;
}

__device__ __forceinline__ float lane_value(float value, int lane)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, value), lane));
}

// Sum across the 64 lanes of a wavefront in a fixed order; every lane receives the total.
__device__ __forceinline__ float wave_sum(float value)
{
    value = row16_sum(value);
    return (lane_value(value, 0) + lane_value(value, 16)) +
           (lane_value(value, 32) + lane_value(value, 48));
}

__device__ __forceinline__ float wave_max(float value)
{
    value = row16_max(value);
    return fmaxf(fmaxf(lane_value(value, 0), lane_value(value, 16)),
                 fmaxf(lane_value(value, 32), lane_value(value, 48)));
}
// Tile of a lower-triangle launch: workgroup t of a one-dimensional grid owns column tile j of row
// tile i, the tiles of a row (those that reach the diagonal: (i + 1) * TILE / COLUMNS of them)
// numbered before those of the next row. Returns false for a tile beyond the last column.
template <int TILE_ROWS, int TILE_COLUMNS>
__device__ __forceinline__ bool lower_tile(unsigned t, int n, int &row0, int &col0)
{
    constexpr unsigned PER_ROW = TILE_ROWS / TILE_COLUMNS; // column tiles added by every row tile
    int i = int((sqrtf(8.f * float(t / PER_ROW) + 1.f) - 1.f) * 0.5f);
    while (PER_ROW * unsigned(i + 1) * unsigned(i + 2) / 2 <= t)
        ++i;
    while (PER_ROW * unsigned(i) * unsigned(i + 1) / 2 > t)
        --i;
    row0 = i * TILE_ROWS;
    col0 = int(t - PER_ROW * unsigned(i) * unsigned(i + 1) / 2) * TILE_COLUMNS;
    return col0 < n;
}

// workgroups of a lower-triangle launch over an n x n output
template <int TILE_ROWS, int TILE_COLUMNS> inline unsigned lower_tile_count(int n)
{
    const unsigned rows = unsigned((n + TILE_ROWS - 1) / TILE_ROWS);
    return TILE_ROWS / TILE_COLUMNS * rows * (rows + 1) / 2;
}
} // namespace camblas_hip
