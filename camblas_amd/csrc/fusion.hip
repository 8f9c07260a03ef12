// Decode-layer epilogues: SiLU*up, SwiGLU, RMS normalisation (optionally fused with the residual
// add, any number of rows), BF16 squares, RMS scaling and rotary embedding. All are bandwidth or
// latency bound; they use 128-bit accesses where the row layout allows and FP32 arithmetic with
// the storage roundings of the reference (src/cuda/inference_fusion.cuh:19-207).
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
// ---------------------------------------------------------------- SiLU(gate) * up
// round_T(g / (1 + exp(-g))) then round_T(that * u)   (ref: inference_fusion.cuh:19-28)
template <typename T>
__global__ void silu_multiply_kernel(size_t count, const T *gate, const T *up, T *out)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < count;
         index += size_t(gridDim.x) * blockDim.x) {
        float g = storage<T>::load(gate + index);
        float activated = storage<T>::round(g / (1.f + expf(-g)));
        storage<T>::store(out + index, __fmul_rn(activated, storage<T>::load(up + index)));
    }
}

// Eight BF16 per thread per step; same arithmetic.
__global__ void silu_multiply_bf16x8_kernel(size_t vectors, const u32x4_t *gate, const u32x4_t *up,
                                            u32x4_t *out)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < vectors;
         index += size_t(gridDim.x) * blockDim.x) {
        u32x4_t g = gate[index], u = up[index], r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float g0 = __uint_as_float(g[e] << 16), g1 = __uint_as_float(g[e] & 0xffff0000u);
            float u0 = __uint_as_float(u[e] << 16), u1 = __uint_as_float(u[e] & 0xffff0000u);
            float a0 = bf16_bits_to_float(float_to_bf16_bits(g0 / (1.f + expf(-g0))));
            float a1 = bf16_bits_to_float(float_to_bf16_bits(g1 / (1.f + expf(-g1))));
            r[e] = pack_bf16x2(__fmul_rn(a0, u0), __fmul_rn(a1, u1));
        }
        out[index] = r;
    }
}

// ---------------------------------------------------------------- SwiGLU
// optional clamp with NaN-preserving compares, FP32 silu(g)*u, optional per-row routing factor,
// one final rounding (ref: inference_fusion.cuh:30-51)
template <typename T>
__global__ void swiglu_kernel(size_t count, int width, float limit, const T *gate, const T *up,
                              const float *routing, T *out)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < count;
         index += size_t(gridDim.x) * blockDim.x) {
        float g = storage<T>::load(gate + index), u = storage<T>::load(up + index);
        if (limit > 0) {
            if (g > limit)
                g = limit;
            if (u > limit)
                u = limit;
            if (u < -limit)
                u = -limit;
        }
        float value = __fmul_rn(g / (1.f + expf(-g)), u);
        if (routing)
            value = __fmul_rn(routing[index / size_t(width)], value);
        storage<T>::store(out + index, value);
    }
}

// Eight BF16 per thread per step; same arithmetic (a row is a whole number of such vectors, so one
// routing factor serves a vector).
__global__ void swiglu_bf16x8_kernel(size_t vectors, int row_vectors, float limit, const u32x4_t *gate,
                                     const u32x4_t *up, const float *routing, u32x4_t *out)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < vectors;
         index += size_t(gridDim.x) * blockDim.x) {
        const u32x4_t g = gate[index], u = up[index];
        const float factor = routing ? routing[index / size_t(row_vectors)] : 1.f;
        u32x4_t r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float value[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float gv = __uint_as_float(h ? g[e] & 0xffff0000u : g[e] << 16);
                float uv = __uint_as_float(h ? u[e] & 0xffff0000u : u[e] << 16);
                if (limit > 0) {
                    if (gv > limit)
                        gv = limit;
                    if (uv > limit)
                        uv = limit;
                    if (uv < -limit)
                        uv = -limit;
                }
                value[h] = __fmul_rn(gv / (1.f + expf(-gv)), uv);
                if (routing)
                    value[h] = __fmul_rn(factor, value[h]);
            }
            r[e] = pack_bf16x2(value[0], value[1]);
        }
        out[index] = r;
    }
}

// ---------------------------------------------------------------- RMS normalisation rows
// One workgroup per row. added = round_T(x + r) when a residual is given; scale = rsqrt(mean(v^2) +
// eps); out = round_T(round_T(v*scale) * w) or, without intermediate rounding, round_T((v*scale)*w)
// (ref: inference_fusion.cuh:53-86 and :136-191). The sum of squares uses a fixed order: per-thread
// strided partial sums, a 64-lane butterfly, then the wave partials in index order.
template <typename T, typename W>
__global__ __launch_bounds__(256) void rms_rows_kernel(int width, float epsilon,
                                                       bool round_before_weight, const T *input,
                                                       const T *residual, const W *weight, T *added,
                                                       T *out)
{
    __shared__ float partial[4];
    const size_t base = size_t(blockIdx.x) * width;
    const T *x = input + base;
    const T *r = residual ? residual + base : nullptr;
    float sum = 0.f;
    for (int column = threadIdx.x; column < width; column += 256) {
        float value = storage<T>::load(x + column);
        if (r)
            value = storage<T>::round(__fadd_rn(value, storage<T>::load(r + column)));
        sum = __fadd_rn(sum, __fmul_rn(value, value));
    }
    sum = wave_sum(sum);
    if (threadIdx.x % 64 == 0)
        partial[threadIdx.x / 64] = sum;
    __syncthreads();
    float total = __fadd_rn(__fadd_rn(partial[0], partial[1]), __fadd_rn(partial[2], partial[3]));
    float scale = rsqrtf(__fadd_rn(total / float(width), epsilon));
    for (int column = threadIdx.x; column < width; column += 256) {
        float value = storage<T>::load(x + column);
        if (r) {
            value = storage<T>::round(__fadd_rn(value, storage<T>::load(r + column)));
            storage<T>::store(added + base + column, value);
        }
        float normalised = __fmul_rn(value, scale);
        if (round_before_weight)
            normalised = storage<T>::round(normalised);
        storage<T>::store(out + base + column,
                          __fmul_rn(normalised, storage<W>::load(weight + column)));
    }
}

// BF16 rows whose width is a multiple of 8 and whose buffers are 16-byte aligned: the row is read
// once with 128-bit loads and kept in registers (THREADS x VECTORS vectors of 8 columns), same
// arithmetic and reduction order class as above. Decode batches have few rows, so a row is spread
// over up to 1024 threads to keep the dependent chain per thread short, and the weights are
// fetched before the reduction so that their latency overlaps it.
template <int VECTORS, bool WEIGHT_BF16, int THREADS>
__global__ __launch_bounds__(THREADS) void rms_rows_bf16_kernel(int width, float epsilon,
                                                            bool round_before_weight,
                                                            const unsigned short *input,
                                                            const unsigned short *residual,
                                                            const void *weight,
                                                            unsigned short *added,
                                                            unsigned short *out)
{
    __shared__ float partial[THREADS / 64];
    const size_t base = size_t(blockIdx.x) * width;
    const int vectors = width / 8;
    const u32x4_t *x = reinterpret_cast<const u32x4_t *>(input + base);
    const u32x4_t *r = residual ? reinterpret_cast<const u32x4_t *>(residual + base) : nullptr;
    float values[VECTORS][8];
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < VECTORS; ++v) {
        int index = v * THREADS + threadIdx.x;
        if (index < vectors) {
            u32x4_t xv = x[index];
            u32x4_t rv = {0u, 0u, 0u, 0u};
            if (r)
                rv = r[index];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float lo = __uint_as_float(xv[e] << 16), hi = __uint_as_float(xv[e] & 0xffff0000u);
                if (r) {
                    lo = bf16_bits_to_float(
                        float_to_bf16_bits(__fadd_rn(lo, __uint_as_float(rv[e] << 16))));
                    hi = bf16_bits_to_float(
                        float_to_bf16_bits(__fadd_rn(hi, __uint_as_float(rv[e] & 0xffff0000u))));
                }
                values[v][2 * e] = lo;
                values[v][2 * e + 1] = hi;
                sum = __fadd_rn(sum, __fmul_rn(lo, lo));
                sum = __fadd_rn(sum, __fmul_rn(hi, hi));
            }
            if (r) {
                u32x4_t packed;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    packed[e] = (__float_as_uint(values[v][2 * e]) >> 16) |
                                (__float_as_uint(values[v][2 * e + 1]) & 0xffff0000u);
                reinterpret_cast<u32x4_t *>(added + base)[index] = packed;
            }
        }
    }
    // weights of this thread's columns, requested before the reduction
    float w[VECTORS][8];
#pragma unroll
    for (int v = 0; v < VECTORS; ++v) {
        int index = v * THREADS + threadIdx.x;
        index = index < vectors ? index : vectors - 1;
        if constexpr (WEIGHT_BF16) {
            u32x4_t wv = reinterpret_cast<const u32x4_t *>(weight)[index];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[v][2 * e] = __uint_as_float(wv[e] << 16);
                w[v][2 * e + 1] = __uint_as_float(wv[e] & 0xffff0000u);
            }
        } else {
            const f32x4_t *wf = reinterpret_cast<const f32x4_t *>(weight) + 2 * index;
            f32x4_t w0 = wf[0], w1 = wf[1];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[v][e] = w0[e];
                w[v][4 + e] = w1[e];
            }
        }
    }
    sum = wave_sum(sum);
    if (threadIdx.x % 64 == 0)
        partial[threadIdx.x / 64] = sum;
    __syncthreads();
    float total = partial[0];
#pragma unroll
    for (int part = 1; part < THREADS / 64; ++part)
        total = __fadd_rn(total, partial[part]);
    float scale = rsqrtf(__fadd_rn(total / float(width), epsilon));
#pragma unroll
    for (int v = 0; v < VECTORS; ++v) {
        int index = v * THREADS + threadIdx.x;
        if (index < vectors) {
            u32x4_t packed;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float n0 = __fmul_rn(values[v][2 * e], scale);
                float n1 = __fmul_rn(values[v][2 * e + 1], scale);
                if (round_before_weight) {
                    n0 = bf16_bits_to_float(float_to_bf16_bits(n0));
                    n1 = bf16_bits_to_float(float_to_bf16_bits(n1));
                }
                packed[e] = pack_bf16x2(__fmul_rn(n0, w[v][2 * e]), __fmul_rn(n1, w[v][2 * e + 1]));
            }
            reinterpret_cast<u32x4_t *>(out + base)[index] = packed;
        }
    }
}

// ---------------------------------------------------------------- helpers kept for the binding
__global__ void bf16_square_kernel(size_t count, const unsigned short *input, float *out)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < count;
         index += size_t(gridDim.x) * blockDim.x) {
        float value = bf16_bits_to_float(input[index]);
        out[index] = __fmul_rn(value, value);
    }
}

// ref: inference_fusion.cuh:106-119
template <typename T>
__global__ void rms_scale_kernel(size_t count, int width, float epsilon, const T *input,
                                 const T *weight, const float *means, T *out)
{
    for (size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x; index < count;
         index += size_t(gridDim.x) * blockDim.x) {
        float scale = rsqrtf(__fadd_rn(means[index / size_t(width)], epsilon));
        float normalised = storage<T>::round(__fmul_rn(storage<T>::load(input + index), scale));
        storage<T>::store(out + index,
                          __fmul_rn(normalised, storage<T>::load(weight + index % size_t(width))));
    }
}

// ---------------------------------------------------------------- rotary embedding
// Rotate-half pairing (i, i + dim/2), angle = position * theta^(-2i/dim), FP32 sin/cos, one BF16
// rounding per element. One thread per (token, head, i).
__device__ __forceinline__ void rotate_pair(float position, int i, int dim, float theta, float lo,
                                            float hi, unsigned short &out_lo, unsigned short &out_hi)
{
    float s, c;
    pair_sincos(position, i, dim, theta, s, c);
    rotate_by(s, c, lo, hi, out_lo, out_hi);
}

__global__ void rope_kernel(int tokens, int heads, int dim, int token_stride, float theta,
                            const int32_t *positions, unsigned short *x)
{
    const int half = dim / 2;
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    size_t count = size_t(tokens) * heads * half;
    if (index >= count)
        return;
    int i = int(index % half);
    int head = int((index / half) % heads);
    int token = int(index / (size_t(half) * heads));
    unsigned short *v = x + size_t(token) * token_stride + size_t(head) * dim;
    rotate_pair(float(positions[token]), i, dim, theta, bf16_bits_to_float(v[i]),
                bf16_bits_to_float(v[i + half]), v[i], v[i + half]);
}

// Many tokens: one workgroup per token works out the sine and cosine of each pair index once (they
// do not depend on the head; one thread per (token, head, i) repeats them for every head and runs at
// the rate of the trigonometry, 2 TB/s) and then rotates eight pairs per thread with 16-byte
// accesses. Same arithmetic per element as rope_kernel.
__global__ __launch_bounds__(256) void rope_rows_kernel(int heads, int dim, int token_stride, float theta,
                                                        const int32_t *positions, unsigned short *x)
{
    __shared__ float sines[512], cosines[512];
    const int half = dim / 2, token = blockIdx.x, thread = threadIdx.x;
    const float position = float(positions[token]);
    for (int i = thread; i < half; i += 256)
        pair_sincos(position, i, dim, theta, sines[i], cosines[i]);
    __syncthreads();
    const int chunks = half / 8; // 8 pairs per thread and step
    unsigned short *row = x + size_t(token) * token_stride;
    for (int item = thread; item < heads * chunks; item += 256) {
        const int head = item / chunks, first = item % chunks * 8;
        u32x4_t *lo_at = reinterpret_cast<u32x4_t *>(row + size_t(head) * dim + first);
        u32x4_t *hi_at = reinterpret_cast<u32x4_t *>(row + size_t(head) * dim + half + first);
        const u32x4_t lo = *lo_at, hi = *hi_at;
        u32x4_t out_lo, out_hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            unsigned short l0, h0, l1, h1;
            rotate_by(sines[first + 2 * e], cosines[first + 2 * e], __uint_as_float(lo[e] << 16),
                      __uint_as_float(hi[e] << 16), l0, h0);
            rotate_by(sines[first + 2 * e + 1], cosines[first + 2 * e + 1], __uint_as_float(lo[e] & 0xffff0000u),
                      __uint_as_float(hi[e] & 0xffff0000u), l1, h1);
            out_lo[e] = unsigned(l0) | (unsigned(l1) << 16);
            out_hi[e] = unsigned(h0) | (unsigned(h1) << 16);
        }
        *lo_at = out_lo;
        *hi_at = out_hi;
    }
}

// Decode-step form of the two kernels above and below in one launch: a fused QKV activation row
// [q heads | k heads | v heads] per sequence; q and k heads are rotated in place, the rotated k
// heads and the v heads are also written to the caches at positions[b] (skipped when outside the
// cache). One thread per (sequence, head, i); same arithmetic as rope_kernel, bit for bit.
__global__ void rope_kv_append_kernel(int batch, int q_heads, int kv_heads, int dim,
                                      int token_stride, float theta, const int32_t *positions,
                                      unsigned short *qkv, int context_length,
                                      unsigned short *k_cache, unsigned short *v_cache)
{
    const int half = dim / 2, heads = q_heads + 2 * kv_heads;
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= size_t(batch) * heads * half)
        return;
    const int i = int(index % half);
    const int head = int((index / half) % heads);
    const int b = int(index / (size_t(half) * heads));
    const int position = positions[b];
    const bool cached = position >= 0 && position < context_length;
    unsigned short *v = qkv + size_t(b) * token_stride + size_t(head) * dim;
    unsigned short lo = v[i], hi = v[i + half];
    unsigned short *cache = nullptr;
    if (head < q_heads + kv_heads) {
        rotate_pair(float(position), i, dim, theta, bf16_bits_to_float(lo), bf16_bits_to_float(hi),
                    lo, hi);
        v[i] = lo;
        v[i + half] = hi;
        if (head >= q_heads)
            cache = k_cache + ((size_t(b) * context_length + position) * kv_heads + (head - q_heads)) * dim;
    } else {
        cache = v_cache + ((size_t(b) * context_length + position) * kv_heads +
                           (head - q_heads - kv_heads)) * dim;
    }
    if (cache && cached) {
        cache[i] = lo;
        cache[i + half] = hi;
    }
}

// Writes the new token's K and V heads (taken from a fused QKV activation row) into the caches at
// each sequence's position: 16 bytes per thread.
__global__ void kv_append_kernel(int batch, int kv_heads, int dim, int context_length,
                                 const int32_t *positions, const unsigned short *k_new,
                                 const unsigned short *v_new, int token_stride,
                                 unsigned short *k_cache, unsigned short *v_cache)
{
    const int vectors = kv_heads * dim / 8;
    size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= size_t(batch) * vectors)
        return;
    const int b = int(index / vectors), v = int(index % vectors);
    const int position = positions[b];
    if (position < 0 || position >= context_length)
        return;
    const size_t target = ((size_t(b) * context_length + position) * kv_heads * dim) / 8 + v;
    reinterpret_cast<u32x4_t *>(k_cache)[target] =
        reinterpret_cast<const u32x4_t *>(k_new + size_t(b) * token_stride)[v];
    reinterpret_cast<u32x4_t *>(v_cache)[target] =
        reinterpret_cast<const u32x4_t *>(v_new + size_t(b) * token_stride)[v];
}

unsigned stride_blocks(uint64_t count)
{
    uint64_t blocks = (count + 255) / 256;
    return unsigned(blocks < 65535 ? blocks : 65535);
}

bool aligned16(const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }
} // namespace

hipError_t launch_silu_multiply(hipStream_t stream, int dtype, uint64_t count, const void *gate,
                                const void *up, void *out)
{
    if (dtype == 0)
        silu_multiply_kernel<float><<<stride_blocks(count), 256, 0, stream>>>(
            count, static_cast<const float *>(gate), static_cast<const float *>(up),
            static_cast<float *>(out));
    else if (count % 8 == 0 && aligned16(gate) && aligned16(up) && aligned16(out))
        silu_multiply_bf16x8_kernel<<<stride_blocks(count / 8), 256, 0, stream>>>(
            count / 8, static_cast<const u32x4_t *>(gate), static_cast<const u32x4_t *>(up),
            static_cast<u32x4_t *>(out));
    else
        silu_multiply_kernel<bf16_storage><<<stride_blocks(count), 256, 0, stream>>>(
            count, static_cast<const bf16_storage *>(gate), static_cast<const bf16_storage *>(up),
            static_cast<bf16_storage *>(out));
    return launch_status();
}

hipError_t launch_swiglu(hipStream_t stream, int dtype, uint64_t count, int width, float limit,
                         const void *gate, const void *up, const float *routing, void *out)
{
    if (dtype == 0)
        swiglu_kernel<float><<<stride_blocks(count), 256, 0, stream>>>(
            count, width, limit, static_cast<const float *>(gate), static_cast<const float *>(up),
            routing, static_cast<float *>(out));
    else if (width % 8 == 0 && count % 8 == 0 && aligned16(gate) && aligned16(up) && aligned16(out))
        swiglu_bf16x8_kernel<<<stride_blocks(count / 8), 256, 0, stream>>>(
            count / 8, width / 8, limit, static_cast<const u32x4_t *>(gate), static_cast<const u32x4_t *>(up), routing,
            static_cast<u32x4_t *>(out));
    else
        swiglu_kernel<bf16_storage><<<stride_blocks(count), 256, 0, stream>>>(
            count, width, limit, static_cast<const bf16_storage *>(gate),
            static_cast<const bf16_storage *>(up), routing, static_cast<bf16_storage *>(out));
    return launch_status();
}

hipError_t launch_rms_rows(hipStream_t stream, int dtype, int weight_dtype, int rows, int width,
                           float epsilon, bool round_before_weight, const void *input,
                           const void *residual, const void *weight, void *added, void *out)
{
    if (dtype == 0) {
        rms_rows_kernel<float, float><<<rows, 256, 0, stream>>>(
            width, epsilon, round_before_weight, static_cast<const float *>(input),
            static_cast<const float *>(residual), static_cast<const float *>(weight),
            static_cast<float *>(added), static_cast<float *>(out));
        return launch_status();
    }
    const unsigned short *x = static_cast<const unsigned short *>(input);
    const unsigned short *r = static_cast<const unsigned short *>(residual);
    unsigned short *a = static_cast<unsigned short *>(added), *o = static_cast<unsigned short *>(out);
    bool vector = width % 8 == 0 && width <= 32768 && aligned16(input) && aligned16(out) &&
                  aligned16(weight) && (!residual || (aligned16(residual) && aligned16(added)));
#define CAMBLAS_RMS_ROWS(VECTORS, BF16_WEIGHT, THREADS)                                            \
    rms_rows_bf16_kernel<VECTORS, BF16_WEIGHT, THREADS>                                            \
        <<<rows, THREADS, 0, stream>>>(width, epsilon, round_before_weight, x, r, weight, a, o)
    if (vector) {
        const bool bf16_weight = weight_dtype == 2;
        if (width <= 2048) {
            if (bf16_weight)
                CAMBLAS_RMS_ROWS(1, true, 256);
            else
                CAMBLAS_RMS_ROWS(1, false, 256);
        } else if (width <= 8192) {
            if (bf16_weight)
                CAMBLAS_RMS_ROWS(1, true, 1024);
            else
                CAMBLAS_RMS_ROWS(1, false, 1024);
        } else {
            if (bf16_weight)
                CAMBLAS_RMS_ROWS(4, true, 1024);
            else
                CAMBLAS_RMS_ROWS(4, false, 1024);
        }
#undef CAMBLAS_RMS_ROWS
    } else if (weight_dtype == 2) {
        rms_rows_kernel<bf16_storage, bf16_storage><<<rows, 256, 0, stream>>>(
            width, epsilon, round_before_weight, static_cast<const bf16_storage *>(input),
            static_cast<const bf16_storage *>(residual), static_cast<const bf16_storage *>(weight),
            static_cast<bf16_storage *>(added), static_cast<bf16_storage *>(out));
    } else {
        rms_rows_kernel<bf16_storage, float><<<rows, 256, 0, stream>>>(
            width, epsilon, round_before_weight, static_cast<const bf16_storage *>(input),
            static_cast<const bf16_storage *>(residual), static_cast<const float *>(weight),
            static_cast<bf16_storage *>(added), static_cast<bf16_storage *>(out));
    }
    return launch_status();
}

namespace
{
// One workgroup per row: added = round(x + r), and the row's sum of squares of `added` in a fixed
// order (a thread's elements ascending, then the threads of a wavefront, then the wavefronts).
__global__ __launch_bounds__(256) void add_residual_squares_kernel(int width, const unsigned short *x,
                                                                   const unsigned short *residual,
                                                                   unsigned short *added, float *squares)
{
    __shared__ float partial[4];
    const size_t base = size_t(blockIdx.x) * width;
    float sum = 0.f;
    for (int column = threadIdx.x; column < width; column += 256) {
        const unsigned short bits = float_to_bf16_bits(
            __fadd_rn(bf16_bits_to_float(x[base + column]), bf16_bits_to_float(residual[base + column])));
        added[base + column] = bits;
        const float value = bf16_bits_to_float(bits);
        sum = __fadd_rn(sum, __fmul_rn(value, value));
    }
    sum = wave_sum(sum);
    if (threadIdx.x % 64 == 0)
        partial[threadIdx.x / 64] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
        squares[blockIdx.x] = __fadd_rn(__fadd_rn(partial[0], partial[1]), __fadd_rn(partial[2], partial[3]));
}
} // namespace

hipError_t launch_add_residual_squares(hipStream_t stream, int rows, int width, const void *x, const void *residual,
                                       void *added, float *squares)
{
    add_residual_squares_kernel<<<rows, 256, 0, stream>>>(width, static_cast<const unsigned short *>(x),
                                                          static_cast<const unsigned short *>(residual),
                                                          static_cast<unsigned short *>(added), squares);
    return launch_status();
}

hipError_t launch_bf16_square(hipStream_t stream, uint64_t count, const void *input, float *out)
{
    bf16_square_kernel<<<stride_blocks(count), 256, 0, stream>>>(
        count, static_cast<const unsigned short *>(input), out);
    return launch_status();
}

hipError_t launch_rms_scale(hipStream_t stream, int dtype, uint64_t count, int width, float epsilon,
                            const void *input, const void *weight, const float *means, void *out)
{
    if (dtype == 0)
        rms_scale_kernel<float><<<stride_blocks(count), 256, 0, stream>>>(
            count, width, epsilon, static_cast<const float *>(input),
            static_cast<const float *>(weight), means, static_cast<float *>(out));
    else
        rms_scale_kernel<bf16_storage><<<stride_blocks(count), 256, 0, stream>>>(
            count, width, epsilon, static_cast<const bf16_storage *>(input),
            static_cast<const bf16_storage *>(weight), means, static_cast<bf16_storage *>(out));
    return launch_status();
}

hipError_t launch_kv_append(hipStream_t stream, int batch, int kv_heads, int dim, int context_length,
                            const int32_t *positions, const void *k_new, const void *v_new,
                            int token_stride, void *k_cache, void *v_cache)
{
    size_t count = size_t(batch) * kv_heads * dim / 8;
    kv_append_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(
        batch, kv_heads, dim, context_length, positions, static_cast<const unsigned short *>(k_new),
        static_cast<const unsigned short *>(v_new), token_stride,
        static_cast<unsigned short *>(k_cache), static_cast<unsigned short *>(v_cache));
    return launch_status();
}

hipError_t launch_rope_kv_append(hipStream_t stream, int batch, int q_heads, int kv_heads, int dim,
                                 int token_stride, float theta, const int32_t *positions, void *qkv,
                                 int context_length, void *k_cache, void *v_cache)
{
    size_t count = size_t(batch) * (q_heads + 2 * kv_heads) * (dim / 2);
    rope_kv_append_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(
        batch, q_heads, kv_heads, dim, token_stride, theta, positions,
        static_cast<unsigned short *>(qkv), context_length, static_cast<unsigned short *>(k_cache),
        static_cast<unsigned short *>(v_cache));
    return launch_status();
}

hipError_t launch_rope(hipStream_t stream, int tokens, int heads, int dim, int token_stride,
                       float theta, const int32_t *positions, void *x)
{
    // (from 64 tokens on; fewer tokens are spread over more workgroups by the kernel below)
    if (tokens >= 64 && dim % 16 == 0 && dim <= 1024 && token_stride % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        rope_rows_kernel<<<unsigned(tokens), 256, 0, stream>>>(heads, dim, token_stride, theta, positions,
                                                               static_cast<unsigned short *>(x));
        return launch_status();
    }
    size_t count = size_t(tokens) * heads * (dim / 2);
    rope_kernel<<<unsigned((count + 255) / 256), 256, 0, stream>>>(
        tokens, heads, dim, token_stride, theta, positions, static_cast<unsigned short *>(x));
    return launch_status();
}
} // namespace camblas_hip
