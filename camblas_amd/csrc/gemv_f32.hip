// FP32 single-vector projection y = alpha W x + beta y for row-major W [rows, inner] (ld >= inner):
// full FP32 FMA, no reduced-precision path, bandwidth-bound on W. One wavefront owns four rows:
// 128-bit loads, two independent accumulators per row and lane, a fixed-order 64-lane butterfly.
// Contract and gate: ref src/cuda/decode_float.cuh:2-52, src/cuda/backend.cu:810-815. The
// reference's reduction tree is tied to 32-wide warps; this one is its wavefront-64 counterpart
// (fixed order, run-to-run deterministic).
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int WAVES = 4, ROWS_PER_WAVE = 4, ROWS_PER_BLOCK = WAVES * ROWS_PER_WAVE;

// One wavefront owns four consecutive rows so that every 128-bit load of x is reused four times;
// two column steps are in flight per lane (eight W loads).
__global__ __launch_bounds__(WAVES * 64) void gemv_f32_kernel(int rows, int inner, float alpha,
                                                              const float *w, int ld, const float *x,
                                                              float beta, float *y)
{
    const int lane = threadIdx.x % 64;
    const size_t row0 = size_t(blockIdx.x) * ROWS_PER_BLOCK + size_t(threadIdx.x / 64) * ROWS_PER_WAVE;
    if (row0 >= size_t(rows))
        return;
    const f32x4_t *wv[ROWS_PER_WAVE];
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
        size_t row = row0 + r < size_t(rows) ? row0 + r : size_t(rows) - 1; // clamp: result unused
        wv[r] = reinterpret_cast<const f32x4_t *>(w + row * ld);
    }
    const f32x4_t *xv = reinterpret_cast<const f32x4_t *>(x);
    const int vectors = inner / 4;
    float acc[ROWS_PER_WAVE][2] = {};
    int index = lane;
    for (; index + 64 < vectors; index += 128) {
        f32x4_t b0 = xv[index], b1 = xv[index + 64];
        f32x4_t a0[ROWS_PER_WAVE], a1[ROWS_PER_WAVE];
#pragma unroll
        for (int r = 0; r < ROWS_PER_WAVE; ++r) {
            a0[r] = __builtin_nontemporal_load(wv[r] + index); // W is read exactly once
            a1[r] = __builtin_nontemporal_load(wv[r] + index + 64);
        }
#pragma unroll
        for (int r = 0; r < ROWS_PER_WAVE; ++r)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[r][0] = fmaf(a0[r][e], b0[e], acc[r][0]);
                acc[r][1] = fmaf(a1[r][e], b1[e], acc[r][1]);
            }
    }
    for (; index < vectors; index += 64) {
        f32x4_t b0 = xv[index];
#pragma unroll
        for (int r = 0; r < ROWS_PER_WAVE; ++r) {
            f32x4_t a0 = __builtin_nontemporal_load(wv[r] + index);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc[r][0] = fmaf(a0[e], b0[e], acc[r][0]);
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
        float sum = wave_sum(acc[r][0] + acc[r][1]);
        if (lane == 0 && row0 + r < size_t(rows)) {
            float value = alpha * sum;
            if (beta != 0.f)
                value = fmaf(beta, y[row0 + r], value);
            y[row0 + r] = value;
        }
    }
}
} // namespace

hipError_t launch_gemv_f32(hipStream_t stream, int rows, int inner, float alpha, const float *w,
                           int ld, const float *x, float beta, float *y)
{
    unsigned blocks = unsigned((size_t(rows) + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
    gemv_f32_kernel<<<blocks, WAVES * 64, 0, stream>>>(rows, inner, alpha, w, ld, x, beta, y);
    return launch_status();
}
} // namespace camblas_hip
