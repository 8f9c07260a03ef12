// FP32 single-vector projection y = alpha W x + beta y for row-major W [rows, inner] (ld >= inner):
// full FP32 FMA, no reduced-precision path, bandwidth-bound on W. One wavefront owns one row:
// 128-bit loads, four independent accumulators per lane, a fixed-order 64-lane butterfly.
// Contract and gate: ref src/cuda/decode_float.cuh:2-52, src/cuda/backend.cu:810-815. The
// reference's reduction tree is tied to 32-wide warps; this one is its wavefront-64 counterpart
// (fixed order, run-to-run deterministic).
#include "common.hpp"
#include "device.hpp"

namespace camblas_hip
{
namespace
{
constexpr int ROWS_PER_BLOCK = 4;

__global__ __launch_bounds__(ROWS_PER_BLOCK * 64) void gemv_f32_kernel(int rows, int inner,
                                                                       float alpha, const float *w,
                                                                       int ld, const float *x,
                                                                       float beta, float *y)
{
    const int lane = threadIdx.x % 64;
    const size_t row = size_t(blockIdx.x) * ROWS_PER_BLOCK + threadIdx.x / 64;
    if (row >= size_t(rows))
        return;
    const f32x4_t *wv = reinterpret_cast<const f32x4_t *>(w + row * ld);
    const f32x4_t *xv = reinterpret_cast<const f32x4_t *>(x);
    const int vectors = inner / 4;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    int index = lane;
    for (; index + 192 < vectors; index += 256) {
        f32x4_t a0 = __builtin_nontemporal_load(wv + index);
        f32x4_t a1 = __builtin_nontemporal_load(wv + index + 64);
        f32x4_t a2 = __builtin_nontemporal_load(wv + index + 128);
        f32x4_t a3 = __builtin_nontemporal_load(wv + index + 192);
        f32x4_t b0 = xv[index], b1 = xv[index + 64], b2 = xv[index + 128], b3 = xv[index + 192];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            acc[0] = fmaf(a0[e], b0[e], acc[0]);
            acc[1] = fmaf(a1[e], b1[e], acc[1]);
            acc[2] = fmaf(a2[e], b2[e], acc[2]);
            acc[3] = fmaf(a3[e], b3[e], acc[3]);
        }
    }
    for (; index < vectors; index += 64) {
        f32x4_t a0 = wv[index], b0 = xv[index];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            acc[0] = fmaf(a0[e], b0[e], acc[0]);
    }
    float sum = wave_sum((acc[0] + acc[1]) + (acc[2] + acc[3]));
    if (lane == 0) {
        float value = alpha * sum;
        if (beta != 0.f)
            value = fmaf(beta, y[row], value);
        y[row] = value;
    }
}
} // namespace

hipError_t launch_gemv_f32(hipStream_t stream, int rows, int inner, float alpha, const float *w,
                           int ld, const float *x, float beta, float *y)
{
    unsigned blocks = unsigned((size_t(rows) + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
    gemv_f32_kernel<<<blocks, ROWS_PER_BLOCK * 64, 0, stream>>>(rows, inner, alpha, w, ld, x, beta,
                                                                y);
    return launch_status();
}
} // namespace camblas_hip
