// Launch parameters shared by the BF16 prefill kernels (bgemm_dma.hip, bgemm_wave4.hip).
#pragma once

#include "common.hpp"

namespace camblas_hip
{
struct DmaParams {
    const unsigned short *w;
    const unsigned short *x;
    unsigned short *y;
    const unsigned short *z; // what beta multiplies: z[token * ldz + feature] (y and ldc by default)
    int lda, ldb, ldc, ldz;
    int n, m, k;
    float alpha, beta;
    int tiles_n, tiles_m;
    // K divided over gridDim.y workgroups per tile: each takes `share_steps` steps of BK and leaves
    // its FP32 sums in plane blockIdx.y of `partials` ([share][token][feature])
    float *partials;
    int share_steps;
};

// The four-wavefront tiles of bgemm_wave4.hip: rows 256 or 320 weight rows x 256 tokens x 64. Needs what
// launch_bgemm_dma needs and an even number (at least two) of 64-element K steps per share.
// weights_as_they_lie (256 rows only): p.w is W[K, N] with the outputs contiguous, p.lda its row pitch
// (a multiple of 8 elements), the product still y = x W.
hipError_t launch_bgemm_wave4(hipStream_t stream, int rows, DmaParams p, int shares, bool weights_as_they_lie = false);
// y = alpha * (sum of the shares' planes in index order) + beta * z (bgemm_dma.hip)
hipError_t launch_sum_shares(hipStream_t stream, const DmaParams &p, int shares);
} // namespace camblas_hip
