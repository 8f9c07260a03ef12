// Shared declarations of libcamblas_hip.so: context, error convention, kernel launch prototypes.
#pragma once

#include "camblas_hip.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <vector>

// One device, one stream, scratch, counters, last error text.
// Mirrors the role of the reference context (src/cuda/backend.cu:57-77) without vendor handles.
struct camblas_cuda_context {
    int device = 0;
    int algorithm = CAMBLAS_CUDA_AUTO;
    hipStream_t stream = nullptr;
    int compute_units = 256;
    void *scratch = nullptr;       // split-K partials, attention partials
    size_t scratch_bytes = 0;
    size_t held_bytes = 0;         // leading bytes of the arena an enclosing helper keeps live across nested products
    std::vector<void *> retired;   // superseded scratch kept alive for captured graphs
    size_t retired_bytes = 0;      // what those arenas hold together
    bool seen_capture = false;     // the arena has been used by a launch under stream capture
    unsigned *arrivals = nullptr;  // zeroed counters of the divided-K streaming kernel (made on first use)
    int override_kernel = -1;      // diagnostics: forced kernel variant
    int override_split = 0;
    std::atomic<uint64_t> counts[8] = {};
    char error[256] = "";
};

namespace camblas_hip
{
// Formats "<operation> failed (status <code>)" into the context (or the calling thread's creation
// buffer when context is null) and returns -code for positive codes, else -1
// (ref: src/cuda/backend.cu:81-86).
int fail(camblas_cuda_context *context, const char *operation, int code);

// Ensures the context scratch holds at least `bytes`; refuses to grow while the stream is
// capturing (ref: src/cuda/backend.cu:399-426). Returns hipSuccess or the failing status.
hipError_t reserve_scratch(camblas_cuda_context *context, size_t bytes);
// Room for `bytes` of temporaries of one product: from the arena's start, or, while an enclosing
// helper holds the leading held_bytes of it (attention scores, column-sum partials), behind them
// and only if the arena already has the room: growing would free what the helper holds. Null
// when there is no room (the caller then runs the form that needs none).
void *claim_scratch(camblas_cuda_context *context, size_t bytes);
// Marks the leading `bytes` of the arena as held until the end of the scope.
struct ScratchHold {
    camblas_cuda_context *context;
    ScratchHold(camblas_cuda_context *c, size_t bytes) : context(c) { c->held_bytes = bytes; }
    ~ScratchHold() { context->held_bytes = 0; }
    ScratchHold(const ScratchHold &) = delete;
    ScratchHold &operator=(const ScratchHold &) = delete;
};
// The context's arrival counters (STREAM_ARRIVAL_SLOTS of them, zero between launches), made and
// cleared on first use; never under stream capture.
hipError_t reserve_arrivals(camblas_cuda_context *context);

inline hipError_t launch_status() { return hipGetLastError(); }

// Per kernel instantiation and device: which devices have had the kernel's dynamic LDS limit raised.
// Contexts on different host threads may launch the same kernel at the same time, so the flags are
// atomic; setting the attribute twice is harmless, so no lock is needed.
struct LdsLimitFlags {
    std::atomic<bool> raised[64] = {};
};

// Raises `kernel`'s dynamic shared memory limit to `bytes` once per device (the current one).
inline hipError_t raise_lds_limit(LdsLimitFlags &flags, const void *kernel, size_t bytes)
{
    int device = 0;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess)
        return status;
    const bool tracked = device >= 0 && device < 64;
    if (tracked && flags.raised[device].load(std::memory_order_acquire))
        return hipSuccess;
    status = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes));
    if (status == hipSuccess && tracked)
        flags.raised[device].store(true, std::memory_order_release);
    return status;
}

// ---------------------------------------------------------------- planner (pure host)
enum KernelFamily {
    FAMILY_GENERIC = 0, // LDS-tiled VALU kernel, any transpose / leading dimension / alignment
    FAMILY_GEMV_F32 = 1,
    FAMILY_MFMA_TN = 2, // BF16 'T','N', K-contiguous operands, MFMA tiles staged through LDS
    FAMILY_FP8_BLOCK = 3,
    FAMILY_STREAM = 4, // BF16 'T','N' with few tokens: weight-streaming kernel, one pass over W
    FAMILY_DMA = 5,    // BF16 'T','N' prefill: large MFMA tiles fed by direct global->LDS loads
    FAMILY_FP8_DMA = 6, // FP8 block-scaled prefill: the same structure with one scale group per step
    FAMILY_FP8_STREAM = 7, // FP8 block-scaled decode: weight-streaming kernel (10*row_tiles + token_tiles)
    FAMILY_MFMA_F32 = 8,   // FP32, any layout: 128 x 128 tiles on the FP32 matrix-core instruction
    FAMILY_MFMA_BF16 = 9,  // BF16, any layout: the same structure on the BF16 matrix-core instruction
    FAMILY_NN = 10         // BF16 'N','N' with up to a few hundred tokens: one pass over a W that has its outputs contiguous
};

struct Plan {
    int family = FAMILY_GENERIC;
    int kernel = 0;   // variant index inside the family (stream family: 100*log2(K blocks per step) + 10*row_tiles + token_tiles)
    int split_k = 1;  // number of K partitions (partials reduced in fixed order)
    int counter = 0;  // stats slot incremented at launch
    // FP8 prefill tiles: the last tail_outputs outputs run on variant tail_kernel in a second launch
    int tail_kernel = 0, tail_outputs = 0;
};

// dtype: 0 FP32, 2 BF16, 3 FP8 block-scaled ('T','N' implied). aligned16: every operand pointer
// is 16-byte aligned. compute_units sizes split-K. Pure function: no device access.
Plan make_plan(int dtype, int algorithm, bool trans_a, bool trans_b, int m, int n, int k, int lda,
               int ldb, int ldc, bool aligned16, int compute_units);
void describe_plan(const Plan &plan, int dtype, char *text, size_t bytes);

struct TnVariant {
    const char *name;
    int block_n, block_m, block_k, threads;
};
int tn_variant_count();
const TnVariant &tn_variant(int index);
int dma_variant_count();
const TnVariant &dma_variant(int index);
int fp8_dma_variant_count();
const TnVariant &fp8_dma_variant(int index);
int fp8_variant_count();
const TnVariant &fp8_variant(int index);

// ---------------------------------------------------------------- launchers (each returns a hipError_t)
hipError_t launch_scale_f32(hipStream_t stream, int m, int n, float beta, float *c, int ldc);
hipError_t launch_scale_bf16(hipStream_t stream, int m, int n, float beta, void *c, int ldc);
// c[i + j*ldc] = z[i + j*ldz] for BF16 storage; ldz == 0 repeats one column of m values
hipError_t launch_spread_bf16(hipStream_t stream, int m, int n, const void *z, int ldz, void *c, int ldc);
hipError_t launch_scale_f64(hipStream_t stream, int m, int n, double beta, double *c, int ldc);
hipError_t launch_generic_f32(hipStream_t stream, bool ta, bool tb, int m, int n, int k, float alpha,
                              const float *a, int lda, const float *b, int ldb, float beta, float *c,
                              int ldc);
// wide: 128 x 128 output tiles per workgroup, else 128 x 64
// batches > 1: that many independent products, operands and outputs batch_stride elements apart;
// lower_only (square outputs): only the tiles that reach the diagonal run, as a one-dimensional grid
// (the caller mirrors the lower triangle)
hipError_t launch_sgemm_mfma(hipStream_t stream, bool wide, bool ta, bool tb, int m, int n, int k,
                             float alpha, const float *a, int lda, const float *b, int ldb, float beta,
                             float *c, int ldc, int batches = 1, size_t batch_stride = 0,
                             bool lower_only = false);
// The FP32 product with K divided over `shares` workgroups per 128 x 64 tile (k % shares == 0; planes:
// shares * m * n floats, summed in share order): few columns of C against a large A.
hipError_t launch_sgemm_mfma_divided(hipStream_t stream, bool ta, bool tb, int m, int n, int k, float alpha,
                                     const float *a, int lda, const float *b, int ldb, float beta, float *c,
                                     int ldc, int shares, float *planes, bool narrow);
hipError_t launch_dgemm_mfma(hipStream_t stream, bool ta, bool tb, int m, int n, int k, double alpha,
                             const double *a, int lda, const double *b, int ldb, double beta, double *c,
                             int ldc, int batches = 1, size_t batch_stride = 0, bool lower_only = false);
hipError_t launch_dgemm_mfma_divided(hipStream_t stream, bool ta, bool tb, int m, int n, int k, double alpha,
                                     const double *a, int lda, const double *b, int ldb, double beta,
                                     double *c, int ldc, int shares, double *planes, int tile_columns);
// c[row, column] = c[column, row] for row < column of a column-major n x n matrix (dtype 0 FP32, 1 FP64)
hipError_t launch_mirror_lower(hipStream_t stream, int dtype, int n, void *c, int ldc);
// Strassen policies for square 'N','N' products (strassen.hip). strassen_levels: recursion depth of
// a policy for size n (0: the policy does not apply). strassen_gemm returns STRASSEN_DONE,
// STRASSEN_FALL_BACK (guard raised or no scratch: counted, the caller runs the ordinary kernel),
// STRASSEN_NOT_ELIGIBLE (capture, operands in scratch, non-finite alpha: nothing counted), or a
// negative status after fail().
enum { STRASSEN_DONE = 0, STRASSEN_FALL_BACK = 1, STRASSEN_NOT_ELIGIBLE = 2 };
int strassen_levels(int algorithm, int n);
template <typename T>
int strassen_gemm(camblas_cuda_context *context, int levels, int n, T alpha, const T *a, int lda, const T *b,
                  int ldb, T beta, T *c, int ldc);
hipError_t launch_generic_bf16(hipStream_t stream, bool ta, bool tb, int m, int n, int k,
                               float alpha, const void *a, int lda, const void *b, int ldb,
                               float beta, void *c, int ldc);
hipError_t launch_generic_f64(hipStream_t stream, bool ta, bool tb, int m, int n, int k,
                              double alpha, const double *a, int lda, const double *b, int ldb,
                              double beta, double *c, int ldc);
// BF16 for any transpose pair / leading dimension / alignment on the matrix cores (bgemm_any.hip);
// wide: 128 x 128 tiles, else 128 x 64.
hipError_t launch_bgemm_any(hipStream_t stream, bool wide, bool ta, bool tb, int m, int n, int k,
                            float alpha, const void *a, int lda, const void *b, int ldb, float beta,
                            void *c, int ldc);
// dst[c * ld_dst + r] = src[r * ld_src + c], BF16 storage, `cols` the contiguous extent of src
hipError_t launch_transpose_bf16(hipStream_t stream, int rows, int cols, const void *src, int ld_src, void *dst,
                                 int ld_dst);
hipError_t launch_gemv_f32(hipStream_t stream, int rows, int inner, float alpha, const float *w,
                           int ld, const float *x, float beta, float *y);
// Where the beta term of a BF16 linear is read from: by default the output itself; otherwise
// z[token * ldz + feature] with ldz == 0 for one row broadcast over the tokens (a bias vector).
// z must not overlap the output.
struct BetaSource {
    const void *z = nullptr;
    int ldz = 0;
};
// y[M,N] (ldc) = alpha * x[M,K] (ldb) * W[N,K]^T (lda) + beta * (source or y), BF16 storage.
// partials: FP32 [split_k, M, N] when split_k > 1.
hipError_t launch_bgemm_tn(hipStream_t stream, int variant, int split_k, int n_out, int m_rows,
                           int k, float alpha, const void *w, int lda, const void *x, int ldb,
                           float beta, void *y, int ldc, float *partials, const BetaSource &source = {});
// Prefill BF16 linear with direct-to-LDS operand loads; variants are listed by dma_variant().
// Needs k % 64 == 0, n_out % 4 == 0, ldc % 4 == 0, y 8-byte aligned (and the same of a beta source).
hipError_t launch_bgemm_dma(hipStream_t stream, int variant, int n_out, int m_rows, int k,
                            float alpha, const void *w, int lda, const void *x, int ldb, float beta,
                            void *y, int ldc, const BetaSource &source = {}, int shares = 1,
                            float *partials = nullptr);
// y = alpha * (plane 0 + ... + plane shares-1) + beta * z, planes [share][token][output] FP32, added in
// index order; n_out, ldc, ldz multiples of four, y and z 8-byte aligned.
hipError_t launch_sum_shares(hipStream_t stream, const float *partials, int shares, int n_out, int m_rows,
                             float alpha, float beta, const void *z, int ldz, void *y, int ldc);
// y[M,N] (ldc) = alpha * x[M,K] (ldb) * W[K,N] (lda: outputs contiguous) + beta * y for few tokens; needs
// k % 64 == 0, n_out % 4 == 0, lda % 8 == 0, ldb % 8 == 0, ldc % 4 == 0, 16-byte aligned W and x, 8-byte
// aligned y. partials: FP32 [shares, M, N] when shares > 1.
hipError_t launch_bgemm_nn(hipStream_t stream, int n_out, int m_rows, int k, float alpha, const void *w, int lda,
                           const void *x, int ldb, float beta, void *y, int ldc, int shares = 1,
                           float *partials = nullptr);
// Decode-shaped BF16 linear: each workgroup streams 16*row_tiles weight rows over the whole K.
// depth_log2: a K step is 2^depth_log2 blocks of 128 elements (0..3); row_tiles << depth_log2 <= 8
// and (row_tiles + token_tiles) << depth_log2 <= 16 or the launch is refused.
// shares: with count > 1 the K extent is divided over that many workgroups per output tile; each
// parks FP32 sums in its plane of `partials` (stream_partial_bytes() in all, 16-byte aligned) and
// the last to arrive adds the planes in index order. `arrivals` holds STREAM_ARRIVAL_SLOTS counters that are zero between
// launches (the kernel leaves them so); one per output tile is used.
constexpr size_t STREAM_ARRIVAL_SLOTS = 4096;
// The FP8 streaming kernel keeps a row of K / 128 scales per token in LDS: rows of this many floats
// (whole 64-float loads, odd so that tokens fall on different banks), at most 192 groups (K <= 24576).
constexpr int STREAM_SCALE_PITCH = 193, STREAM_SCALE_GROUPS = 192;
size_t stream_partial_bytes(int row_tiles, int token_tiles, int n_out, int m_rows, int shares);
struct StreamShares {
    int count = 1;
    float *partials = nullptr;
    unsigned *arrivals = nullptr;
};
int undivided_stream_kernel(int outputs, int tokens, int k, int compute_units);
// The residual-add + RMSNorm around a decode linear, moved into the linears on either side of it.
// norm_weight (BF16 [k], 16-byte aligned): x is normalised while it is staged, with the row scales
// rsqrt(sum / k + epsilon), sum = ssq_in[0 * ssq_ld + token] + ssq_in[1 * ssq_ld + token] + ... over
// ssq_count entries in index order. residual (BF16, ld_residual >= outputs): y = round(round(alpha *
// x W^T) + residual) (beta must be 0), and every workgroup along the outputs leaves the sums of
// squares of its features of each row of y in ssq_out[workgroup * ssq_ld_out + token]; the number of
// such workgroups is stream_workgroups_along_outputs().
struct StreamFusion {
    const void *norm_weight = nullptr;
    const float *ssq_in = nullptr;
    int ssq_count = 0, ssq_ld = 0;
    float epsilon = 0.f;
    const void *residual = nullptr;
    int ld_residual = 0;
    float *ssq_out = nullptr;
    int ssq_ld_out = 0;
};
inline int stream_workgroups_along_outputs(int row_tiles, int n_out) { return (n_out + row_tiles * 16 - 1) / (row_tiles * 16); }
hipError_t launch_bgemv_stream(hipStream_t stream, int depth_log2, int row_tiles, int token_tiles, int n_out,
                               int m_rows, int k, float alpha, const void *w, int lda,
                               const void *x, int ldb, float beta, void *y, int ldc,
                               const BetaSource &source = {}, const StreamShares &shares = {},
                               const StreamFusion &fusion = {});
// The gated-MLP front end for decode batches in one pass over both weight matrices:
// y = round(round(silu(g)) * u), g = round(x gate^T), u = round(x up^T). pair_tiles 1..4 (16 output
// rows each: that many gate rows and the same up rows per workgroup), token_tiles 1, 2 or 4.
hipError_t launch_gated_stream(hipStream_t stream, int pair_tiles, int token_tiles, int n_out, int m_rows,
                               int k, const void *gate, const void *up, int lda, const void *x, int ldb,
                               void *y, int ldc, const StreamFusion &fusion = {});
hipError_t launch_fp8_block(hipStream_t stream, int variant, int split_k, int rows, int outputs,
                            int inner, const void *a, const float *a_scale, const void *w,
                            const float *w_scale, void *out, float *partials);
// Prefill FP8 block-scaled linear with direct-to-LDS loads; needs outputs % 4 == 0.
// split_k > 1: K groups divided over that many workgroups per tile, FP32 planes in `partials`
// ([split_k, rows, outputs]) summed in index order.
hipError_t launch_fp8_dma(hipStream_t stream, int variant, int split_k, int rows, int outputs, int inner,
                          const void *a, const float *a_scale, const void *w, const float *w_scale,
                          void *out, float *partials, int tail_variant = 0, int tail_outputs = 0);
// fp8_wave4.hip: the same product on four wavefronts per workgroup (192 x 256 tiles); inner % 1024 == 0,
// inner >= 2048, undivided K only.
hipError_t launch_fp8_wave4(hipStream_t stream, int rows, int outputs, int inner, const void *a, const float *a_scale,
                            const void *w, const float *w_scale, void *out, int out_pitch);
hipError_t launch_fp8_split_sum(hipStream_t stream, int splits, size_t count, const float *partials, void *out);
// row_tiles 1..8 (16 weight rows each), token_tiles 1 to 4 (16 tokens each); product <= 20, sum <= 10.
hipError_t launch_fp8_stream(hipStream_t stream, int row_tiles, int token_tiles, int rows, int outputs,
                             int inner, const void *a, const float *a_scale, const void *w,
                             const float *w_scale, void *out);
// Single-token product with 32-wide FP32 scale blocks; sx null: x is BF16 and quantised on the fly.
// forced_waves 1, 2 or 4: wavefronts per workgroup (0: by the number of outputs).
hipError_t launch_fp8_block32_decode(hipStream_t stream, int outputs, int inner, const void *x,
                                     const float *sx, int sx_stride, const void *w, const float *sw,
                                     int sw_row, int sw_col, void *out, int forced_waves = 0);
// One token through an FP8 (1x128 . 128x128 scales) mixture-of-experts layer: gate/up products,
// clipped SiLU-multiply, down products, routed sum. scratch: fp8_moe_decode_scratch_bytes().
size_t fp8_moe_decode_scratch_bytes(int choices, int width);
hipError_t launch_fp8_moe_decode(hipStream_t stream, int experts, int choices, int hidden, int width,
                                 int hidden_out, const void *x, const void *w1, const float *s1,
                                 const void *w2, const float *s2, const int32_t *ids,
                                 const float *routing, float factor, void *scratch, void *out);
// E8M0 block-scaled product (E4M3 or packed E2M1 weights); groups == 0 plain, >= 1 grouped.
// kernel: -1 chooses by shape; 0 the weight-streaming kernel; 20 + v the prefill kernel variant v.
hipError_t launch_mx_matmul(hipStream_t stream, int kernel, int compute_units, bool packed, int groups,
                            int weight_groups, int rows, int outputs, int inner,
                            int activation_block, const void *input,
                            const void *input_scale, const void *weight, const void *weight_scale,
                            const void *metadata, const void *active, const void *counts, void *out,
                            int forced_shares = 0, float *planes = nullptr);
// Workgroups that launch_mx_matmul would divide K over for a plain product (1: K is not divided);
// `planes` then needs that many times rows * outputs floats, and without it K is not divided.
int mx_matmul_shares(int kernel, int forced_shares, int compute_units, bool packed, int rows, int outputs,
                     int inner, int activation_block, const void *input, const void *weight, const void *out);
// Prefill-sized E8M0 product (hardware-scaled matrix instructions, operands loaded straight into
// LDS); needs inner % 128 == 0, 16-byte aligned operands and an 8-byte aligned output.
int mx_dma_variant_count();
bool mx_dma_supported(int outputs, int inner, const void *input, const void *weight, const void *out);
hipError_t launch_mx_dma(hipStream_t stream, int variant, bool packed, int groups, int weight_groups,
                         int rows, int outputs, int inner, int activation_block, const void *input,
                         const void *input_scale, const void *weight, const void *weight_scale,
                         const void *metadata, const void *active, const void *counts, void *out,
                         int tail_variant = 0, int tail_outputs = 0, int shares = 1, float *planes = nullptr);
// mx_wave4.hip: the product on four wavefronts per workgroup (192 x 256 tiles); one input scale per 32 inputs,
// inner % 1024 == 0, inner >= 2048, input scales 16-byte aligned, packed weights' scales 16-byte aligned.
// metadata != nullptr: the grouped product (E4M3 weights only, out_pitch = outputs).
hipError_t launch_mx_wave4(hipStream_t stream, bool packed, int rows, int outputs, int inner, const void *input,
                           const void *input_scale, const void *weight, const void *weight_scale, void *out, int out_pitch,
                           int groups = 0, int weight_groups = 0, const void *metadata = nullptr,
                           const void *active = nullptr, const void *counts = nullptr);
// Mixture-of-experts routing helpers.
hipError_t launch_route_groups(hipStream_t stream, int tokens, int choices, int first_expert,
                               int groups, int rows, const void *experts, const void *active,
                               void *counts, void *slots, void *reverse);
hipError_t launch_reduce_groups(hipStream_t stream, int tokens, int choices, int width,
                                int grouped_rows, const void *experts, const void *reverse,
                                const void *input, void *output);
// Dense helpers (dtype 0 FP32, 1 FP64): bias + optional ReLU over a row-major [count/columns, columns]
// matrix; in-place softmax(scale * row); column sums in `chunks` row chunks (partial: [chunks, columns]
// scratch when chunks > 1), optionally zeroing grad where activation <= 0 first.
hipError_t launch_bias_activation(hipStream_t stream, int dtype, void *out, const void *bias,
                                  size_t count, int columns, bool relu);
hipError_t launch_softmax_rows(hipStream_t stream, int dtype, void *scores, int rows, int columns,
                               double scale);
hipError_t launch_column_sums(hipStream_t stream, int dtype, bool mask, void *grad,
                              const void *activation, int rows, int columns, int chunks,
                              int chunk_rows, void *partial, void *sums);
hipError_t launch_fp8_quantise(hipStream_t stream, int rows, int inner, const void *x, void *q,
                               float *scale);
hipError_t launch_silu_multiply(hipStream_t stream, int dtype, uint64_t count, const void *gate,
                                const void *up, void *out);
hipError_t launch_swiglu(hipStream_t stream, int dtype, uint64_t count, int width, float limit,
                         const void *gate, const void *up, const float *routing, void *out);
hipError_t launch_rms_rows(hipStream_t stream, int dtype, int weight_dtype, int rows, int width,
                           float epsilon, bool round_before_weight, const void *input,
                           const void *residual, const void *weight, void *added, void *out);
// added[row] = round(x[row] + residual[row]) (BF16, contiguous rows of `width`), squares[row] = sum of added^2
hipError_t launch_add_residual_squares(hipStream_t stream, int rows, int width, const void *x, const void *residual,
                                       void *added, float *squares);
hipError_t launch_bf16_square(hipStream_t stream, uint64_t count, const void *input, float *out);
hipError_t launch_rms_scale(hipStream_t stream, int dtype, uint64_t count, int width, float epsilon,
                            const void *input, const void *weight, const float *means, void *out);
hipError_t launch_kv_append(hipStream_t stream, int batch, int kv_heads, int dim, int context_length,
                            const int32_t *positions, const void *k_new, const void *v_new,
                            int token_stride, void *k_cache, void *v_cache);
hipError_t launch_rope_kv_append(hipStream_t stream, int batch, int q_heads, int kv_heads, int dim,
                                 int token_stride, float theta, const int32_t *positions, void *qkv,
                                 int context_length, void *k_cache, void *v_cache);
hipError_t launch_rope(hipStream_t stream, int tokens, int heads, int dim, int token_stride,
                       float theta, const int32_t *positions, void *x);
size_t gqa_decode_scratch_bytes(int batch, int q_heads, int dim, int context_length, int *splits);
// Fixed device array for the allocation-free attention entry point: its size, and its address on
// `device` (which must be current; resolved with hipGetSymbolAddress on first use per device).
size_t gqa_resident_scratch_bytes();
hipError_t gqa_resident_scratch(int device, void **address);
// positions (with theta, k_new, v_new) non-null: the step's new token arrives un-rotated, q / k_new /
// v_new rows q_stride apart per sequence; the kernel rotates q and k_new, attends over positions + 1
// entries and writes the new K and V rows into the caches (k and v are then written to); lengths unused.
hipError_t launch_gqa_decode(hipStream_t stream, int batch, int q_heads, int kv_heads, int dim,
                             int context_length, const int32_t *lengths, float scale, const void *q,
                             int q_stride, const void *k, const void *v, void *out, void *partials,
                             int splits, const int32_t *positions = nullptr, float theta = 0.f,
                             const void *k_new = nullptr, const void *v_new = nullptr, const float *table = nullptr);
// table[b][0][i] = sin, table[b][1][i] = cos of positions[b] * theta^(-2i/dim) for i < dim / 2
hipError_t launch_rope_table(hipStream_t stream, int batch, int dim, float theta, const int32_t *positions,
                             float *table);
} // namespace camblas_hip
