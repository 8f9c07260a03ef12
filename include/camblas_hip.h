/*
 * C ABI of libcamblas_hip.so: the MI355X (gfx950) backend for the CAMBLAS GPU linear path.
 *
 * The exported symbols keep the reference's names (camblas_cuda_*) and signatures so the
 * reference's ctypes loader (camblas/_native.py:97-173) and tensor binding resolve them
 * unchanged when CAMBLAS_CUDA_LIBRARY points at this library. Each declaration cites the reference
 * interface it replaces as "ref: file:line" (paths relative to the reference tree). Entry points
 * marked "extension" have no counterpart in include/camblas_cuda.h; the comment says which
 * reference code defines their arithmetic.
 *
 * Conventions (ref: include/camblas_cuda.h:25-38, src/cuda/backend.cu:81-86):
 *  - every operation returns 0 on success and a negative code on failure; the message is
 *    available from camblas_cuda_error(context) (or camblas_cuda_error(NULL) for creation errors,
 *    which are stored per host thread);
 *  - one context owns one device and one HIP stream (hipStream_t passed as void*); calls enqueue
 *    work on that stream and return; the caller keeps operands alive until the stream completes;
 *  - a context is single-threaded and not fork-safe; use one per (thread, device, stream);
 *  - stream capture: create contexts and run each shape once before capturing; scratch growth is
 *    refused while the stream is capturing.
 */
#ifndef CAMBLAS_HIP_H
#define CAMBLAS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct camblas_cuda_context camblas_cuda_context;

/* ref: include/camblas_cuda.h:14-23. On this backend AUTO and LT select the planned MFMA/GEMV
 * kernels (counter slot 4), CLASSICAL counts in slot 0 (and for BF16 forces the generic LDS-tiled
 * kernel). Under SYMMETRIC an sgemm / dgemm call with a == b, opposite transposes, m == n,
 * lda == ldb and beta == 0 (a matrix times its own transpose; ref: src/cuda/backend.cu:819-835)
 * computes only the tiles that reach the diagonal and copies the lower triangle into the upper one,
 * so C equals its transpose bit for bit (counter slot 2); every other call is an ordinary product.
 * STRASSEN / _TWO / _THREE / _FOUR apply to sgemm and dgemm of square 'N','N' products of even
 * size from 256 (ref: src/cuda/backend.cu:442-551, :836-853): one to four levels of Strassen's
 * seven-product recursion, as deep as n stays divisible by two and the leaves keep 32 rows, the 7^L
 * leaf products in one batched matrix-core launch (counter slot 1). The first pass checks the
 * operands: a NaN, an infinity or a magnitude above sqrt(max / (16 4^L n max(1, |alpha|))) sends the
 * call to the ordinary kernel instead (counter slot 5), as does a scratch allocation failure, which
 * first tries fewer levels. That check is one stream synchronisation per call, so the policy is
 * skipped while the stream is capturing, and for operands inside the context's scratch. AUTO uses
 * two levels from n = 8192, where they are measured 10-20 % faster than the ordinary kernel, and
 * fewer (or none) where the scratch would exceed 16 GiB; a named policy takes what it needs:
 * (3 (7/4)^L + (7/4)^(L-1)) n^2 elements, kept by the context like all of its scratch.
 * Every other product under these policies runs the ordinary kernels with ordinary rounding. */
enum camblas_cuda_algorithm {
    CAMBLAS_CUDA_AUTO = 0,
    CAMBLAS_CUDA_CLASSICAL = 1,
    CAMBLAS_CUDA_STRASSEN = 2,
    CAMBLAS_CUDA_LT = 3,
    CAMBLAS_CUDA_SYMMETRIC = 4,
    CAMBLAS_CUDA_STRASSEN_TWO = 5,
    CAMBLAS_CUDA_STRASSEN_THREE = 6,
    CAMBLAS_CUDA_STRASSEN_FOUR = 7
};

/* ref: include/camblas_cuda.h:39-42, src/cuda/backend.cu:954-1055 */
int camblas_cuda_create(int device, void *stream, camblas_cuda_context **out);
int camblas_cuda_destroy(camblas_cuda_context *context);
const char *camblas_cuda_error(const camblas_cuda_context *context);
int camblas_cuda_set_algorithm(camblas_cuda_context *context, int algorithm);

/* Column-major C = alpha op(A) op(B) + beta C, FP32 throughout (no reduced-precision matrix
 * path). beta==0 never reads C; output may not alias A or B; A/B may be NULL when alpha==0 or
 * k==0. ref: include/camblas_cuda.h:44-59, src/cuda/backend.cu:786-866 (validation order) and
 * src/cuda/decode_float.cuh:2-52 (the n==1 'T','N' GEMV shortcut under AUTO). */
int camblas_cuda_sgemm(camblas_cuda_context *context, char trans_a, char trans_b, int m, int n,
                       int k, float alpha, const float *a, int lda, const float *b, int ldb,
                       float beta, float *c, int ldc);

/* Same contract with BF16 storage, float alpha/beta, FP32 accumulation and one round-to-nearest
 * conversion to BF16. ref: include/camblas_cuda.h:64-69, src/cuda/bfloat16.cuh:11-57.
 * The linear path always arrives as ('T','N', m=out_features, n=tokens, k=in_features) with both
 * operands K-contiguous (ref: src/cuda/torch_bindings.cpp:146-199). */
int camblas_cuda_bgemm(camblas_cuda_context *context, char trans_a, char trans_b, int m, int n,
                       int k, float alpha, const void *a, int lda, const void *b, int ldb,
                       float beta, void *c, int ldc);

/* C = alpha op(A) op(B) + beta Z with the addend Z stored apart from C: an m x n column-major matrix
 * with leading dimension ldz >= m, or, with ldz == 0, one column of m values added to every column
 * of the product (the bias row of a linear layer as the 'T','N' mapping above sees it). Z is never
 * read when beta == 0 and may not overlap C; everything else as camblas_cuda_bgemm. No counterpart
 * in the reference header: its aten::addmm first copies the broadcast bias into the output and then
 * runs the beta form (ref: src/cuda/torch_backend.cuh:60-88), which costs one write and one read
 * of the whole output. */
int camblas_cuda_bgemm_add(camblas_cuda_context *context, char trans_a, char trans_b, int m, int n,
                           int k, float alpha, const void *a, int lda, const void *b, int ldb,
                           float beta, const void *z, int ldz, void *c, int ldc);

/* Same contract in FP64 (ref: include/camblas_cuda.h:60-62, src/cuda/backend.cu:1066-1073):
 * FP64 matrix-core tiles for every layout (IEEE double multiply-add); products with m or n below
 * 16 run an LDS-tiled FMA kernel. */
int camblas_cuda_dgemm(camblas_cuda_context *context, char trans_a, char trans_b, int m, int n,
                       int k, double alpha, const double *a, int lda, const double *b, int ldb,
                       double beta, double *c, int ldc);

/* Dense FP32 / FP64 helpers (dtype 0 FP32, 1 FP64), all arrays row-major, contiguous and owned by
 * the caller. Products run through the same GEMM as sgemm / dgemm; the elementwise and reduction
 * passes have a fixed order, so results repeat bit for bit.
 * affine: output[rows, columns] = x[rows, inner] . weight[inner, columns] + bias[columns], then
 *   ReLU when relu != 0 (NaN stays NaN). rows == 0 or columns == 0 succeeds without touching
 *   anything; inner == 0 yields the bias (x and weight may be null).
 *   ref: include/camblas_cuda.h:71-75, src/cuda/backend.cu:871-905, :1086-1101.
 * mlp: hidden_output = relu(x . w1 + b1), output = hidden_output . w2 + b2; the two outputs may not
 *   share storage. ref: include/camblas_cuda.h:76-78, src/cuda/backend.cu:1103-1117.
 * attention: output[queries, values] = softmax(scale . q k^T) v, single head, no mask; the scores
 *   live in context scratch (growth is refused during stream capture); keys == 0 gives zeros.
 *   ref: include/camblas_cuda.h:80-85, src/cuda/fusion.cuh:95-157, backend.cu:1495-1510.
 * mlp_backward: gradients of mlp; every non-null gradient pointer is filled; grad_hidden
 *   [rows, hidden] is caller scratch, required when dx, dw1 or db1 is requested.
 *   ref: include/camblas_cuda.h:87-94, src/cuda/fusion.cuh:207-275, backend.cu:1512-1535.
 * Launch counters: affine -> slot 3, attention -> slot 6, mlp_backward -> slot 7. */
int camblas_cuda_affine(camblas_cuda_context *context, int dtype, int rows, int inner, int columns,
                        const void *x, const void *weight, const void *bias, int relu,
                        void *output);
int camblas_cuda_mlp(camblas_cuda_context *context, int dtype, int rows, int inputs, int hidden,
                     int outputs, const void *x, const void *w1, const void *b1, const void *w2,
                     const void *b2, void *hidden_output, void *output);
int camblas_cuda_attention(camblas_cuda_context *context, int dtype, int queries, int keys,
                           int depth, int values, double scale, const void *q, const void *k,
                           const void *v, void *output);
int camblas_cuda_mlp_backward(camblas_cuda_context *context, int dtype, int rows, int inputs,
                              int hidden, int outputs, const void *x, const void *w1,
                              const void *w2, const void *hidden_output, const void *grad_output,
                              void *grad_hidden, void *dx, void *dw1, void *db1, void *dw2,
                              void *db2);

/* SiLU(gate)*up, dtype 0 FP32 / 2 BF16, intermediate rounding to the storage type.
 * ref: include/camblas_cuda.h:96-100, src/cuda/inference_fusion.cuh:19-28 */
int camblas_cuda_silu_multiply(camblas_cuda_context *context, int dtype, uint64_t count,
                               const void *gate, const void *up, void *output);
/* ref: include/camblas_cuda.h:101-109, src/cuda/inference_fusion.cuh:30-51 */
int camblas_cuda_swiglu(camblas_cuda_context *context, int dtype, uint64_t count, int width,
                        float limit, const void *gate, const void *up, const float *routing,
                        void *output);

/* Row-major RMS normalisation, rounding the normalised value to storage before the weight
 * multiply. ref: include/camblas_cuda.h:185-189, src/cuda/inference_fusion.cuh:53-86 */
int camblas_cuda_rms_norm(camblas_cuda_context *context, int dtype, int rows, int width,
                          float epsilon, const void *input, const void *weight, void *output);
/* Single row, explicit rounding policy. `descending` selects a reduction order in the reference;
 * here it is validated and otherwise has no effect (one fixed wavefront-64 order).
 * ref: include/camblas_cuda.h:190-196, src/cuda/inference_fusion.cuh:136-191 */
int camblas_cuda_rms_norm_decode(camblas_cuda_context *context, int dtype, int weight_dtype,
                                 int width, float epsilon, int round_before_weight, int descending,
                                 const void *input, const void *weight, void *output);
/* Single-row residual add + RMS norm. ref: include/camblas_cuda.h:197-202 */
int camblas_cuda_add_rms_norm(camblas_cuda_context *context, int dtype, int width, float epsilon,
                              const void *input, const void *residual, const void *weight,
                              void *added, void *output);
/* ref: include/camblas_cuda.h:203-209, src/cuda/inference_fusion.cuh:99-119 */
int camblas_cuda_bfloat16_square(camblas_cuda_context *context, uint64_t count, const void *input,
                                 float *output);
int camblas_cuda_rms_scale(camblas_cuda_context *context, int dtype, uint64_t count, int width,
                           float epsilon, const void *input, const void *weight, const float *means,
                           void *output);

/* Host launch counters, length 6 or 8: [0] classical/generic/GEMV, [1] strassen (always 0),
 * [2] gram (always 0), [3] affine (0), [4] planned MFMA GEMM ("lt"), [5] guard fallback
 * (scratch could not grow: generic kernel used), [6] attention, [7] backward (0).
 * ref: include/camblas_cuda.h:211-215, src/cuda/backend.cu:1477-1493 */
int camblas_cuda_stats(const camblas_cuda_context *context, uint64_t *counts, int length);
int camblas_cuda_reset_stats(camblas_cuda_context *context);

/* Row-major FP8 E4M3 input [rows, inner] times weight [outputs, inner]^T with E8M0 block scales,
 * FP32 accumulation, BF16 [rows, outputs]. packed=1: weights are E2M1 nibbles, low/high order,
 * [outputs, inner/2] with scales [outputs, inner/32]; packed=0: E4M3 bytes with scales
 * [ceil(outputs/32), inner/32]. Input scales are [rows, inner/activation_block]; activation_block
 * is 32 (both) or 128 (E2M1 only). outputs a positive multiple of eight, inner of 32, rows
 * 0..65535. ref: include/camblas_cuda.h:110-123, src/cuda/backend.cu:1165-1191. Runs on the
 * scaled matrix-core instruction of gfx950, which applies the E8M0 scales itself. Input and weight
 * must be 16-byte aligned here (the reference asks for 4 and 2/4); the scale arrays may start at
 * any byte. Up to 64 rows a weight-streaming kernel runs; above that, when inner is a multiple of
 * 128 and the output is 8-byte aligned, a kernel that tiles both operands through LDS. */
int camblas_cuda_quantized_matmul(camblas_cuda_context *context, int packed, int rows, int outputs,
                                  int inner, int activation_block, const void *input,
                                  const void *input_scale, const void *weight,
                                  const void *weight_scale, void *output);
/* Batched form: input [groups, rows, inner], output [groups, rows, outputs]; metadata is device
 * uint64 [weight_groups, 2] holding weight / scale addresses in the layouts above; active and
 * counts are device int32 [groups]. Invalid active indices produce zeros, counts are clipped to
 * [0, rows], padding rows are zeroed. ref: include/camblas_cuda.h:156-167,
 * src/cuda/backend.cu:1258-1303. */
int camblas_cuda_grouped_quantized_matmul(camblas_cuda_context *context, int packed, int groups,
                                          int weight_groups, int rows, int outputs, int inner,
                                          int activation_block, const void *input,
                                          const void *input_scale, const void *metadata,
                                          const void *active, const void *counts, void *output);

/* Route int64 expert IDs [tokens, choices] to local int32 active IDs [groups]: initialises counts
 * [groups], slots [groups, rows] and reverse [tokens, choices]; unassigned slots / reverse are -1,
 * rows beyond `rows` are discarded (counts still counts them), duplicate active IDs select their
 * first group, IDs outside [first_expert, INT_MAX) are ignored.
 * ref: include/camblas_cuda.h:168-176, src/cuda/backend.cu:1306-1337. Rows of a group are handed
 * out in ascending slot order (the reference's order depends on its atomic counter). */
int camblas_cuda_route_groups(camblas_cuda_context *context, int tokens, int choices,
                              int first_expert, int groups, int rows, const void *experts,
                              const void *active, void *counts, void *slots, void *reverse);
/* Sum BF16 grouped rows in ascending expert-ID / choice order into FP32 [tokens, width]; reverse
 * maps [tokens, choices] to rows of input [grouped_rows, width]; negative or out-of-range expert
 * IDs and rows are ignored; choices is 1..64.
 * ref: include/camblas_cuda.h:177-185, src/cuda/backend.cu:1339-1361. */
int camblas_cuda_reduce_groups(camblas_cuda_context *context, int tokens, int choices, int width,
                               int grouped_rows, const void *experts, const void *reverse,
                               const void *input, void *output);

/* Single-token FP8 E4M3 [inner] times contiguous [outputs, inner] weights with 32-wide scale
 * blocks: FP32 input scales [inner/32] and weight scales [ceil(outputs/32), inner/32] with
 * positive element strides; sum = fma(dot_b * weight_scale, input_scale, sum) for b ascending, BF16
 * out [outputs]. inner a multiple of 32 in [32, 8192], outputs a positive multiple of 16.
 * ref: include/camblas_cuda.h:124-155, src/cuda/backend.cu:1193-1256, src/cuda/fp8_decode.cuh:150-157.
 * camblas_cuda_fp8_linear takes a BF16 token and quantises it per block with the power-of-two
 * scale 2^ceil(log2(max(|x|, 1e-10) / 448)) (ref: src/cuda/fp8_decode.cuh:58-72). Both run as one
 * kernel: the workspace query returns 0 and the workspace arguments are ignored. The weight must be
 * 16-byte aligned here (the reference asks for 4). */
int camblas_cuda_fp8_decode_supported(const camblas_cuda_context *context);
int camblas_cuda_fp8_decode(camblas_cuda_context *context, int outputs, int inner,
                            const void *input, const float *input_scale, const void *weight,
                            const float *weight_scale, int input_scale_stride,
                            int weight_scale_row_stride, int weight_scale_column_stride,
                            void *workspace, size_t workspace_bytes, void *output);
size_t camblas_cuda_fp8_workspace_size(int quantise, int outputs, int inner);
int camblas_cuda_fp8_linear(camblas_cuda_context *context, int outputs, int inner,
                            const void *input, const void *weight, const float *weight_scale,
                            int weight_scale_row_stride, int weight_scale_column_stride,
                            void *workspace, size_t workspace_bytes, void *output);

/* ------------------------------------------------------------------ extensions */

/* extension. FP8 E4M3fn block-scaled linear: a [rows, inner] bytes with FP32 scales
 * [rows, inner/128] (one per 1x128 group), w [outputs, inner] bytes with FP32 scales
 * [ceil(outputs/128), inner/128] (one per 128x128 block), BF16 out [rows, outputs].
 * Arithmetic rule (ref: camblas/_hopper.py:118-126 and :168-182, which implement it for rows==1):
 * per 128-wide K group the unscaled FP32 dot product, then
 * acc = fma(dot_g, a_scale[r,g] * w_scale[n/128,g], acc) for g ascending, one BF16 rounding.
 * inner is a positive multiple of 128, outputs >= 1, rows 0..65535; a, w 16-byte aligned. */
int camblas_cuda_fp8_block_matmul(camblas_cuda_context *context, int rows, int outputs, int inner,
                                  const void *a_fp8, const float *a_scale, const void *w_fp8,
                                  const float *w_scale, void *out_bf16);
/* extension. Dynamic 1x128 activation quantiser (ref: camblas/_hopper.py:82-98): amax =
 * max(|x|, 1e-10) per group, scale = amax/448, q = e4m3(clamp(x * (448/amax), +-448)). */
int camblas_cuda_fp8_quantise_1x128(camblas_cuda_context *context, int rows, int inner,
                                    const void *x_bf16, void *q_fp8, float *scale);
/* extension. BF16 input, quantised on the fly, then the product above. `workspace` holds the
 * quantised activations: rows*inner bytes + rows*(inner/128) floats, 16-byte aligned. */
size_t camblas_cuda_fp8_block_workspace_size(int rows, int inner);
int camblas_cuda_fp8_block_linear(camblas_cuda_context *context, int rows, int outputs, int inner,
                                  const void *x_bf16, const void *w_fp8, const float *w_scale,
                                  void *workspace, size_t workspace_bytes, void *out_bf16);

/* extension. Multi-row residual add + RMS norm with the arithmetic of camblas_cuda_add_rms_norm
 * (ref: src/cuda/inference_fusion.cuh:136-191) applied to each of `rows` rows; residual may be
 * NULL (plain norm, `added` ignored). weight_dtype 0 FP32 / 2 BF16. */
int camblas_cuda_add_rms_norm_rows(camblas_cuda_context *context, int dtype, int weight_dtype,
                                   int rows, int width, float epsilon, int round_before_weight,
                                   const void *input, const void *residual, const void *weight,
                                   void *added, void *output);

/* extension (no reference counterpart; the reference leaves RoPE and KV-cache attention to the
 * serving engine, configs/sglang.json:44). Rotate-half rotary embedding in place on BF16
 * x [tokens, heads, dim] whose token stride is token_stride elements; positions int32 [tokens]. */
int camblas_cuda_rope(camblas_cuda_context *context, int tokens, int heads, int dim,
                      int token_stride, float theta, const int32_t *positions, void *x_bf16);
/* extension. The front end of a gated MLP for a decode batch (at most 64 rows) in one streaming pass
 * over both weight matrices: out[rows, outputs] = silu_multiply(x gate^T, x up^T), BF16 storage,
 * FP32 accumulation, with the rounding points of the composition the reference's binding makes from
 * two linears and camblas_cuda_silu_multiply (src/cuda/torch_bindings.cpp:703-723,
 * src/cuda/inference_fusion.cuh:19-28): g = bf16(x gate^T), u = bf16(x up^T),
 * out = bf16(bf16(silu(g)) * u). x [rows, inner] with row stride ldx, gate and up [outputs, inner]
 * with row stride ldw, out with row stride ldo (elements). inner, ldx and ldw multiples of 8;
 * x, gate, up 16-byte aligned. More than 64 rows are refused: compose the three calls instead. */
int camblas_cuda_bf16_gated_linear(camblas_cuda_context *context, int rows, int outputs, int inner,
                                   const void *x, int ldx, const void *gate, const void *up, int ldw,
                                   void *out, int ldo);
/* extension (no reference counterpart). camblas_cuda_rope_kv_append and
 * camblas_cuda_gqa_decode_attention in one call, two launches instead of three: qkv holds the step's
 * un-rotated activation rows [q heads | k heads | v heads] (token_stride elements apart, a multiple
 * of 8), positions[b] the cache slot of sequence b's new token. The queries are rotated in registers
 * by every workgroup that needs them, the new K row is rotated by the workgroup whose positions
 * hold its slot, which also writes it and the new V row into the caches and attends to them; the
 * attention covers positions[b] + 1 entries. Output and caches equal the two separate calls bit for
 * bit (lengths = positions + 1); qkv itself is left unrotated. A position outside [0, context_length)
 * appends nothing (the attention then covers min(positions + 1, context_length) entries, none if
 * negative). angles: NULL, or what camblas_cuda_rope_angles made for these positions and theta. */
int camblas_cuda_rope_append_gqa_decode_attention(camblas_cuda_context *context, int batch, int q_heads,
                                                  int kv_heads, int dim, int context_length,
                                                  const int32_t *positions, float theta, float scale,
                                                  const void *qkv_bf16, int token_stride, void *k_cache,
                                                  void *v_cache, const float *angles, void *output);
/* extension (no reference counterpart). The rotation angles of one decode step, which are the same
 * for every layer of a model: angles[b][0][i] = sin, angles[b][1][i] = cos of positions[b] *
 * theta^(-2i/dim) for i < dim / 2 (FP32 [batch][2][dim / 2]), exactly the values the rotary kernels
 * work out themselves. camblas_cuda_rope_append_gqa_decode_attention takes them as `angles` (made with
 * the same positions and theta; NULL: every workgroup works them out). */
int camblas_cuda_rope_angles(camblas_cuda_context *context, int batch, int dim, float theta,
                             const int32_t *positions, float *angles);
/* extension. The residual-add + RMSNorm between two decode linears, moved into those linears (the
 * arithmetic and its rounding points are the reference's norm, src/cuda/inference_fusion.cuh:136-191,
 * binding src/cuda/torch_bindings.cpp:675-701: added = bf16(x + r), scale = rsqrt(mean(added^2) + eps),
 * out = bf16(bf16(added * scale) * weight)). The linear BEFORE the norm:
 *   added[tokens, outputs] = bf16(bf16(x w^T) + residual), and for every workgroup g along the outputs
 *   squares[g * squares_ld + token] = the sum of added^2 over g's outputs (fixed order);
 *   *squares_count (host) receives the number of such workgroups; it depends on the shape and the
 *   device only. squares needs room for squares_capacity >= that many rows of squares_ld >= tokens
 *   floats (ceil(outputs / 16) rows always suffice), else the call is refused.
 * At most 64 tokens; inner, ldx, ldw multiples of 8; x and w 16-byte aligned. */
int camblas_cuda_bf16_linear_residual(camblas_cuda_context *context, int tokens, int outputs, int inner,
                                      const void *x, int ldx, const void *w, int ldw, const void *residual,
                                      int ld_residual, void *added, int ld_added, float *squares, int squares_ld,
                                      int squares_capacity, int *squares_count);
/* extension. The linear AFTER the norm: y = bf16(normalised(x) w^T) where x holds the un-normalised
 * rows (`added` above), squares [squares_count][squares_ld] their partial sums of squares (added in
 * index order; mean = sum / inner) and norm_weight the BF16 norm weights [inner], 16-byte aligned. The
 * tokens are normalised while the kernel stages them, so the normalised rows never exist in memory.
 * Same shape limits as above. */
int camblas_cuda_bf16_rms_linear(camblas_cuda_context *context, int tokens, int outputs, int inner, const void *x,
                                 int ldx, const float *squares, int squares_ld, int squares_count,
                                 const void *norm_weight, float epsilon, const void *w, int ldw, void *y, int ldy);
/* extension. camblas_cuda_bf16_gated_linear with the same fused normalisation of its input. */
int camblas_cuda_bf16_rms_gated_linear(camblas_cuda_context *context, int rows, int outputs, int inner,
                                       const void *x, int ldx, const float *squares, int squares_ld,
                                       int squares_count, const void *norm_weight, float epsilon, const void *gate,
                                       const void *up, int ldw, void *out, int ldo);
/* extension. The state those calls pass along, made from scratch (a model's first layer): added
 * [rows, width] = bf16(x + residual), squares[row] = the sum of added^2 over the row (one partial
 * sum per row: squares_count 1, squares_ld >= rows). BF16, contiguous rows. */
int camblas_cuda_add_residual_squares(camblas_cuda_context *context, int rows, int width, const void *x,
                                      const void *residual, void *added, float *squares);
/* extension (no reference counterpart). Writes each sequence's new K and V heads, rows of k_new /
 * v_new [batch, kv_heads*dim] with row stride token_stride elements (e.g. slices of a fused QKV
 * activation), into the caches [batch, context, kv_heads, dim] at positions[batch]; positions
 * outside [0, context) are skipped. dim % 8 == 0, 16-byte aligned buffers. */
int camblas_cuda_kv_append(camblas_cuda_context *context, int batch, int kv_heads, int dim,
                           int context_length, const int32_t *positions, const void *k_new,
                           const void *v_new, int token_stride, void *k_cache, void *v_cache);
/* extension (no reference counterpart). camblas_cuda_rope on the q and k heads of a fused QKV
 * activation [batch, (q_heads + 2*kv_heads)*dim] (row stride token_stride) followed by
 * camblas_cuda_kv_append of its k and v heads, in one launch and with the same results. */
int camblas_cuda_rope_kv_append(camblas_cuda_context *context, int batch, int q_heads, int kv_heads,
                                int dim, int token_stride, float theta, const int32_t *positions,
                                void *qkv_bf16, int context_length, void *k_cache, void *v_cache);
/* extension. Grouped-query decode attention, one query per sequence: q [batch, q_heads, dim]
 * (token stride q_stride elements), K/V caches [batch, context, kv_heads, dim] BF16, lengths int32
 * [batch] or NULL (= context), out [batch, q_heads, dim] BF16. dim must be 128, q_heads a
 * multiple of kv_heads with ratio <= 16. Split-K over the context with an ordered combine;
 * partials live in context scratch. */
int camblas_cuda_gqa_decode_attention(camblas_cuda_context *context, int batch, int q_heads,
                                      int kv_heads, int dim, int context_length,
                                      const int32_t *lengths, float scale, const void *q,
                                      int q_stride, const void *k_cache, const void *v_cache,
                                      void *output);
/* No counterpart in the reference. camblas_cuda_gqa_decode_attention for callers that cannot
 * allocate device memory (code under HIP graph capture on a context that has not grown its scratch
 * yet, tight serving loops, harnesses that forbid hipMalloc): same arguments, same kernels, same
 * results, but the split partials live in a fixed 16 MiB device array inside the library instead
 * of context scratch, and the call performs no hipMalloc / hipFree. A call whose partials
 * (batch * q_heads * ceil(context_length / 256) * 520 bytes) exceed
 * camblas_cuda_gqa_decode_attention_noalloc_limit() fails with a message and launches nothing.
 * Every GPU holds one such array for the life of the process and all contexts on that GPU share
 * it: calls that overlap in time on one GPU (different streams or threads) race. Nothing in it
 * has to start at zero: each call writes every partial it later reads. */
int camblas_cuda_gqa_decode_attention_noalloc(camblas_cuda_context *context, int batch, int q_heads,
                                              int kv_heads, int dim, int context_length,
                                              const int32_t *lengths, float scale, const void *q,
                                              int q_stride, const void *k_cache,
                                              const void *v_cache, void *output);
size_t camblas_cuda_gqa_decode_attention_noalloc_limit(void);

/* extension (the reference runs this step from Python on Triton kernels, camblas/_hopper.py:329-401,
 * behind its SGLang hook camblas/sglang.py:340-455; here it is an entry point like the other
 * products). One BF16 token x [hidden] through a mixture-of-experts layer with E4M3 weights and
 * FP32 scales per 128 x 128 block: w1 [experts, 2*width, hidden] (gate rows, then up rows) with
 * w1_scale [experts, 2*width/128, hidden/128], w2 [experts, hidden_out, width] with w2_scale
 * [experts, ceil(hidden_out/128), width/128], expert_ids int32 [choices] and routing FP32
 * [choices] on the device. Per choice: x quantised per 128 inputs (amax/448), gate/up product
 * rounded to BF16, silu(min(gate, 10)) * clamp(up, -10, 10) rounded to BF16 and quantised per 128,
 * down product times the routing weight rounded to BF16; the choices are summed in order and the
 * sum times `factor` is rounded to BF16 into output [hidden_out], which may be x itself.
 * hidden and width multiples of 128, hidden_out of 16, 1..16 choices, choices * width / 128 at
 * most 512. Uses context scratch. */
int camblas_cuda_fp8_moe_decode(camblas_cuda_context *context, int experts, int choices, int hidden,
                                int width, int hidden_out, const void *x, const void *w1,
                                const float *w1_scale, const void *w2, const float *w2_scale,
                                const int32_t *expert_ids, const float *routing, float factor,
                                void *output);

/* extension. Planner introspection (the GPU counterpart of the reference CPU planner's
 * camblas_plan_format, src/planner.c:654-669): writes a one-line description of the kernel the
 * planner picks for a GEMM call into `text` and returns 1000 * family + variant (>=0) without touching a
 * device. dtype 0 FP32, 2 BF16, 3 FP8-block. Pure host function: works without a GPU. */
int camblas_hip_plan_describe(int dtype, int algorithm, char trans_a, char trans_b, int m, int n,
                              int k, int lda, int ldb, int ldc, int aligned16, char *text,
                              size_t text_bytes);
/* extension. Diagnostics for tests and tuning: force the planner's choice for BF16/FP8 GEMMs on
 * this context (kernel < 0 restores the planner; split_k <= 0 lets the planner choose). For the
 * E8M0 products: 0 the weight-streaming kernel, 20 / 21 / 22 / 23 the tiled kernel with
 * 256 x 256, 256 x 128, (E4M3 weights only) 192 x 256 and 128 x 128 tiles, 24 the four-wavefront
 * 192 x 256 tile (grouped calls: E4M3 weights only); a forced kernel that cannot run the call makes
 * the call fail. (BF16: 100 + 100 d + 10 r + t the weight-streaming kernel with 2^d K blocks per
 * step, r row tiles and t token tiles of 16 (t up to 8, above 4 with d = 0 only); 20 + n the
 * direct-to-LDS tile n, of which 38 / 39 are the four-wavefront 256- and 320-row tiles and 40 the
 * 256-row tile for weights stored with their outputs contiguous; FP8 with FP32 scales: 36 the
 * four-wavefront 192 x 256 tile; the single-token product with 32-wide scale blocks: 301 / 302 / 304
 * one, two or four wavefronts per workgroup.)
 * TEST-ONLY: the override is state of the context it is set on (no other context sees it, and it
 * ends with the context), it bypasses the planner's eligibility rules, and a forced variant may be
 * far slower than the planner's choice or refuse shapes the planner would serve. Serving code never
 * calls it; nothing in the library or its Python surface sets it outside the test suite. */
int camblas_hip_set_plan_override(camblas_cuda_context *context, int kernel, int split_k);
/* extension. Number of kernel variants `camblas_hip_set_plan_override` accepts for a dtype. */
int camblas_hip_kernel_count(int dtype);

#ifdef __cplusplus
}
#endif
#endif
