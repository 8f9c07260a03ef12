// The GEMM family of the C ABI: sgemm / dgemm / bgemm and the FP32 / FP64 helpers composed from them
// (affine, mlp, dense attention, mlp_backward). Argument rules and their order follow the
// reference (src/cuda/backend.cu:786-866 for the dense product, src/cuda/bfloat16.cuh:11-57 for
// BF16, :871-905 and src/cuda/fusion.cuh:95-157, :207-275 for the helpers); every kernel is this
// library's own.
#include "entry.hpp"

#include <algorithm>
#include <cmath>
#include <limits>

namespace camblas_hip
{
namespace
{
// The shape part of a column-major product C[m, n] = alpha op(A) op(B) + beta C.
struct Product {
    int trans_a, trans_b; // 0 'N', 1 'T', -1 neither
    int m, n, k, lda, ldb, ldc;

    Product(char ta, char tb, int m_, int n_, int k_, int lda_, int ldb_, int ldc_)
        : trans_a(transposition(ta)), trans_b(transposition(tb)), m(m_), n(n_), k(k_), lda(lda_),
          ldb(ldb_), ldc(ldc_)
    {
    }
    bool well_formed() const
    {
        return trans_a >= 0 && trans_b >= 0 && m >= 0 && n >= 0 && k >= 0 && lda >= 1 && ldb >= 1 && ldc >= 1;
    }
    bool empty() const { return m == 0 || n == 0; }
    // a leading dimension covers the stored rows of its operand (at least 1)
    bool strides_cover() const
    {
        return lda >= std::max(1, trans_a ? k : m) && ldb >= std::max(1, trans_b ? n : k) && ldc >= m;
    }
};

// What the three GEMM entry points share: the reference's order of checks. `names` are the three
// failure texts (arguments, output/strides, operands). Returns 1 when the caller should go on to
// launch the product, 0 when the call is complete, negative on failure.
template <typename Scalar, typename ScaleOutput>
int admit_product(const Entry &entry, const Product &p, Scalar alpha, Scalar beta, const void *a,
                  const void *b, const void *c, const char *const (&names)[4], ScaleOutput scale_output)
{
    if (!p.well_formed())
        return entry.refuse(names[0]);
    if (p.empty())
        return 0;
    if (!c || !p.strides_cover())
        return entry.refuse(names[1]);
    if (alpha == Scalar(0) || p.k == 0) { // only beta acts; beta == 0 writes zeros without reading C
        if (beta == Scalar(1))
            return 0;
        return entry.finish(scale_output(), names[2]);
    }
    if (!a || !b || a == c || b == c)
        return entry.refuse(names[3]);
    return 1;
}

// C = A A^T or A^T A over the whole of C under the symmetric policy (ref: backend.cu:819-835): the
// tiles that reach the diagonal are computed and the rest mirrored, so C equals its transpose
// bit for bit.
bool is_gram(const camblas_cuda_context *context, const Product &p, const void *a, const void *b,
             bool overwrites)
{
    return context->algorithm == CAMBLAS_CUDA_SYMMETRIC && a == b && p.trans_a != p.trans_b &&
           p.m == p.n && p.lda == p.ldb && overwrites;
}

// square, untransposed, even, at least 256: the products the Strassen policies split
// (ref: backend.cu:843-853)
int strassen_depth(const camblas_cuda_context *context, const Product &p)
{
    if (p.trans_a || p.trans_b || p.m != p.n || p.n != p.k || p.n % 2 || p.n < 256)
        return 0;
    return strassen_levels(context->algorithm, p.n);
}

template <typename T> struct Kernels;

template <> struct Kernels<float> {
    static constexpr int dtype = 0;
    static hipError_t scale(hipStream_t s, const Product &p, float beta, float *c)
    {
        return launch_scale_f32(s, p.m, p.n, beta, c, p.ldc);
    }
    static hipError_t vector(hipStream_t s, const Product &p, float alpha, const float *a, const float *b,
                             float beta, float *c)
    {
        return launch_generic_f32(s, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a, p.lda, b, p.ldb, beta, c,
                                  p.ldc);
    }
    static bool matrix_worthwhile(const Product &p) { return p.m >= 32 && p.k >= 16; }
    // 128 x 128 tiles once the tiles that reach the diagonal number two per compute unit
    static hipError_t triangle(const camblas_cuda_context *context, const Product &p, float alpha,
                               const float *a, const float *b, float beta, float *c)
    {
        const double rows = (p.n + 127) / 128;
        const bool wide = rows * (rows + 1) / 2 >= 2.0 * context->compute_units;
        return launch_sgemm_mfma(context->stream, wide, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a, p.lda,
                                 b, p.ldb, beta, c, p.ldc, 1, 0, true);
    }
};

template <> struct Kernels<double> {
    static constexpr int dtype = 1;
    static hipError_t scale(hipStream_t s, const Product &p, double beta, double *c)
    {
        return launch_scale_f64(s, p.m, p.n, beta, c, p.ldc);
    }
    static hipError_t vector(hipStream_t s, const Product &p, double alpha, const double *a, const double *b,
                             double beta, double *c)
    {
        return launch_generic_f64(s, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a, p.lda, b, p.ldb, beta, c,
                                  p.ldc);
    }
    static bool matrix_worthwhile(const Product &p) { return p.m >= 16 && p.k >= 4; }
    static hipError_t triangle(const camblas_cuda_context *context, const Product &p, double alpha,
                               const double *a, const double *b, double beta, double *c)
    {
        return launch_dgemm_mfma(context->stream, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a, p.lda, b, p.ldb,
                                 beta, c, p.ldc, 1, 0, true);
    }
};

// The planner's choice for an ordinary FP32 product, with any forced kernel applied.
Plan fp32_plan(const camblas_cuda_context *context, const Product &p, const float *a, const float *b)
{
    Plan plan = make_plan(0, context->algorithm, p.trans_a, p.trans_b, p.m, p.n, p.k, p.lda, p.ldb, p.ldc,
                          is_aligned(a, 16) && is_aligned(b, 16), context->compute_units);
    if (plan.family != FAMILY_GEMV_F32 && context->override_kernel >= 0) {
        // tests: 0 vector-ALU tiles, 1 / 2 matrix-core tiles
        plan.family = context->override_kernel >= 1 ? FAMILY_MFMA_F32 : FAMILY_GENERIC;
        plan.kernel = context->override_kernel == 2 ? 1 : 0;
        plan.split_k = 1;
    }
    if (plan.family != FAMILY_MFMA_F32)
        plan.split_k = 1;
    return plan;
}

// Into how many workgroups per tile an ordinary FP64 product divides K, and the tile width: a
// handful of columns against a large A would occupy a fraction of the compute units with the
// 128 x 128 tiles alone (the FP32 rule with this kernel's tiles: up to 32 columns tiles of
// 128 x 16, up to 64 of 128 x 64, and four workgroups per compute unit).
struct Fp64Plan {
    bool matrix;
    int shares, tile_columns;
};
Fp64Plan fp64_plan(const camblas_cuda_context *context, const Product &p)
{
    // (fewer than 16 columns against a large A still go to the tiles: with K divided they run at
    // five times the rate of the vector-ALU kernel, whose grid would be a few dozen workgroups)
    Fp64Plan plan{p.m >= 16 && (p.n >= 16 || (p.m >= 256 && p.k >= 512)) && p.k >= 4, 1,
                  p.n <= 32 ? 16 : p.n <= 64 ? 64 : 128};
    if (context->override_kernel >= 0) // tests: 0 vector-ALU tiles, else matrix-core tiles
        plan.matrix = context->override_kernel >= 1;
    const bool narrow = plan.tile_columns < 128;
    if (plan.matrix && context->override_kernel < 0 && p.m >= 256 && p.k >= 512) {
        const long long tiles =
            (long long)((p.m + 127) / 128) * ((p.n + plan.tile_columns - 1) / plan.tile_columns);
        for (int s : {32, 16, 8, 4, 2})
            if (tiles * s <= (narrow ? 4LL : 2LL) * context->compute_units && p.k % s == 0 && p.k / s >= 256) {
                plan.shares = s;
                break;
            }
    }
    return plan;
}

// Bytes of FP32 / FP64 planes the ordinary product of this shape would claim (0: K undivided).
size_t plane_bytes(const camblas_cuda_context *context, const Product &p, const float *a, const float *b)
{
    const int shares = fp32_plan(context, p, a, b).split_k;
    return shares > 1 ? size_t(shares) * size_t(p.m) * size_t(p.n) * sizeof(float) : 0;
}
size_t plane_bytes(const camblas_cuda_context *context, const Product &p, const double *, const double *)
{
    const int shares = fp64_plan(context, p).shares;
    return shares > 1 ? size_t(shares) * size_t(p.m) * size_t(p.n) * sizeof(double) : 0;
}

// the ordinary FP32 product: the planner's choice (decode GEMV, matrix-core tiles, vector-ALU tiles)
int ordinary(const Entry &entry, const Product &p, float alpha, const float *a, const float *b, float beta,
             float *c, bool classical_counter)
{
    camblas_cuda_context *context = entry.context();
    const Plan plan = fp32_plan(context, p, a, b);
    context->counts[classical_counter ? 0 : plan.counter]++;
    if (plan.family == FAMILY_GEMV_F32)
        return entry.finish(launch_gemv_f32(context->stream, p.m, p.k, alpha, a, p.lda, b, beta, c),
                            "FP32 native GEMV");
    if (plan.split_k > 1) {
        // without room for the planes (allocation failure, capture in progress, an enclosing
        // helper holding the arena) K stays undivided
        if (void *planes = claim_scratch(context, size_t(plan.split_k) * size_t(p.m) * size_t(p.n) * 4))
            return entry.finish(launch_sgemm_mfma_divided(context->stream, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a,
                                                          p.lda, b, p.ldb, beta, c, p.ldc, plan.split_k,
                                                          static_cast<float *>(planes), plan.kernel == 2),
                                "classical GEMM");
        context->counts[5]++;
    }
    const hipError_t launched =
        plan.family == FAMILY_MFMA_F32
            ? launch_sgemm_mfma(context->stream, plan.kernel == 0, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha,
                                a, p.lda, b, p.ldb, beta, c, p.ldc)
            : Kernels<float>::vector(context->stream, p, alpha, a, b, beta, c);
    return entry.finish(launched, "classical GEMM");
}

// the ordinary FP64 product: matrix cores when every dimension holds a 16 x 16 x 4 tile, K divided
// over workgroups when the tiles alone would leave most compute units idle
// (ref: backend.cu:1066-1073)
int ordinary(const Entry &entry, const Product &p, double alpha, const double *a, const double *b,
             double beta, double *c, bool)
{
    camblas_cuda_context *context = entry.context();
    context->counts[0]++;
    const Fp64Plan plan = fp64_plan(context, p);
    if (plan.shares > 1) {
        // without room for the planes (allocation failure, capture in progress, an enclosing
        // helper holding the arena) K stays undivided
        if (void *planes = claim_scratch(context, size_t(plan.shares) * size_t(p.m) * size_t(p.n) * 8))
            return entry.finish(launch_dgemm_mfma_divided(context->stream, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha,
                                                          a, p.lda, b, p.ldb, beta, c, p.ldc, plan.shares,
                                                          static_cast<double *>(planes), plan.tile_columns),
                                "classical FP64 GEMM");
        context->counts[5]++;
    }
    const hipError_t launched =
        plan.matrix ? launch_dgemm_mfma(context->stream, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a, p.lda, b,
                                        p.ldb, beta, c, p.ldc)
                    : Kernels<double>::vector(context->stream, p, alpha, a, b, beta, c);
    return entry.finish(launched, "classical FP64 GEMM");
}

// FP32 / FP64 product on the entry's stream: policies first (symmetric, Strassen), then the
// ordinary kernels. Shared by the public entry points and by the helpers below.
template <typename T>
int dense_product(const Entry &entry, const Product &p, T alpha, const T *a, const T *b, T beta, T *c)
{
    static const char *const names[4] = {"invalid GEMM arguments",
                                         "invalid device pointer or leading dimension", "scale output",
                                         "missing or aliased GEMM operand"};
    camblas_cuda_context *context = entry.context();
    const int admitted = admit_product(entry, p, alpha, beta, a, b, c, names,
                                       [&] { return Kernels<T>::scale(context->stream, p, beta, c); });
    if (admitted <= 0)
        return admitted;
    if (is_gram(context, p, a, b, beta == T(0))) {
        context->counts[2]++;
        const hipError_t lower = Kernels<T>::matrix_worthwhile(p)
                                     ? Kernels<T>::triangle(context, p, alpha, a, b, beta, c)
                                     : Kernels<T>::vector(context->stream, p, alpha, a, b, beta, c);
        if (lower != hipSuccess)
            return entry.refuse("symmetric Gram", int(lower));
        return entry.finish(launch_mirror_lower(context->stream, Kernels<T>::dtype, p.n, c, p.ldc),
                            "Gram mirroring");
    }
    bool guarded = false; // the Strassen guard sent the call here: it counts as a classical product
    if (const int depth = strassen_depth(context, p)) {
        const int outcome = strassen_gemm(context, depth, p.n, alpha, a, p.lda, b, p.ldb, beta, c, p.ldc);
        if (outcome != STRASSEN_FALL_BACK && outcome != STRASSEN_NOT_ELIGIBLE)
            return outcome;
        guarded = outcome == STRASSEN_FALL_BACK;
    }
    return ordinary(entry, p, alpha, a, b, beta, c, guarded);
}

// Row-major out[rows, columns] = x[rows, inner] weight[inner, columns] + bias, optional ReLU
// (ref: backend.cu:871-905): the column-major product out^T = weight^T-view x^T-view, then one
// bias / activation pass.
template <typename T>
int affine_layer(const Entry &entry, int rows, int inner, int columns, const T *x, const T *weight,
                 const T *bias, bool relu, T *output)
{
    if (rows < 0 || inner < 0 || columns < 0)
        return entry.refuse("invalid affine dimensions");
    if (rows == 0 || columns == 0)
        return 0;
    if (!output || !bias || (inner > 0 && (!x || !weight)))
        return entry.refuse("missing affine operand");
    entry.context()->counts[3]++;
    const Product p('N', 'N', columns, rows, inner, std::max(1, columns), std::max(1, inner), columns);
    if (const int status = dense_product(entry, p, T(1), weight, x, T(0), output))
        return status;
    return entry.finish(launch_bias_activation(entry.stream(), Kernels<T>::dtype, output, bias,
                                               size_t(rows) * columns, columns, relu),
                        "bias/activation");
}

// softmax(scale q k^T) v with the score matrix in the context's scratch (ref: fusion.cuh:95-157)
template <typename T>
int score_attention(const Entry &entry, int queries, int keys, int depth, int values, T scale, const T *q,
                    const T *k, const T *v, T *output)
{
    if (queries < 0 || keys < 0 || depth < 0 || values < 0)
        return entry.refuse("invalid attention dimensions");
    if (queries == 0 || values == 0)
        return 0;
    if (!output || (depth > 0 && !q) || (keys > 0 && depth > 0 && !k) || (keys > 0 && !v))
        return entry.refuse("missing attention operand");
    if (keys > 0 && size_t(queries) > std::numeric_limits<size_t>::max() / sizeof(T) / size_t(keys))
        return entry.refuse("attention scratch size overflow", 2);
    camblas_cuda_context *context = entry.context();
    context->counts[6]++;
    const int depth_ld = std::max(1, depth), keys_ld = std::max(1, keys), values_ld = std::max(1, values);
    const Product score('T', 'N', keys, queries, depth, depth_ld, depth_ld, keys_ld);
    const Product mix('N', 'N', values, queries, keys, values_ld, keys_ld, values_ld);
    // One reservation for the scores and, behind them, the planes of whichever of the two
    // products divides K: the scores stay live across both, so the arena must not move or be
    // handed out again in between. (If the larger request cannot be met, the scores alone are
    // reserved and the products run undivided.)
    const size_t own = size_t(queries) * keys * sizeof(T);
    const size_t behind = std::max(plane_bytes(context, score, k, q), plane_bytes(context, mix, v, static_cast<const T *>(nullptr)));
    hipError_t grown = hipErrorOutOfMemory;
    if (behind)
        grown = reserve_scratch(context, (own + 255) / 256 * 256 + behind);
    if (grown != hipSuccess)
        grown = reserve_scratch(context, own);
    if (grown != hipSuccess)
        return entry.refuse("attention scratch", int(grown));
    T *scores = static_cast<T *>(context->scratch);
    const ScratchHold hold(context, std::max<size_t>(own, 1));
    // scores[queries, keys] = q k^T; with no keys the second product just writes zeros
    if (const int status = dense_product(entry, score, T(1), k, q, T(0), scores))
        return status;
    const hipError_t softened =
        launch_softmax_rows(context->stream, Kernels<T>::dtype, scores, queries, keys, double(scale));
    if (softened != hipSuccess)
        return entry.refuse("attention softmax", int(softened));
    return dense_product(entry, mix, T(1), v, scores, T(0), output);
}

// Gradients of output = relu(x w1 + b1) w2 + b2 (ref: fusion.cuh:207-275). A null gradient pointer
// skips that gradient; grad_hidden is the caller's scratch and is left holding the masked gradient.
template <typename T> struct BackwardPass {
    const Entry &entry;
    int rows, inputs, hidden, outputs;
    const T *x, *w1, *w2, *h, *grad;
    T *dh, *dx, *dw1, *db1, *dw2, *db2;

    // column sums run over chunks of 128 rows; more than one chunk goes through context scratch
    int chunks() const
    {
        return int(std::min<size_t>(65535, std::max<size_t>(1, (size_t(rows) + 127) / 128)));
    }
    int product(char ta, char tb, int m, int n, int k, const T *a, int lda, const T *b, int ldb, T *c,
                int ldc) const
    {
        return dense_product(entry, Product(ta, tb, m, n, k, std::max(1, lda), std::max(1, ldb), std::max(1, ldc)),
                             T(1), a, b, T(0), c);
    }
    int run() const
    {
        if (rows < 0 || inputs < 0 || hidden < 0 || outputs < 0)
            return entry.refuse("invalid backward dimensions");
        const bool first_layer = dx || dw1 || db1;
        const bool needs_output_gradient = rows > 0 && outputs > 0;
        const bool needs_hidden = rows > 0 && hidden > 0 && first_layer;
        if ((needs_output_gradient && !grad) || (needs_hidden && (!dh || !h)))
            return entry.refuse("missing backward operand");
        camblas_cuda_context *context = entry.context();
        context->counts[7]++;
        const int parts = chunks(), part_rows = std::max(1, int((int64_t(rows) + parts - 1) / parts));
        T *partial = nullptr;
        size_t own = 0;
        if (parts > 1 && ((db2 && outputs > 0) || (db1 && hidden > 0))) {
            // the column-sum partials stay live across the products below: one reservation for
            // them and, behind them, the largest set of planes any of those products divides K into
            own = size_t(parts) * std::max(hidden, outputs) * sizeof(T);
            size_t behind = 0;
            auto planes = [&](char ta, char tb, int m, int n, int k, const T *a, int lda, const T *b, int ldb, int ldc) {
                if (m > 0 && n > 0 && k > 0)
                    behind = std::max(behind, plane_bytes(context, Product(ta, tb, m, n, k, std::max(1, lda), std::max(1, ldb), std::max(1, ldc)), a, b));
            };
            if (dw2)
                planes('N', 'T', outputs, hidden, rows, grad, outputs, h, hidden, outputs);
            if (first_layer) {
                planes('T', 'N', hidden, rows, outputs, w2, outputs, grad, outputs, hidden);
                if (dw1)
                    planes('N', 'T', hidden, inputs, rows, dh, hidden, x, inputs, hidden);
                if (dx)
                    planes('T', 'N', inputs, rows, hidden, w1, hidden, dh, hidden, inputs);
            }
            hipError_t grown = hipErrorOutOfMemory;
            if (behind)
                grown = reserve_scratch(context, (own + 255) / 256 * 256 + behind);
            if (grown != hipSuccess)
                grown = reserve_scratch(context, own);
            if (grown != hipSuccess)
                return entry.refuse("backward scratch", int(grown));
            partial = static_cast<T *>(context->scratch);
        }
        const ScratchHold hold(context, own);
        // second layer: dw2[hidden, outputs] = h^T grad, db2 = column sums of grad
        if (dw2)
            if (const int status = product('N', 'T', outputs, hidden, rows, grad, outputs, h, hidden, dw2, outputs))
                return status;
        if (db2 && outputs > 0) {
            const hipError_t summed =
                launch_column_sums(context->stream, Kernels<T>::dtype, false, const_cast<T *>(grad), nullptr, rows,
                                   outputs, parts, part_rows, partial, db2);
            if (summed != hipSuccess)
                return entry.refuse("backward bias", int(summed));
        }
        if (!first_layer)
            return 0;
        // dh[rows, hidden] = grad w2^T, zeroed where the ReLU was inactive, summed over rows for db1
        if (const int status = product('T', 'N', hidden, rows, outputs, w2, outputs, grad, outputs, dh, hidden))
            return status;
        if (hidden > 0) {
            const hipError_t masked =
                launch_column_sums(context->stream, Kernels<T>::dtype, true, dh, h, rows, hidden, parts, part_rows,
                                   db1 ? partial : nullptr, db1);
            if (masked != hipSuccess)
                return entry.refuse("backward activation", int(masked));
        }
        if (dw1) // dw1[inputs, hidden] = x^T dh
            if (const int status = product('N', 'T', hidden, inputs, rows, dh, hidden, x, inputs, dw1, hidden))
                return status;
        if (dx) // dx[rows, inputs] = dh w1^T
            return product('T', 'N', inputs, rows, hidden, w1, hidden, dh, hidden, dx, inputs);
        return 0;
    }
};

// The register-staged plan for a product whose output or addend the direct-to-LDS kernel cannot
// take (8-byte stores and loads): the tile of the same shape, or the nearest one, one launch.
void use_register_staged_tiles(Plan &plan)
{
    const TnVariant &tile = dma_variant(plan.kernel);
    plan.family = FAMILY_MFMA_TN;
    plan.kernel = tile.block_n >= 256 && tile.block_m >= 256 ? 0 : tile.block_n >= 256 ? 1 : 2;
    plan.tail_outputs = 0;
}

// Launches one planned BF16 product. `reserved`: FP32 room for a split K that the caller already
// holds inside the context's arena (null: reserve it here).
int launch_bf16_plan(const Entry &entry, Plan plan, const Product &p, float alpha, const void *a, const void *b,
                     float beta, void *c, BetaSource source, float *reserved)
{
    camblas_cuda_context *context = entry.context();
    hipStream_t stream = context->stream;
    const bool in_epilogue =
        plan.family == FAMILY_MFMA_TN || plan.family == FAMILY_STREAM || plan.family == FAMILY_DMA;
    if (source.z && !in_epilogue) {
        const hipError_t spread = launch_spread_bf16(stream, p.m, p.n, source.z, source.ldz, c, p.ldc);
        if (spread != hipSuccess)
            return entry.finish(spread, "BF16 GEMM addend");
        source = BetaSource{};
    }
    switch (plan.family) {
    case FAMILY_DMA: {
        context->counts[plan.counter]++;
        // (a plan may end with a second launch over the last outputs, which would have made a
        // partly filled last round of workgroups on the first tile)
        const int first = p.m - plan.tail_outputs;
        float *partials = reserved;
        if (plan.split_k > 1 && !partials) {
            // without room for the partials (allocation failure, capture in progress) run undivided
            if (reserve_scratch(context, size_t(plan.split_k) * size_t(p.m) * size_t(p.n) * 4) == hipSuccess) {
                partials = static_cast<float *>(context->scratch);
            } else {
                context->counts[5]++;
                plan.split_k = 1;
            }
        }
        hipError_t status = launch_bgemm_dma(stream, plan.kernel, first, p.n, p.k, alpha, a, p.lda, b, p.ldb, beta,
                                             c, p.ldc, source, plan.split_k, partials);
        if (status == hipSuccess && plan.tail_outputs) {
            const unsigned short *weights = static_cast<const unsigned short *>(a) + size_t(first) * p.lda;
            BetaSource rest = source;
            if (rest.z)
                rest.z = static_cast<const unsigned short *>(rest.z) + first;
            status = launch_bgemm_dma(stream, plan.tail_kernel, plan.tail_outputs, p.n, p.k, alpha, weights, p.lda,
                                      b, p.ldb, beta, static_cast<unsigned short *>(c) + first, p.ldc, rest);
        }
        return entry.finish(status, "BF16 MFMA GEMM (direct LDS loads)");
    }
    case FAMILY_STREAM: {
        StreamShares shares;
        if (plan.split_k > 1) {
            // K divided over several workgroups per tile needs FP32 planes and zeroed counters;
            // without them (allocation failure, capture in progress) the undivided choice runs
            const size_t bytes = stream_partial_bytes(plan.kernel / 10 % 10, plan.kernel % 10, p.m, p.n, plan.split_k);
            if (reserve_arrivals(context) == hipSuccess &&
                (reserved || reserve_scratch(context, bytes) == hipSuccess)) {
                float *planes = reserved ? reserved : static_cast<float *>(context->scratch);
                shares = StreamShares{plan.split_k, planes, context->arrivals};
            } else {
                context->counts[5]++;
                plan.kernel = undivided_stream_kernel(p.m, p.n, p.k, context->compute_units);
            }
        }
        context->counts[plan.counter]++;
        return entry.finish(launch_bgemv_stream(stream, plan.kernel / 100, plan.kernel / 10 % 10,
                                                plan.kernel % 10, p.m, p.n, p.k, alpha, a, p.lda, b, p.ldb,
                                                beta, c, p.ldc, source, shares),
                            "BF16 streaming GEMV");
    }
    case FAMILY_MFMA_TN: {
        float *partials = reserved;
        if (plan.split_k > 1 && !partials) {
            // without room for the partials (allocation failure, capture in progress) run unsplit
            if (reserve_scratch(context, size_t(plan.split_k) * size_t(p.m) * size_t(p.n) * 4) == hipSuccess) {
                partials = static_cast<float *>(context->scratch);
            } else {
                context->counts[5]++;
                plan.split_k = 1;
            }
        }
        context->counts[plan.counter]++;
        return entry.finish(launch_bgemm_tn(stream, plan.kernel, plan.split_k, p.m, p.n, p.k, alpha, a, p.lda, b,
                                            p.ldb, beta, c, p.ldc, partials, source),
                            "BF16 MFMA GEMM");
    }
    case FAMILY_NN: {
        float *partials = reserved;
        if (plan.split_k > 1 && !partials) {
            // without room for the partials (allocation failure, capture in progress) run undivided
            if (reserve_scratch(context, size_t(plan.split_k) * size_t(p.m) * size_t(p.n) * 4) == hipSuccess) {
                partials = static_cast<float *>(context->scratch);
            } else {
                context->counts[5]++;
                plan.split_k = 1;
            }
        }
        context->counts[plan.counter]++;
        return entry.finish(launch_bgemm_nn(stream, p.m, p.n, p.k, alpha, a, p.lda, b, p.ldb, beta, c, p.ldc,
                                            plan.split_k, partials),
                            "BF16 GEMM (outputs contiguous)");
    }
    case FAMILY_MFMA_BF16:
        context->counts[plan.counter]++;
        return entry.finish(launch_bgemm_any(stream, plan.kernel == 0, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha,
                                             a, p.lda, b, p.ldb, beta, c, p.ldc),
                            "BF16 MFMA GEMM (any layout)");
    default:
        context->counts[0]++;
        return entry.finish(launch_generic_bf16(stream, p.trans_a, p.trans_b, p.m, p.n, p.k, alpha, a, p.lda, b,
                                                p.ldb, beta, c, p.ldc),
                            "BF16 GEMM");
    }
}

// A large product whose operands are not both K-contiguous: the ones that are not are first copied
// transposed into the arena, after which the product is the linear-layer shape and runs on the
// direct-to-LDS tiles: measured 132 against 557 us at 4096^3 and 19 against 25 us at 512^3, the
// cost being one extra pass over each copied operand. Returns 1 when the arena could not hold the
// copies.
constexpr double TRANSPOSE_WORTHWHILE_FLOPS = 2.5e8; // about 512^3: below, the extra launches cost more
// tokens_only: only the second operand (the tokens of a linear layer: few rows) is copied, and the
// first stays as it lies, whichever way that is.
int bf16_product_transposing(const Entry &entry, const Product &p, float alpha, const void *a, const void *b,
                             float beta, void *c, const BetaSource &source, bool tokens_only = false)
{
    camblas_cuda_context *context = entry.context();
    hipStream_t stream = context->stream;
    const auto padded = [](size_t elements) { return (elements * 2 + 255) / 256 * 256; };
    const bool copy_a = !p.trans_a && !tokens_only;
    const size_t a_bytes = copy_a ? padded(size_t(p.m) * p.k) : 0;
    const size_t b_bytes = p.trans_b ? padded(size_t(p.n) * p.k) : 0;
    Product q = p;
    q.trans_a = copy_a ? 1 : p.trans_a, q.trans_b = 0;
    q.lda = copy_a ? p.k : p.lda;
    q.ldb = p.trans_b ? p.k : p.ldb;
    const bool aligned = (copy_a || is_aligned(a, 16)) && (p.trans_b || is_aligned(b, 16));
    Plan plan = make_plan(2, context->algorithm, q.trans_a, 0, q.m, q.n, q.k, q.lda, q.ldb, q.ldc, aligned,
                          context->compute_units);
    if (plan.family == FAMILY_DMA && (!is_aligned(c, 8) || !is_aligned(source.z, 8) || source.ldz % 4))
        use_register_staged_tiles(plan);
    if (plan.family == FAMILY_NN && !is_aligned(c, 8))
        plan = make_plan(2, context->algorithm, q.trans_a, 0, q.m, q.n, q.k, q.lda, q.ldb, q.ldc, false,
                         context->compute_units);
    size_t partial_bytes = 0; // room for a divided K, held in the same arena behind the copies
    if (plan.split_k > 1 && (plan.family == FAMILY_MFMA_TN || plan.family == FAMILY_DMA || plan.family == FAMILY_NN))
        partial_bytes = size_t(plan.split_k) * size_t(p.m) * size_t(p.n) * 4;
    else if (plan.split_k > 1 && plan.family == FAMILY_STREAM)
        partial_bytes = stream_partial_bytes(plan.kernel / 10 % 10, plan.kernel % 10, p.m, p.n, plan.split_k);
    if (reserve_scratch(context, a_bytes + b_bytes + partial_bytes) != hipSuccess)
        return 1;
    char *arena = static_cast<char *>(context->scratch);
    if (copy_a) { // a[i + l*lda] -> [i*k + l]
        const hipError_t status = launch_transpose_bf16(stream, p.k, p.m, a, p.lda, arena, p.k);
        if (status != hipSuccess)
            return entry.finish(status, "BF16 operand transposition");
        a = arena;
    }
    if (p.trans_b) { // b[j + l*ldb] -> [j*k + l]
        const hipError_t status = launch_transpose_bf16(stream, p.k, p.n, b, p.ldb, arena + a_bytes, p.k);
        if (status != hipSuccess)
            return entry.finish(status, "BF16 operand transposition");
        b = arena + a_bytes;
    }
    float *reserved = partial_bytes ? reinterpret_cast<float *>(arena + a_bytes + b_bytes) : nullptr;
    return launch_bf16_plan(entry, plan, q, alpha, a, b, beta, c, source, reserved);
}

// BF16 'T','N' and the other layouts: the planner's kernel, or the one a test forced.
// `source`: where the beta term is read from when that is not C itself (see BetaSource). The
// K-contiguous families read it in their epilogues; for the others it is first spread over C.
int bf16_product(const Entry &entry, const Product &p, float alpha, const void *a, const void *b, float beta,
                 void *c, BetaSource source = {})
{
    camblas_cuda_context *context = entry.context();
    Plan plan = make_plan(2, context->algorithm, p.trans_a, p.trans_b, p.m, p.n, p.k, p.lda, p.ldb, p.ldc,
                          is_aligned(a, 16) && is_aligned(b, 16), context->compute_units);
    const int forced = context->override_kernel;
    // W as it lies (the planner's variant 20 for 'N','N'): the other kernels of that family assume
    // K-contiguous weights, so neither the register-staged substitute nor a forced variant applies;
    // tests: 60 and 61 ask for the layout-agnostic kernel or the transposing route instead
    bool as_it_lies = plan.family == FAMILY_DMA && plan.kernel == 20 && !p.trans_a;
    // tests: 40 forces that tile for an 'N','N' call of any size whose operands it can take (a launch that
    // cannot run fails), and is refused for every other layout
    if (forced == 40) {
        if (p.trans_a || p.trans_b)
            return entry.refuse("the forced tile takes 'N','N' operands only");
        plan.family = FAMILY_DMA;
        plan.kernel = 20;
        plan.split_k = 1;
        plan.tail_outputs = 0;
        plan.counter = 4;
        as_it_lies = true;
    }
    if (as_it_lies) {
        if (!is_aligned(c, 8) || !is_aligned(source.z, 8) || source.ldz % 4 || forced == 60 || forced == 61)
            plan = make_plan(2, context->algorithm, p.trans_a, p.trans_b, p.m, p.n, p.k, p.lda, p.ldb, p.ldc, false,
                             context->compute_units);
        else
            return launch_bf16_plan(entry, plan, p, alpha, a, b, beta, c, source, nullptr);
    }
    if (plan.family == FAMILY_DMA && (!is_aligned(c, 8) || !is_aligned(source.z, 8) || source.ldz % 4))
        use_register_staged_tiles(plan); // register-staged loads, scalar stores
    // Tokens stored the other way round (K rows of tokens) and few of them: copying them transposed
    // costs next to nothing, and the product then runs on the kernels for few tokens instead of the
    // layout-agnostic tiles or, below 32 tokens, the vector-ALU kernel ([8192, 28672] x 16 tokens:
    // 1760 us).
    if (p.trans_b && p.n <= 512 && forced < 0 && context->algorithm != CAMBLAS_CUDA_CLASSICAL &&
        2.0 * p.m * p.n * p.k >= 1e6) {
        const int status = bf16_product_transposing(entry, p, alpha, a, b, beta, c, source, true);
        if (status <= 0)
            return status;
        context->counts[5]++; // no room for the copy
    }
    // the outputs-contiguous kernel stores eight bytes at a time; tests: 60 and 61 ask for the
    // layout-agnostic kernel or the transposing route instead, 62 sets the workgroups K is divided over
    if (plan.family == FAMILY_NN && (!is_aligned(c, 8) || forced == 60 || forced == 61))
        plan = make_plan(2, context->algorithm, p.trans_a, p.trans_b, p.m, p.n, p.k, p.lda, p.ldb, p.ldc, false,
                         context->compute_units);
    if (plan.family == FAMILY_NN && forced == 62)
        plan.split_k = std::max(1, context->override_split);
    if (plan.family == FAMILY_MFMA_BF16) {
        // tests: 60 keeps the layout-agnostic kernel, 61 takes the transposing route whatever the size
        const bool worthwhile = 2.0 * p.m * p.n * p.k >= TRANSPOSE_WORTHWHILE_FLOPS;
        if (forced == 61 || (forced != 60 && worthwhile)) {
            const int status = bf16_product_transposing(entry, p, alpha, a, b, beta, c, source);
            if (status <= 0)
                return status;
            context->counts[5]++; // no room for the copies: the layout-agnostic kernel after all
        }
        return launch_bf16_plan(entry, plan, p, alpha, a, b, beta, c, source, nullptr);
    }
    const bool matrix_family =
        plan.family == FAMILY_MFMA_TN || plan.family == FAMILY_STREAM || plan.family == FAMILY_DMA;
    if (matrix_family && forced >= 0) {
        // tests: 0.. a register-staged tile variant (with override_split), 20..59 a direct-to-LDS
        // variant, 100 + 100*depth + 10*row_tiles + token_tiles the streaming kernel
        plan.split_k = 1;
        plan.tail_outputs = 0;
        if (forced >= 100) {
            plan.family = FAMILY_STREAM;
            plan.kernel = forced - 100;
            plan.split_k = std::max(1, context->override_split);
        } else if (forced >= 20 && forced < 60) {
            plan.family = FAMILY_DMA;
            plan.kernel = forced - 20;
            plan.split_k = std::max(1, context->override_split);
        } else {
            plan.family = FAMILY_MFMA_TN;
            plan.kernel = forced;
            plan.split_k = std::max(1, context->override_split);
        }
    }
    return launch_bf16_plan(entry, plan, p, alpha, a, b, beta, c, source, nullptr);
}

// A decode linear (at most 64 tokens, weights [outputs, inner] with K contiguous) with one or both
// halves of a residual-add + RMSNorm fused into it: always the weight-streaming kernel, planned like an
// ordinary linear of that shape. workgroups (may be null): receives the number of workgroups along
// the outputs, which is the number of partial sums of squares per token a residual epilogue writes.
int fused_stream_linear(const Entry &entry, int tokens, int outputs, int inner, const void *x, int ldx,
                        const void *w, int ldw, void *y, int ldy, StreamFusion fusion, int capacity, int *workgroups)
{
    camblas_cuda_context *context = entry.context();
    Plan plan = make_plan(2, CAMBLAS_CUDA_AUTO, true, false, outputs, tokens, inner, ldw, ldx, ldy, true,
                          context->compute_units);
    if (plan.family != FAMILY_STREAM || plan.kernel / 100 > 1) {
        // (33 to 64 tokens on a narrow projection plan other kernels: the undivided streaming kernel then)
        plan.family = FAMILY_STREAM;
        plan.kernel = undivided_stream_kernel(outputs, tokens, inner, context->compute_units);
        plan.split_k = 1;
        if (plan.kernel / 100 > 1)
            plan.kernel %= 100;
    }
    StreamShares shares;
    if (plan.split_k > 1) {
        const size_t bytes = stream_partial_bytes(plan.kernel / 10 % 10, plan.kernel % 10, outputs, tokens, plan.split_k);
        if (reserve_arrivals(context) == hipSuccess && reserve_scratch(context, bytes) == hipSuccess) {
            shares = StreamShares{plan.split_k, static_cast<float *>(context->scratch), context->arrivals};
        } else {
            context->counts[5]++;
            plan.kernel = undivided_stream_kernel(outputs, tokens, inner, context->compute_units) % 100;
        }
    }
    if (plan.kernel % 10 == 3) // (the fused forms exist with 1, 2 and 4 token tiles)
        plan.kernel += 1;
    const int row_tiles = plan.kernel / 10 % 10;
    const int count = stream_workgroups_along_outputs(row_tiles, outputs);
    if (workgroups)
        *workgroups = count;
    if (fusion.residual && count > capacity)
        return entry.refuse("room for the partial sums of squares");
    context->counts[plan.counter]++;
    return entry.finish(launch_bgemv_stream(context->stream, plan.kernel / 100, row_tiles, plan.kernel % 10, outputs,
                                            tokens, inner, 1.f, w, ldw, x, ldx, 0.f, y, ldy, BetaSource{}, shares,
                                            fusion),
                        "BF16 streaming linear with fused normalisation");
}

template <typename T>
int typed_gemm(camblas_cuda_context *context, char ta, char tb, int m, int n, int k, T alpha, const T *a,
               int lda, const T *b, int ldb, T beta, T *c, int ldc)
{
    Entry entry(context);
    return entry.run(
        [&] { return dense_product(entry, Product(ta, tb, m, n, k, lda, ldb, ldc), alpha, a, b, beta, c); });
}
} // namespace
} // namespace camblas_hip

using namespace camblas_hip;

extern "C" int camblas_cuda_sgemm(camblas_cuda_context *context, char ta, char tb, int m, int n,
                                  int k, float alpha, const float *a, int lda, const float *b,
                                  int ldb, float beta, float *c, int ldc)
{
    return typed_gemm(context, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

extern "C" int camblas_cuda_dgemm(camblas_cuda_context *context, char ta, char tb, int m, int n,
                                  int k, double alpha, const double *a, int lda, const double *b,
                                  int ldb, double beta, double *c, int ldc)
{
    return typed_gemm(context, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

extern "C" int camblas_cuda_bgemm(camblas_cuda_context *context, char trans_a, char trans_b, int m,
                                  int n, int k, float alpha, const void *a, int lda, const void *b,
                                  int ldb, float beta, void *c, int ldc)
{
    static const char *const names[4] = {"invalid BF16 GEMM arguments",
                                         "invalid BF16 pointer or leading dimension", "scale BF16 output",
                                         "missing or aliased BF16 GEMM operand"};
    Entry entry(context);
    return entry.run([&] {
        const Product p(trans_a, trans_b, m, n, k, lda, ldb, ldc);
        const int admitted = admit_product(entry, p, alpha, beta, a, b, c, names, [&] {
            return launch_scale_bf16(context->stream, m, n, beta, c, ldc);
        });
        return admitted <= 0 ? admitted : bf16_product(entry, p, alpha, a, b, beta, c);
    });
}

// C = alpha op(A) op(B) + beta Z with the addend Z apart from C: an m x n matrix with leading
// dimension ldz >= m, or one column of m values repeated n times (ldz == 0), which is the bias row
// of a linear layer seen column-major. What aten::addmm needs without first spreading the bias
// over the output (the reference spreads it: src/cuda/torch_backend.cuh:60-88).
extern "C" int camblas_cuda_bgemm_add(camblas_cuda_context *context, char trans_a, char trans_b, int m,
                                      int n, int k, float alpha, const void *a, int lda, const void *b,
                                      int ldb, float beta, const void *z, int ldz, void *c, int ldc)
{
    if (beta == 0.f) // Z is never read
        return camblas_cuda_bgemm(context, trans_a, trans_b, m, n, k, alpha, a, lda, b, ldb, 0.f, c, ldc);
    static const char *const names[4] = {"invalid BF16 GEMM arguments",
                                         "invalid BF16 pointer or leading dimension", "scale BF16 output",
                                         "missing or aliased BF16 GEMM operand"};
    Entry entry(context);
    return entry.run([&] {
        const Product p(trans_a, trans_b, m, n, k, lda, ldb, ldc);
        if (!p.well_formed() || ldz < 0)
            return entry.refuse(names[0]);
        if (p.empty())
            return 0;
        if (!c || !z || !p.strides_cover() || (ldz != 0 && ldz < m))
            return entry.refuse(names[1]);
        // the two stored extents may not overlap: C is written while Z is still being read
        const char *z_first = static_cast<const char *>(z), *c_first = static_cast<const char *>(c);
        const size_t z_bytes = (size_t(ldz) * size_t(n - 1) + size_t(m)) * 2;
        const size_t c_bytes = (size_t(ldc) * size_t(n - 1) + size_t(m)) * 2;
        if (z_first < c_first + c_bytes && c_first < z_first + z_bytes)
            return entry.refuse(names[3]);
        if (alpha == 0.f || k == 0) { // only beta acts
            const hipError_t spread = launch_spread_bf16(context->stream, m, n, z, ldz, c, ldc);
            if (spread != hipSuccess)
                return entry.finish(spread, "BF16 GEMM addend");
            return beta == 1.f ? 0 : entry.finish(launch_scale_bf16(context->stream, m, n, beta, c, ldc), names[2]);
        }
        if (!a || !b || a == c || b == c)
            return entry.refuse(names[3]);
        return bf16_product(entry, p, alpha, a, b, beta, c, BetaSource{z, ldz});
    });
}

extern "C" int camblas_cuda_affine(camblas_cuda_context *context, int dtype, int rows, int inner,
                                   int columns, const void *x, const void *weight, const void *bias,
                                   int relu, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        switch (dtype) {
        case 0:
            return affine_layer(entry, rows, inner, columns, static_cast<const float *>(x),
                                static_cast<const float *>(weight), static_cast<const float *>(bias), relu != 0,
                                static_cast<float *>(output));
        case 1:
            return affine_layer(entry, rows, inner, columns, static_cast<const double *>(x),
                                static_cast<const double *>(weight), static_cast<const double *>(bias), relu != 0,
                                static_cast<double *>(output));
        default:
            return entry.refuse("unsupported affine dtype");
        }
    });
}

// two affine layers, the first with ReLU; the hidden activations are an output of their own and
// may not share storage with the result (ref: backend.cu:1103-1117)
extern "C" int camblas_cuda_mlp(camblas_cuda_context *context, int dtype, int rows, int inputs,
                                int hidden, int outputs, const void *x, const void *w1,
                                const void *b1, const void *w2, const void *b2, void *hidden_output,
                                void *output)
{
    const bool shares_storage = rows > 0 && hidden > 0 && hidden_output == output;
    if (rows < 0 || inputs < 0 || hidden < 0 || outputs < 0 || shares_storage)
        return fail(context, "invalid MLP dimensions or aliased outputs", 1);
    if (const int status = camblas_cuda_affine(context, dtype, rows, inputs, hidden, x, w1, b1, 1, hidden_output))
        return status;
    return camblas_cuda_affine(context, dtype, rows, hidden, outputs, hidden_output, w2, b2, 0, output);
}

extern "C" int camblas_cuda_attention(camblas_cuda_context *context, int dtype, int queries, int keys,
                                      int depth, int values, double scale, const void *q,
                                      const void *k, const void *v, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        switch (dtype) {
        case 0:
            return score_attention(entry, queries, keys, depth, values, float(scale),
                                   static_cast<const float *>(q), static_cast<const float *>(k),
                                   static_cast<const float *>(v), static_cast<float *>(output));
        case 1:
            return score_attention(entry, queries, keys, depth, values, scale, static_cast<const double *>(q),
                                   static_cast<const double *>(k), static_cast<const double *>(v),
                                   static_cast<double *>(output));
        default:
            return entry.refuse("unsupported attention dtype");
        }
    });
}

extern "C" int camblas_cuda_mlp_backward(camblas_cuda_context *context, int dtype, int rows,
                                         int inputs, int hidden, int outputs, const void *x,
                                         const void *w1, const void *w2, const void *hidden_output,
                                         const void *grad_output, void *grad_hidden, void *dx,
                                         void *dw1, void *db1, void *dw2, void *db2)
{
    Entry entry(context);
    return entry.run([&] {
        switch (dtype) {
        case 0: {
            using T = float;
            return BackwardPass<T>{entry, rows, inputs, hidden, outputs, static_cast<const T *>(x),
                                   static_cast<const T *>(w1), static_cast<const T *>(w2),
                                   static_cast<const T *>(hidden_output), static_cast<const T *>(grad_output),
                                   static_cast<T *>(grad_hidden), static_cast<T *>(dx), static_cast<T *>(dw1),
                                   static_cast<T *>(db1), static_cast<T *>(dw2), static_cast<T *>(db2)}
                .run();
        }
        case 1: {
            using T = double;
            return BackwardPass<T>{entry, rows, inputs, hidden, outputs, static_cast<const T *>(x),
                                   static_cast<const T *>(w1), static_cast<const T *>(w2),
                                   static_cast<const T *>(hidden_output), static_cast<const T *>(grad_output),
                                   static_cast<T *>(grad_hidden), static_cast<T *>(dx), static_cast<T *>(dw1),
                                   static_cast<T *>(db1), static_cast<T *>(dw2), static_cast<T *>(db2)}
                .run();
        }
        default:
            return entry.refuse("unsupported backward dtype");
        }
    });
}

// ---- the residual-add + RMSNorm around the decode linears, fused into them (extensions; the norm's
// arithmetic is the reference's, src/cuda/inference_fusion.cuh:136-191, binding
// src/cuda/torch_bindings.cpp:675-701)

extern "C" int camblas_cuda_bf16_linear_residual(camblas_cuda_context *context, int tokens, int outputs, int inner,
                                                 const void *x, int ldx, const void *w, int ldw,
                                                 const void *residual, int ld_residual, void *added, int ld_added,
                                                 float *squares, int squares_ld, int squares_capacity,
                                                 int *squares_count)
{
    Entry entry(context);
    return entry.run([&] {
        if (squares_count)
            *squares_count = 0;
        if (!within({{tokens, 0, 64, 1}, {outputs, 0, INT32_MAX, 1}, {inner, 8, (1 << 23) - 8, 8},
                     {ldx, inner, (1 << 23) - 8, 8}, {ldw, inner, (1 << 23) - 8, 8},
                     {ld_residual, outputs, INT32_MAX, 1}, {ld_added, outputs, INT32_MAX, 1},
                     {squares_ld, tokens, INT32_MAX, 1}, {squares_capacity, 0, INT32_MAX, 1}}))
            return entry.refuse("invalid fused linear dimensions");
        if (tokens == 0 || outputs == 0)
            return 0;
        if (!usable({{x, 16}, {w, 16}, {residual, 2}, {added, 2}, {squares, 4}}) || !squares_count ||
            !apart(added, {x, w}) || !apart(squares, {x, w, residual, added}))
            return entry.refuse("invalid fused linear buffers");
        StreamFusion fusion;
        fusion.residual = residual;
        fusion.ld_residual = ld_residual;
        fusion.ssq_out = squares;
        fusion.ssq_ld_out = squares_ld;
        return fused_stream_linear(entry, tokens, outputs, inner, x, ldx, w, ldw, added, ld_added, fusion,
                                   squares_capacity, squares_count);
    });
}

extern "C" int camblas_cuda_bf16_rms_linear(camblas_cuda_context *context, int tokens, int outputs, int inner,
                                            const void *x, int ldx, const float *squares, int squares_ld,
                                            int squares_count, const void *norm_weight, float epsilon,
                                            const void *w, int ldw, void *y, int ldy)
{
    Entry entry(context);
    return entry.run([&] {
        if (!within({{tokens, 0, 64, 1}, {outputs, 0, INT32_MAX, 1}, {inner, 8, (1 << 23) - 8, 8},
                     {ldx, inner, (1 << 23) - 8, 8}, {ldw, inner, (1 << 23) - 8, 8}, {ldy, outputs, INT32_MAX, 1},
                     {squares_ld, tokens, INT32_MAX, 1}, {squares_count, 1, INT32_MAX, 1}}) ||
            !(epsilon >= 0.f) || !std::isfinite(epsilon))
            return entry.refuse("invalid fused linear dimensions");
        if (tokens == 0 || outputs == 0)
            return 0;
        if (!usable({{x, 16}, {w, 16}, {norm_weight, 16}, {squares, 4}, {y, 2}}) || !apart(y, {x, w, norm_weight, squares}))
            return entry.refuse("invalid fused linear buffers");
        StreamFusion fusion;
        fusion.norm_weight = norm_weight;
        fusion.ssq_in = squares;
        fusion.ssq_count = squares_count;
        fusion.ssq_ld = squares_ld;
        fusion.epsilon = epsilon;
        return fused_stream_linear(entry, tokens, outputs, inner, x, ldx, w, ldw, y, ldy, fusion, 0, nullptr);
    });
}

