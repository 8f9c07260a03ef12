// Elementwise and row-wise entry points of the C ABI (SiLU-multiply, SwiGLU, the RMS normalisation
// family) and the decode-layer pieces the reference has no counterpart for (rotary embedding,
// cache append, grouped-query decode attention). What each call rejects follows the reference's
// wrappers, read as text: src/cuda/backend.cu:1119-1163 (activations), :1363-1475 (normalisation).
#include "entry.hpp"

#include <cmath>
#include <cstdint>

namespace camblas_hip
{
namespace
{
bool valid_epsilon(float epsilon) { return std::isfinite(epsilon) && epsilon >= 0; }

// the single-row kernels of the reference accept widths 2048 .. 65536 in multiples of four
bool decode_width(int width) { return within({{width, 2048, 65536, 4}}); }

// count elements of `dtype` fit in a size_t
bool countable(uint64_t count, int dtype) { return count <= SIZE_MAX / storage_bytes(dtype); }
} // namespace
} // namespace camblas_hip

using namespace camblas_hip;

extern "C" int camblas_cuda_silu_multiply(camblas_cuda_context *context, int dtype, uint64_t count,
                                          const void *gate, const void *up, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (!storage_in(dtype, {0, 2}))
            return entry.refuse("unsupported SiLU dtype");
        if (count == 0)
            return 0;
        if (!usable({{gate, 1}, {up, 1}, {output, 1}}) || !countable(count, dtype))
            return entry.refuse("invalid SiLU operands or length");
        return entry.finish(launch_silu_multiply(entry.stream(), dtype, count, gate, up, output), "SiLU multiply");
    });
}

extern "C" int camblas_cuda_swiglu(camblas_cuda_context *context, int dtype, uint64_t count,
                                   int width, float limit, const void *gate, const void *up,
                                   const float *routing, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = storage_in(dtype, {0, 2}) && width > 0 && count % unsigned(width) == 0 &&
                            std::isfinite(limit) && limit >= 0 && countable(count, dtype);
        if (!shaped)
            return entry.refuse("invalid SwiGLU dimensions or clipping limit");
        if (count == 0)
            return 0;
        const size_t element = storage_bytes(dtype);
        if (!usable({{gate, element}, {up, element}, {output, element}, {routing, 4, true}}) ||
            !apart(output, {routing}))
            return entry.refuse("invalid SwiGLU buffers");
        return entry.finish(launch_swiglu(entry.stream(), dtype, count, width, limit, gate, up, routing, output),
                            "SwiGLU");
    });
}

extern "C" int camblas_cuda_rms_norm_decode(camblas_cuda_context *context, int dtype,
                                            int weight_dtype, int width, float epsilon,
                                            int round_before_weight, int descending,
                                            const void *input, const void *weight, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        // FP32 rows take FP32 weights; BF16 rows take either
        const bool typed = storage_in(dtype, {0, 2}) && storage_in(weight_dtype, {0, 2}) &&
                           !(dtype == 0 && weight_dtype != 0);
        const bool ok = typed && decode_width(width) && is_flag(round_before_weight) && is_flag(descending) &&
                        valid_epsilon(epsilon) &&
                        usable({{input, storage_bytes(dtype)},
                                {weight, storage_bytes(weight_dtype)},
                                {output, storage_bytes(dtype)}}) &&
                        apart(output, {input, weight});
        if (!ok)
            return entry.refuse("invalid decode RMS arguments");
        return entry.finish(launch_rms_rows(entry.stream(), dtype, weight_dtype, 1, width, epsilon,
                                            round_before_weight != 0, input, nullptr, weight, nullptr, output),
                            "decode RMS normalisation");
    });
}

extern "C" int camblas_cuda_add_rms_norm(camblas_cuda_context *context, int dtype, int width,
                                         float epsilon, const void *input, const void *residual,
                                         const void *weight, void *added, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        const bool ok = storage_in(dtype, {0, 2}) && decode_width(width) && valid_epsilon(epsilon) &&
                        usable({{input, 1}, {residual, 1}, {weight, 1}, {added, 1}, {output, 1}}) &&
                        apart(added, {output, input, residual, weight}) &&
                        apart(output, {input, residual, weight});
        if (!ok)
            return entry.refuse("invalid residual RMS arguments");
        return entry.finish(launch_rms_rows(entry.stream(), dtype, dtype, 1, width, epsilon, true, input, residual,
                                            weight, added, output),
                            "residual RMS normalisation");
    });
}

// Any number of rows, with or without a residual (no counterpart in the reference header).
extern "C" int camblas_cuda_add_rms_norm_rows(camblas_cuda_context *context, int dtype,
                                              int weight_dtype, int rows, int width, float epsilon,
                                              int round_before_weight, const void *input,
                                              const void *residual, const void *weight, void *added,
                                              void *output)
{
    Entry entry(context);
    return entry.run([&] {
        const bool typed = storage_in(dtype, {0, 2}) && storage_in(weight_dtype, {0, 2}) &&
                           !(dtype == 0 && weight_dtype != 0);
        if (!typed || rows < 0 || width < 0 || !is_flag(round_before_weight) || !valid_epsilon(epsilon))
            return entry.refuse("invalid residual RMS rows arguments");
        if (rows == 0 || width == 0)
            return 0;
        bool ok = usable({{input, 1}, {weight, 1}, {output, 1}}) && apart(output, {weight, input});
        if (ok && residual)
            ok = added && apart(added, {output, input, residual, weight}) && apart(output, {residual});
        if (!ok)
            return entry.refuse("invalid residual RMS rows operands");
        return entry.finish(launch_rms_rows(entry.stream(), dtype, weight_dtype, rows, width, epsilon,
                                            round_before_weight != 0, input, residual, weight, added, output),
                            "residual RMS normalisation");
    });
}

// In-place (output == input) is allowed as in the reference (backend.cu:1423-1439): a thread reads
// an element before it writes it.
extern "C" int camblas_cuda_rms_norm(camblas_cuda_context *context, int dtype, int rows, int width,
                                     float epsilon, const void *input, const void *weight,
                                     void *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (!storage_in(dtype, {0, 2}) || rows < 0 || width < 0 || !valid_epsilon(epsilon))
            return entry.refuse("invalid RMS normalisation dimensions, dtype or epsilon");
        if (rows == 0 || width == 0)
            return 0;
        if (!usable({{input, 1}, {weight, 1}, {output, 1}}) || !apart(output, {weight}))
            return entry.refuse("invalid RMS normalisation operands");
        return entry.finish(launch_rms_rows(entry.stream(), dtype, dtype, rows, width, epsilon, true, input,
                                            nullptr, weight, nullptr, output),
                            "RMS normalisation");
    });
}

extern "C" int camblas_cuda_bfloat16_square(camblas_cuda_context *context, uint64_t count,
                                            const void *input, float *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (count == 0)
            return 0;
        if (!usable({{input, 1}, {output, 1}}) || !countable(count, 0))
            return entry.refuse("invalid BF16 square operands");
        return entry.finish(launch_bf16_square(entry.stream(), count, input, output), "BF16 squares");
    });
}

extern "C" int camblas_cuda_rms_scale(camblas_cuda_context *context, int dtype, uint64_t count,
                                      int width, float epsilon, const void *input,
                                      const void *weight, const float *means, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (!storage_in(dtype, {0, 2}) || width < 0 || !valid_epsilon(epsilon))
            return entry.refuse("invalid RMS scale dimensions, dtype or epsilon");
        if (count == 0)
            return 0;
        const bool ok = width > 0 && count % unsigned(width) == 0 && countable(count, 0) &&
                        usable({{input, 1}, {weight, 1}, {means, 1}, {output, 1}}) && apart(output, {weight});
        if (!ok)
            return entry.refuse("invalid RMS scale operands");
        return entry.finish(launch_rms_scale(entry.stream(), dtype, count, width, epsilon, input, weight, means,
                                             output),
                            "RMS scaling");
    });
}

// The front end of a gated MLP for a decode batch, out = silu_multiply(x gate^T, x up^T), as one
// streaming pass over both weight matrices. The reference composes it from two linears and
// camblas_cuda_silu_multiply in its binding (src/cuda/torch_bindings.cpp:703-723); the rounding
// points here are the same (both products and the activation are rounded to BF16).
extern "C" int camblas_cuda_bf16_gated_linear(camblas_cuda_context *context, int rows, int outputs, int inner,
                                              const void *x, int ldx, const void *gate, const void *up,
                                              int ldw, void *out, int ldo)
{
    Entry entry(context);
    return entry.run([&] {
        if (!within({{rows, 0, 64, 1}, {outputs, 0, INT32_MAX, 1}, {inner, 8, (1 << 23) - 8, 8}, {ldx, inner, (1 << 23) - 8, 8},
                     {ldw, inner, (1 << 23) - 8, 8}, {ldo, outputs, INT32_MAX, 1}}))
            return entry.refuse("invalid gated linear dimensions");
        if (rows == 0 || outputs == 0)
            return 0;
        if (!usable({{x, 16}, {gate, 16}, {up, 16}, {out, 2}}) || !apart(out, {x, gate, up}))
            return entry.refuse("invalid gated linear buffers");
        const int token_tiles = rows <= 16 ? 1 : rows <= 32 ? 2 : rows <= 48 ? 3 : 4;
        // the widest workgroups that still leave one and a half per compute unit (or a test's choice)
        int pair_tiles = 4;
        while (pair_tiles > 1 && (outputs + 16 * pair_tiles - 1) / (16 * pair_tiles) * 2 < 3 * context->compute_units)
            --pair_tiles;
        if (context->override_kernel >= 1 && context->override_kernel <= 4)
            pair_tiles = context->override_kernel;
        context->counts[4]++;
        return entry.finish(launch_gated_stream(context->stream, pair_tiles, token_tiles, outputs, rows, inner,
                                                gate, up, ldw, x, ldx, out, ldo),
                            "BF16 gated streaming linear");
    });
}

// The same with the RMSNorm in front of it fused in: x holds the un-normalised rows, `squares`
// [squares_count][squares_ld] partial sums of squares of each row (added in index order), and the
// tokens are normalised while they are staged (round(round(x * scale) * norm_weight), the reference's
// rounding points, src/cuda/inference_fusion.cuh:186-189).
extern "C" int camblas_cuda_bf16_rms_gated_linear(camblas_cuda_context *context, int rows, int outputs, int inner,
                                                  const void *x, int ldx, const float *squares, int squares_ld,
                                                  int squares_count, const void *norm_weight, float epsilon,
                                                  const void *gate, const void *up, int ldw, void *out, int ldo)
{
    Entry entry(context);
    return entry.run([&] {
        if (!within({{rows, 0, 64, 1}, {outputs, 0, INT32_MAX, 1}, {inner, 8, (1 << 23) - 8, 8}, {ldx, inner, (1 << 23) - 8, 8},
                     {ldw, inner, (1 << 23) - 8, 8}, {ldo, outputs, INT32_MAX, 1}, {squares_ld, rows, INT32_MAX, 1},
                     {squares_count, 1, INT32_MAX, 1}}) ||
            !valid_epsilon(epsilon))
            return entry.refuse("invalid gated linear dimensions");
        if (rows == 0 || outputs == 0)
            return 0;
        if (!usable({{x, 16}, {gate, 16}, {up, 16}, {norm_weight, 16}, {squares, 4}, {out, 2}}) ||
            !apart(out, {x, gate, up, norm_weight, squares}))
            return entry.refuse("invalid gated linear buffers");
        const int token_tiles = rows <= 16 ? 1 : rows <= 32 ? 2 : 4;
        int pair_tiles = 4;
        while (pair_tiles > 1 && (outputs + 16 * pair_tiles - 1) / (16 * pair_tiles) * 2 < 3 * context->compute_units)
            --pair_tiles;
        if (context->override_kernel >= 1 && context->override_kernel <= 4)
            pair_tiles = context->override_kernel;
        context->counts[4]++;
        StreamFusion fusion;
        fusion.norm_weight = norm_weight;
        fusion.ssq_in = squares;
        fusion.ssq_count = squares_count;
        fusion.ssq_ld = squares_ld;
        fusion.epsilon = epsilon;
        return entry.finish(launch_gated_stream(context->stream, pair_tiles, token_tiles, outputs, rows, inner,
                                                gate, up, ldw, x, ldx, out, ldo, fusion),
                            "BF16 gated streaming linear with fused normalisation");
    });
}

// added = round(x + residual) per element and squares[row] = the sum of added^2 over the row: the
// state the fused linears pass along, made from scratch (a model's first layer).
extern "C" int camblas_cuda_add_residual_squares(camblas_cuda_context *context, int rows, int width,
                                                 const void *x, const void *residual, void *added, float *squares)
{
    Entry entry(context);
    return entry.run([&] {
        if (rows < 0 || !within({{width, 0, INT32_MAX, 1}}))
            return entry.refuse("invalid residual squares arguments");
        if (rows == 0)
            return 0;
        if (!usable({{x, 2}, {residual, 2}, {added, 2}, {squares, 4}}) || !apart(squares, {x, residual, added}))
            return entry.refuse("invalid residual squares buffers");
        return entry.finish(launch_add_residual_squares(entry.stream(), rows, width, x, residual, added, squares),
                            "residual add with sums of squares");
    });
}

// ---- decode-layer pieces (no counterpart in the reference)

extern "C" int camblas_cuda_rope(camblas_cuda_context *context, int tokens, int heads, int dim,
                                 int token_stride, float theta, const int32_t *positions, void *x)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = tokens >= 0 && heads >= 1 && within({{dim, 2, INT32_MAX, 2}}) &&
                            token_stride >= int64_t(heads) * dim && std::isfinite(theta) && theta > 0;
        if (!shaped)
            return entry.refuse("invalid rotary embedding arguments");
        if (tokens == 0)
            return 0;
        if (!usable({{positions, 4}, {x, 2}}))
            return entry.refuse("invalid rotary embedding buffers");
        return entry.finish(launch_rope(entry.stream(), tokens, heads, dim, token_stride, theta, positions, x),
                            "rotary embedding");
    });
}

extern "C" int camblas_cuda_kv_append(camblas_cuda_context *context, int batch, int kv_heads, int dim,
                                      int context_length, const int32_t *positions,
                                      const void *k_new, const void *v_new, int token_stride,
                                      void *k_cache, void *v_cache)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = batch >= 0 && kv_heads >= 1 && within({{dim, 8, INT32_MAX, 8}}) &&
                            context_length >= 1 && token_stride >= int64_t(kv_heads) * dim &&
                            token_stride % 8 == 0;
        if (!shaped)
            return entry.refuse("invalid cache append arguments");
        if (batch == 0)
            return 0;
        if (!usable({{positions, 1}, {k_new, 16}, {v_new, 16}, {k_cache, 16}, {v_cache, 16}}) ||
            k_cache == v_cache)
            return entry.refuse("invalid cache append buffers");
        return entry.finish(launch_kv_append(entry.stream(), batch, kv_heads, dim, context_length, positions, k_new,
                                             v_new, token_stride, k_cache, v_cache),
                            "cache append");
    });
}

extern "C" int camblas_cuda_rope_kv_append(camblas_cuda_context *context, int batch, int q_heads,
                                           int kv_heads, int dim, int token_stride, float theta,
                                           const int32_t *positions, void *qkv, int context_length,
                                           void *k_cache, void *v_cache)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = batch >= 0 && q_heads >= 1 && kv_heads >= 1 && within({{dim, 2, INT32_MAX, 2}}) &&
                            context_length >= 1 &&
                            token_stride >= (int64_t(q_heads) + 2 * int64_t(kv_heads)) * dim &&
                            std::isfinite(theta) && theta > 0;
        if (!shaped)
            return entry.refuse("invalid rotary cache append arguments");
        if (batch == 0)
            return 0;
        if (!usable({{positions, 4}, {qkv, 2}, {k_cache, 2}, {v_cache, 2}}) || k_cache == v_cache)
            return entry.refuse("invalid rotary cache append buffers");
        return entry.finish(launch_rope_kv_append(entry.stream(), batch, q_heads, kv_heads, dim, token_stride, theta,
                                                  positions, qkv, context_length, k_cache, v_cache),
                            "rotary cache append");
    });
}

namespace camblas_hip
{
namespace
{
// Both decode-attention entry points: the argument rules, then the two launches with the split
// partials wherever `place(bytes, &where)` puts them (it returns a status of its own on failure).
template <typename Place>
int decode_attention(const Entry &entry, int batch, int q_heads, int kv_heads, int dim, int context_length,
                     const int32_t *lengths, float scale, const void *q, int q_stride, const void *k_cache,
                     const void *v_cache, void *output, Place place)
{
    const bool shaped = batch >= 0 && q_heads >= 1 && kv_heads >= 1 && q_heads % kv_heads == 0 &&
                        q_heads / kv_heads <= 16 && dim == 128 && context_length >= 1 &&
                        q_stride >= q_heads * dim && std::isfinite(scale);
    if (!shaped)
        return entry.refuse("invalid decode attention arguments");
    if (batch == 0)
        return 0;
    if (!usable({{q, 16}, {k_cache, 16}, {v_cache, 16}, {output, 16}}) || q_stride % 8 != 0 ||
        !apart(output, {q, k_cache, v_cache}))
        return entry.refuse("invalid decode attention buffers");
    int splits = 1;
    const size_t bytes = gqa_decode_scratch_bytes(batch, q_heads, dim, context_length, &splits);
    void *partials = nullptr;
    if (const int refused = place(bytes, &partials))
        return refused;
    entry.context()->counts[6]++;
    return entry.finish(launch_gqa_decode(entry.stream(), batch, q_heads, kv_heads, dim, context_length, lengths,
                                          scale, q, q_stride, k_cache, v_cache, output, partials, splits),
                        "decode attention");
}
} // namespace
} // namespace camblas_hip

extern "C" int camblas_cuda_gqa_decode_attention(camblas_cuda_context *context, int batch,
                                                 int q_heads, int kv_heads, int dim,
                                                 int context_length, const int32_t *lengths,
                                                 float scale, const void *q, int q_stride,
                                                 const void *k_cache, const void *v_cache,
                                                 void *output)
{
    Entry entry(context);
    return entry.run([&] {
        return decode_attention(entry, batch, q_heads, kv_heads, dim, context_length, lengths, scale, q, q_stride,
                                k_cache, v_cache, output, [&](size_t bytes, void **where) {
                                    const hipError_t grown = reserve_scratch(context, bytes);
                                    if (grown != hipSuccess)
                                        return entry.refuse("decode attention scratch", int(grown));
                                    *where = context->scratch;
                                    return 0;
                                });
    });
}

// A decode step's rotary embedding, cache append and attention in one call (two launches instead
// of three): qkv holds the step's un-rotated activation rows [q heads | k heads | v heads], token_stride
// elements apart; positions[b] is the cache slot of sequence b's new token. Equals, bit for bit,
// camblas_cuda_rope_kv_append followed by camblas_cuda_gqa_decode_attention with lengths = positions + 1,
// except that qkv itself is left as it was (the rotated queries live in registers only).
extern "C" int camblas_cuda_rope_append_gqa_decode_attention(camblas_cuda_context *context, int batch, int q_heads,
                                                             int kv_heads, int dim, int context_length,
                                                             const int32_t *positions, float theta, float scale,
                                                             const void *qkv, int token_stride, void *k_cache,
                                                             void *v_cache, const float *angles, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = batch >= 0 && q_heads >= 1 && kv_heads >= 1 && q_heads % kv_heads == 0 &&
                            q_heads / kv_heads <= 16 && dim == 128 && context_length >= 1 &&
                            token_stride >= (q_heads + 2 * kv_heads) * dim && token_stride % 8 == 0 &&
                            std::isfinite(scale) && std::isfinite(theta) && theta > 0;
        if (!shaped)
            return entry.refuse("invalid decode attention arguments");
        if (batch == 0)
            return 0;
        if (!usable({{qkv, 16}, {k_cache, 16}, {v_cache, 16}, {output, 16}, {positions, 4}}) ||
            !is_aligned(angles, 4) || !apart(output, {qkv, k_cache, v_cache}) || !apart(k_cache, {qkv, v_cache}) || !apart(v_cache, {qkv}))
            return entry.refuse("invalid decode attention buffers");
        int splits = 1;
        const size_t bytes = gqa_decode_scratch_bytes(batch, q_heads, dim, context_length, &splits);
        const hipError_t grown = reserve_scratch(context, bytes);
        if (grown != hipSuccess)
            return entry.refuse("decode attention scratch", int(grown));
        context->counts[6]++;
        const unsigned short *rows = static_cast<const unsigned short *>(qkv);
        return entry.finish(launch_gqa_decode(entry.stream(), batch, q_heads, kv_heads, dim, context_length, nullptr,
                                              scale, rows, token_stride, k_cache, v_cache, output, context->scratch,
                                              splits, positions, theta, rows + size_t(q_heads) * dim,
                                              rows + size_t(q_heads + kv_heads) * dim, angles),
                            "decode attention with rotary embedding and cache append");
    });
}

// The angles of a decode step, once for all layers: angles[b][0][i] = sin, angles[b][1][i] = cos of
// positions[b] * theta^(-2i/dim), i < dim / 2, FP32, the values the rotary kernels work out themselves.
extern "C" int camblas_cuda_rope_angles(camblas_cuda_context *context, int batch, int dim, float theta,
                                        const int32_t *positions, float *angles)
{
    Entry entry(context);
    return entry.run([&] {
        if (batch < 0 || batch > (1 << 20) || !within({{dim, 2, 1024, 2}}) || !std::isfinite(theta) || !(theta > 0))
            return entry.refuse("invalid rotary embedding arguments");
        if (batch == 0)
            return 0;
        if (!usable({{positions, 4}, {angles, 4}}))
            return entry.refuse("invalid rotary embedding buffers");
        return entry.finish(launch_rope_table(entry.stream(), batch, dim, theta, positions, angles), "rotary angles");
    });
}

extern "C" size_t camblas_cuda_gqa_decode_attention_noalloc_limit(void)
{
    return gqa_resident_scratch_bytes();
}

// The same kernels with the partials in the library's fixed device array: no hipMalloc, no
// hipFree, no context scratch. Calls that overlap on one GPU share that array and race.
extern "C" int camblas_cuda_gqa_decode_attention_noalloc(camblas_cuda_context *context, int batch,
                                                         int q_heads, int kv_heads, int dim,
                                                         int context_length, const int32_t *lengths,
                                                         float scale, const void *q, int q_stride,
                                                         const void *k_cache, const void *v_cache,
                                                         void *output)
{
    Entry entry(context);
    return entry.run([&] {
        return decode_attention(
            entry, batch, q_heads, kv_heads, dim, context_length, lengths, scale, q, q_stride, k_cache, v_cache,
            output, [&](size_t bytes, void **where) {
                if (bytes > gqa_resident_scratch_bytes()) {
                    std::snprintf(context->error, sizeof(context->error),
                                  "decode attention needs %zu bytes of partials; the allocation-free entry "
                                  "point holds %zu",
                                  bytes, gqa_resident_scratch_bytes());
                    return -1;
                }
                return entry.finish(gqa_resident_scratch(context->device, where),
                                    "resident decode attention partials");
            });
    });
}
