// Quantised products of the C ABI: the FP8 E4M3fn block-scaled linear (1 x 128 activation groups,
// 128 x 128 weight blocks, FP32 scales; arithmetic rule of camblas/_hopper.py:118-126, :168-182),
// its dynamic activation quantiser (:82-98), the single-token block-32 pair of the reference
// header (include/camblas_cuda.h:124-155, src/cuda/backend.cu:1193-1256), the E8M0 block-scaled
// products with their grouped form (camblas_cuda.h:110-123, :156-185; backend.cu:1165-1191,
// :1258-1303), the routing helpers (backend.cu:1306-1361) and the fused single-token expert step
// (camblas/_hopper.py:329-401). Argument rules follow those wrappers; the kernels are this
// library's own.
#include "entry.hpp"

#include <climits>
#include <cmath>

namespace camblas_hip
{
namespace
{
constexpr int ROW_LIMIT = 65535; // rows, groups and capacities travel in 16-bit grid dimensions

// Planner's choice for the FP8 block-scaled product, or the variant a test forced:
// 0.. register-staged tiles (with split-K), 20.. direct-to-LDS tiles, 100 + 10*row_tiles +
// token_tiles the streaming kernel.
Plan fp8_plan(const camblas_cuda_context *context, int rows, int outputs, int inner, const void *out)
{
    Plan plan = make_plan(3, context->algorithm, true, false, outputs, rows, inner, inner, inner, outputs, true,
                          context->compute_units);
    if (plan.family == FAMILY_FP8_DMA && !is_aligned(out, 8))
        plan = Plan{FAMILY_FP8_BLOCK, 0, 1, 4};
    const int forced = context->override_kernel;
    if (forced < 0)
        return plan;
    plan.split_k = 1;
    plan.tail_outputs = 0;
    if (forced >= 100) {
        plan.family = FAMILY_FP8_STREAM;
        plan.kernel = forced - 100;
        return plan;
    }
    plan.family = forced >= 20 ? FAMILY_FP8_DMA : FAMILY_FP8_BLOCK;
    plan.kernel = forced >= 20 ? forced - 20 : forced;
    if (context->override_split > 0)
        plan.split_k = std::min(context->override_split, inner / 128);
    return plan;
}

// what both E8M0 products accept as shapes: outputs in eights, inner in 32s, activation scale blocks
// of 32, or of 128 with packed E2M1 weights
bool mx_shapes(int packed, int outputs, int inner, int activation_block)
{
    return is_flag(packed) && within({{outputs, 8, INT_MAX, 8}, {inner, 32, INT_MAX, 32}}) &&
           (activation_block == 32 || (packed && activation_block == 128)) && inner % activation_block == 0;
}

bool block32_shapes(int outputs, int inner, std::initializer_list<int> strides)
{
    for (int stride : strides)
        if (stride < 1)
            return false;
    return within({{outputs, 16, INT_MAX, 16}, {inner, 32, 8192, 32}});
}
} // namespace
} // namespace camblas_hip

using namespace camblas_hip;

// ---- FP8 E4M3fn, FP32 scales per 1 x 128 / 128 x 128 block

extern "C" int camblas_cuda_fp8_block_matmul(camblas_cuda_context *context, int rows, int outputs,
                                             int inner, const void *a, const float *a_scale,
                                             const void *w, const float *w_scale, void *out)
{
    Entry entry(context);
    return entry.run([&] {
        if (!within({{rows, 0, ROW_LIMIT, 1}, {outputs, 1, INT_MAX, 1}, {inner, 128, INT_MAX, 128}}))
            return entry.refuse("invalid FP8 block matrix dimensions");
        if (rows == 0)
            return 0;
        if (!usable({{a, 16}, {w, 16}, {a_scale, 4}, {w_scale, 4}, {out, 2}}) ||
            !apart(out, {a, w, a_scale, w_scale}))
            return entry.refuse("invalid FP8 block matrix buffers");
        Plan plan = fp8_plan(context, rows, outputs, inner, out);
        hipStream_t stream = context->stream;
        if (plan.family == FAMILY_FP8_STREAM) {
            context->counts[plan.counter]++;
            return entry.finish(launch_fp8_stream(stream, plan.kernel / 10, plan.kernel % 10, rows, outputs, inner,
                                                  a, a_scale, w, w_scale, out),
                                "FP8 block-scaled streaming GEMV");
        }
        float *partials = nullptr;
        if (plan.split_k > 1) {
            // without room for the partials (allocation failure, capture in progress) run unsplit
            if (reserve_scratch(context, size_t(plan.split_k) * size_t(rows) * size_t(outputs) * 4) ==
                hipSuccess) {
                partials = static_cast<float *>(context->scratch);
            } else {
                context->counts[5]++;
                plan.split_k = 1;
            }
        }
        context->counts[plan.counter]++;
        if (plan.family == FAMILY_FP8_DMA)
            return entry.finish(launch_fp8_dma(stream, plan.kernel, plan.split_k, rows, outputs, inner, a, a_scale,
                                               w, w_scale, out, partials, plan.tail_kernel, plan.tail_outputs),
                                "FP8 block-scaled GEMM (direct LDS loads)");
        return entry.finish(launch_fp8_block(stream, plan.kernel, plan.split_k, rows, outputs, inner, a, a_scale,
                                             w, w_scale, out, partials),
                            "FP8 block-scaled GEMM");
    });
}

extern "C" int camblas_cuda_fp8_quantise_1x128(camblas_cuda_context *context, int rows, int inner,
                                               const void *x, void *q, float *scale)
{
    Entry entry(context);
    return entry.run([&] {
        if (!within({{rows, 0, INT_MAX, 1}, {inner, 128, INT_MAX, 128}}))
            return entry.refuse("invalid FP8 quantiser dimensions");
        if (rows == 0)
            return 0;
        if (!usable({{x, 16}, {q, 16}, {scale, 4}}) || q == x)
            return entry.refuse("invalid FP8 quantiser buffers");
        return entry.finish(launch_fp8_quantise(context->stream, rows, inner, x, q, scale),
                            "FP8 activation quantisation");
    });
}

// workspace of camblas_cuda_fp8_block_linear: the quantised rows (padded to 16 bytes), then their scales
extern "C" size_t camblas_cuda_fp8_block_workspace_size(int rows, int inner)
{
    if (!within({{rows, 1, INT_MAX, 1}, {inner, 128, INT_MAX, 128}}))
        return 0;
    const size_t bytes = (size_t(rows) * inner + 15) / 16 * 16;
    return bytes + size_t(rows) * (inner / 128) * sizeof(float);
}

extern "C" int camblas_cuda_fp8_block_linear(camblas_cuda_context *context, int rows, int outputs,
                                             int inner, const void *x, const void *w,
                                             const float *w_scale, void *workspace,
                                             size_t workspace_bytes, void *out)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    if (!within({{rows, 0, ROW_LIMIT, 1}, {outputs, 1, INT_MAX, 1}, {inner, 128, INT_MAX, 128}}))
        return fail(context, "invalid FP8 block matrix dimensions", 1);
    if (rows == 0)
        return 0;
    const size_t needed = camblas_cuda_fp8_block_workspace_size(rows, inner);
    if (!usable({{workspace, 16}}) || workspace_bytes < needed || !apart(workspace, {x, w, out}))
        return fail(context, "invalid FP8 block linear workspace", 1);
    unsigned char *codes = static_cast<unsigned char *>(workspace);
    float *scales = reinterpret_cast<float *>(codes + (needed - size_t(rows) * (inner / 128) * sizeof(float)));
    if (const int status = camblas_cuda_fp8_quantise_1x128(context, rows, inner, x, codes, scales))
        return status;
    return camblas_cuda_fp8_block_matmul(context, rows, outputs, inner, codes, scales, w, w_scale, out);
}

// ---- single token, FP32 scales per 32 inputs (the reference header's pair)

extern "C" int camblas_cuda_fp8_decode_supported(const camblas_cuda_context *context)
{
    return context ? 1 : 0;
}

// both operations are single kernels that stage the token in LDS: no workspace
extern "C" size_t camblas_cuda_fp8_workspace_size(int, int, int) { return 0; }

extern "C" int camblas_cuda_fp8_decode(camblas_cuda_context *context, int outputs, int inner,
                                       const void *input, const float *input_scale,
                                       const void *weight, const float *weight_scale,
                                       int input_scale_stride, int weight_scale_row_stride,
                                       int weight_scale_column_stride, void *, size_t, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (!block32_shapes(outputs, inner,
                            {input_scale_stride, weight_scale_row_stride, weight_scale_column_stride}))
            return entry.refuse("invalid FP8 decode dimensions or scale strides");
        if (!usable({{input, 4}, {weight, 16}, {input_scale, 4}, {weight_scale, 4}, {output, 2}}) ||
            !apart(output, {input, weight, input_scale, weight_scale}))
            return entry.refuse("invalid FP8 decode buffers");
        context->counts[4]++;
        const int forced = context->override_kernel; // (tests: 301 / 302 / 304 force the wavefronts per workgroup)
        return entry.finish(launch_fp8_block32_decode(context->stream, outputs, inner, input, input_scale,
                                                      input_scale_stride, weight, weight_scale,
                                                      weight_scale_row_stride, weight_scale_column_stride, output,
                                                      forced == 301 || forced == 302 || forced == 304 ? forced - 300 : 0),
                            "FP8 block-32 decode");
    });
}

extern "C" int camblas_cuda_fp8_linear(camblas_cuda_context *context, int outputs, int inner,
                                       const void *input, const void *weight,
                                       const float *weight_scale, int weight_scale_row_stride,
                                       int weight_scale_column_stride, void *, size_t, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (!block32_shapes(outputs, inner, {weight_scale_row_stride, weight_scale_column_stride}))
            return entry.refuse("invalid FP8 decode dimensions or scale strides");
        if (!usable({{input, 4}, {weight, 16}, {weight_scale, 4}, {output, 2}}) ||
            !apart(output, {input, weight, weight_scale}))
            return entry.refuse("invalid FP8 decode buffers");
        context->counts[4]++;
        // no input scales: the kernel quantises the BF16 token itself
        return entry.finish(launch_fp8_block32_decode(context->stream, outputs, inner, input, nullptr, 1, weight,
                                                      weight_scale, weight_scale_row_stride,
                                                      weight_scale_column_stride, output),
                            "FP8 block-32 linear");
    });
}

// ---- E8M0 scales per 32 inputs (E4M3 or packed E2M1 weights)

extern "C" int camblas_cuda_quantized_matmul(camblas_cuda_context *context, int packed, int rows,
                                             int outputs, int inner, int activation_block,
                                             const void *input, const void *input_scale,
                                             const void *weight, const void *weight_scale,
                                             void *output)
{
    Entry entry(context);
    return entry.run([&] {
        if (!mx_shapes(packed, outputs, inner, activation_block) || !within({{rows, 0, ROW_LIMIT, 1}}))
            return entry.refuse("invalid quantized matrix dimensions");
        if (rows == 0)
            return 0;
        if (!usable({{input, 16}, {input_scale, 1}, {weight, 16}, {weight_scale, 1}, {output, 2}}) ||
            !apart(output, {input, input_scale, weight, weight_scale}))
            return entry.refuse("invalid quantized matrix buffers");
        context->counts[4]++;
        // K divided over several workgroups per tile needs FP32 planes; without them (allocation
        // failure, capture in progress) the same tiles run with K undivided
        const int shares = mx_matmul_shares(context->override_kernel, context->override_split, context->compute_units,
                                            packed != 0, rows, outputs, inner, activation_block, input, weight, output);
        float *planes = nullptr;
        if (shares > 1) {
            if (reserve_scratch(context, size_t(shares) * size_t(rows) * size_t(outputs) * 4) == hipSuccess)
                planes = static_cast<float *>(context->scratch);
            else
                context->counts[5]++;
        }
        return entry.finish(launch_mx_matmul(context->stream, context->override_kernel, context->compute_units,
                                             packed != 0, 0, 0, rows, outputs, inner, activation_block, input,
                                             input_scale, weight, weight_scale, nullptr, nullptr, nullptr, output,
                                             context->override_split, planes),
                            "quantized matrix multiplication");
    });
}

// The kernel writes the zeros of inactive groups and of padding rows itself, so the call holds no
// memset and can be captured in a graph.
extern "C" int camblas_cuda_grouped_quantized_matmul(camblas_cuda_context *context, int packed,
                                                     int groups, int weight_groups, int rows,
                                                     int outputs, int inner, int activation_block,
                                                     const void *input, const void *input_scale,
                                                     const void *metadata, const void *active,
                                                     const void *counts, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = mx_shapes(packed, outputs, inner, activation_block) &&
                            within({{groups, 0, ROW_LIMIT, 1}, {weight_groups, 1, ROW_LIMIT, 1}, {rows, 0, ROW_LIMIT, 1}}) &&
                            uint64_t(groups) * uint64_t(rows) <= SIZE_MAX / (uint64_t(outputs) * 2);
        if (!shaped)
            return entry.refuse("invalid grouped matrix dimensions");
        if (groups == 0 || rows == 0)
            return 0;
        if (!usable({{input, 16}, {input_scale, 1}, {metadata, 8}, {active, 4}, {counts, 4}, {output, 2}}) ||
            !apart(output, {input, input_scale, metadata, active, counts}))
            return entry.refuse("invalid grouped matrix buffers");
        context->counts[4]++;
        return entry.finish(launch_mx_matmul(context->stream, context->override_kernel, context->compute_units,
                                             packed != 0, groups, weight_groups, rows, outputs, inner,
                                             activation_block, input, input_scale, nullptr, nullptr, metadata,
                                             active, counts, output),
                            "grouped multiplication");
    });
}

// ---- expert routing

extern "C" int camblas_cuda_route_groups(camblas_cuda_context *context, int tokens, int choices,
                                         int first_expert, int groups, int rows,
                                         const void *experts, const void *active, void *counts,
                                         void *slots, void *reverse)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped =
            within({{tokens, 0, INT_MAX, 1}, {choices, 1, 64, 1}, {first_expert, 0, INT_MAX, 1},
                    {groups, 1, ROW_LIMIT, 1}, {rows, 1, ROW_LIMIT, 1},
                    {int64_t(tokens) * choices, 0, INT_MAX, 1}, {int64_t(groups) * rows, 0, INT_MAX, 1}});
        // with no tokens the expert table and the reverse map may be absent
        const bool present = usable({{counts, 4}, {slots, 4}, {active, 4}, {experts, 8, tokens == 0},
                                     {reverse, 4, tokens == 0}});
        const bool distinct = all_apart({counts, slots, reverse, active}) && apart(experts, {counts, slots, reverse});
        if (!shaped || !present || !distinct)
            return entry.refuse("invalid routing dimensions or buffers");
        return entry.finish(launch_route_groups(context->stream, tokens, choices, first_expert, groups, rows,
                                                experts, active, counts, slots, reverse),
                            "expert routing");
    });
}

extern "C" int camblas_cuda_reduce_groups(camblas_cuda_context *context, int tokens, int choices,
                                          int width, int grouped_rows, const void *experts,
                                          const void *reverse, const void *input, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        const bool shaped = within({{tokens, 0, INT_MAX, 1}, {choices, 1, 64, 1}, {width, 1, INT_MAX, 1},
                                    {grouped_rows, 0, INT_MAX, 1}, {int64_t(tokens) * choices, 0, INT_MAX, 1}});
        const bool present = usable({{input, 2, grouped_rows == 0}, {experts, 8, tokens == 0},
                                     {reverse, 4, tokens == 0}, {output, 4, tokens == 0}});
        if (!shaped || !present || (tokens && !apart(output, {experts, reverse, input})))
            return entry.refuse("invalid grouped reduction arguments");
        if (tokens == 0)
            return 0;
        return entry.finish(launch_reduce_groups(context->stream, tokens, choices, width, grouped_rows, experts,
                                                 reverse, input, output),
                            "grouped reduction");
    });
}

// ---- one token through a block-scaled FP8 mixture-of-experts layer (the reference reaches this
// step from Python only; here it is an entry point like the other products)

extern "C" int camblas_cuda_fp8_moe_decode(camblas_cuda_context *context, int experts, int choices,
                                           int hidden, int width, int hidden_out, const void *x,
                                           const void *w1, const float *w1_scale, const void *w2,
                                           const float *w2_scale, const int32_t *expert_ids,
                                           const float *routing, float factor, void *output)
{
    Entry entry(context);
    return entry.run([&] {
        // choices * width / 128 scale products live in the second launch's LDS
        const bool shaped = within({{experts, 1, INT_MAX, 1}, {choices, 1, 16, 1}, {hidden, 128, INT_MAX, 128},
                                    {width, 128, INT_MAX, 128}, {hidden_out, 16, INT_MAX, 16}}) &&
                            int64_t(choices) * (width / 128) <= 512 && std::isfinite(factor);
        if (!shaped)
            return entry.refuse("invalid FP8 expert dimensions");
        if (!usable({{x, 16}, {w1, 16}, {w2, 16}, {w1_scale, 4}, {w2_scale, 4}, {expert_ids, 4}, {routing, 4},
                     {output, 2}}) ||
            !apart(output, {w1, w2}))
            return entry.refuse("invalid FP8 expert buffers");
        const hipError_t grown = reserve_scratch(context, fp8_moe_decode_scratch_bytes(choices, width));
        if (grown != hipSuccess)
            return entry.refuse("FP8 expert scratch", int(grown));
        context->counts[4]++;
        return entry.finish(launch_fp8_moe_decode(context->stream, experts, choices, hidden, width, hidden_out, x,
                                                  w1, w1_scale, w2, w2_scale, expert_ids, routing, factor,
                                                  context->scratch, output),
                            "FP8 expert step");
    });
}
