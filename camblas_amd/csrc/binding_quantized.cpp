// Quantised products of the ATen binding: the FP8 block-scaled linear (1 x 128 / 128 x 128 FP32
// scales), the single-token block-32 pair, the E8M0 block-scaled products with their grouped form,
// and the expert routing helpers (ref for what each takes and returns:
// src/cuda/torch_bindings.cpp:328-600; the C entry points are declared in include/camblas_hip.h).
//
// Operands are admitted with binding::admit against a `Want` (dtypes, rank, density), all on the
// device of the first operand; block geometry is checked with the small helpers below.
#include "binding.hpp"

#include <c10/hip/HIPFunctions.h>

#include <algorithm>
#include <cstdint>
#include <tuple>

namespace py = pybind11;

namespace binding
{
namespace
{
constexpr at::ScalarType E4M3 = at::kFloat8_e4m3fn;
constexpr at::ScalarType E2M1_PAIRS = at::ScalarType::Float4_e2m1fn_x2;
constexpr at::ScalarType E8M0 = at::ScalarType::Float8_e8m0fnu;
constexpr int64_t ROW_LIMIT = 65535; // rows, groups and capacities travel in 16-bit grid dimensions

int64_t blocks(int64_t extent, int64_t block) { return (extent + block - 1) / block; }

camblas_cuda_context *default_context(const Tensor &anchor)
{
    return context_for(anchor.get_device(), current_default_algorithm());
}

// result shaped like `input` with the last dimension replaced
Tensor bf16_like(const Tensor &input, int64_t last)
{
    auto shape = input.sizes().vec();
    shape.back() = last;
    return at::empty(shape, input.options().dtype(at::kBFloat16));
}

// scale tensor of `values`: same leading dimensions, `last` entries in the last one
void admit_row_scales(const char *role, const Tensor &scales, const Tensor &values, int64_t last)
{
    require(scales.dim() == values.dim(), std::string(role) + " rank does not match its values");
    for (int64_t axis = 0; axis + 1 < values.dim(); ++axis)
        require(scales.size(axis) == values.size(axis), std::string(role) + " shape mismatch");
    require(scales.size(-1) == last, std::string(role) + " shape mismatch");
}

// ---------------------------------------------------------------------------- FP32 scales per 128
Tensor fp8_block_matmul_public(const Tensor &a, const Tensor &a_scale, const Tensor &weight,
                               const Tensor &weight_scale)
{
    same_process();
    require(a.is_cuda(), "FP8 operands must live on one GPU");
    const at::Device device = a.device();
    admit("FP8 input", a, device, {{E4M3}, 2, false});
    admit("FP8 weight", weight, device, {{E4M3}, 2, false});
    admit("FP8 input scales", a_scale, device, {{at::kFloat}, 2, false});
    admit("FP8 weight scales", weight_scale, device, {{at::kFloat}, 2, false});
    const int64_t rows = a.size(0), inner = a.size(1), outputs = weight.size(0);
    require(inner > 0 && inner % 128 == 0 && weight.size(1) == inner && rows <= ROW_LIMIT,
            "FP8 block matmul needs [rows, inner] x [outputs, inner] with inner a multiple of 128");
    require(a_scale.size(0) == rows && a_scale.size(1) == inner / 128 &&
                weight_scale.size(0) == blocks(outputs, 128) && weight_scale.size(1) == inner / 128,
            "FP8 scale shapes must be [rows, inner/128] and [ceil(outputs/128), inner/128]");
    c10::DeviceGuard guard(device);
    const Tensor ac = a.contiguous(), wc = weight.contiguous(), as = a_scale.contiguous(),
                 ws = weight_scale.contiguous();
    Tensor result = at::empty({rows, outputs}, a.options().dtype(at::kBFloat16));
    if (rows == 0 || outputs == 0)
        return result;
    camblas_cuda_context *context = default_context(a);
    succeed(camblas_cuda_fp8_block_matmul(context, int(rows), int(outputs), int(inner), ac.const_data_ptr(),
                                          as.const_data_ptr<float>(), wc.const_data_ptr(),
                                          ws.const_data_ptr<float>(), result.mutable_data_ptr()),
            context);
    return result;
}

// ---------------------------------------------------------------------------- FP32 scales per 32, one token
bool fp8_decode_supported_public(int device)
{
    same_process();
    if (device < 0)
        device = int(c10::hip::current_device());
    c10::DeviceGuard guard(c10::Device(c10::kCUDA, c10::DeviceIndex(device)));
    return camblas_cuda_fp8_decode_supported(context_for(device, current_default_algorithm())) != 0;
}

// element stride of a scale tensor along `axis`, as the positive int the C ABI takes
int scale_stride(const Tensor &scales, int64_t axis)
{
    const int64_t stride = scales.stride(axis);
    require(stride > 0 && stride <= INT_MAX, "FP8 scale strides must be positive LP64 values");
    return int(stride);
}

// One token (any leading dimensions of extent one) times E4M3 weights [outputs, inner] whose FP32
// scales [ceil(outputs/32), inner/32] may be strided. With `token_scales` the token is E4M3 with
// FP32 scales per 32 inputs; without, it is BF16 and the kernel quantises it.
Tensor block32_token_product(const Tensor &token, const Tensor *token_scales, const Tensor &weight,
                             const Tensor &weight_scale)
{
    same_process();
    require(token.is_cuda(), "FP8 linear requires GPU BF16/FP8 input and E4M3 weight");
    const at::Device device = token.device();
    admit("FP8 linear input", token, device, {{token_scales ? E4M3 : at::kBFloat16}, -1, true});
    admit("FP8 linear weight", weight, device, {{E4M3}, 2, true});
    admit("FP8 linear weight scales", weight_scale, device, {{at::kFloat}, 2, false});
    const int64_t inner = token.size(-1), outputs = weight.size(0);
    require(inner >= 32 && inner <= 8192 && inner % 32 == 0 && outputs >= 16 && outputs % 16 == 0 &&
                token.numel() == inner && weight.size(1) == inner,
            "Invalid FP8 linear matrix dimensions");
    require(weight_scale.size(0) == blocks(outputs, 32) && weight_scale.size(1) == inner / 32,
            "FP8 weight scale shape does not match its blocks");
    const int row_stride = scale_stride(weight_scale, 0), column_stride = scale_stride(weight_scale, 1);
    c10::DeviceGuard guard(device);
    Tensor result = bf16_like(token, outputs);
    camblas_cuda_context *context = default_context(token);
    if (!token_scales) {
        succeed(camblas_cuda_fp8_linear(context, int(outputs), int(inner), token.const_data_ptr(),
                                        weight.const_data_ptr(), weight_scale.const_data_ptr<float>(), row_stride,
                                        column_stride, nullptr, 0, result.mutable_data_ptr()),
                context);
        return result;
    }
    admit("FP8 input scales", *token_scales, device, {{at::kFloat}, -1, false});
    admit_row_scales("FP8 input scale", *token_scales, token, inner / 32);
    succeed(camblas_cuda_fp8_decode(context, int(outputs), int(inner), token.const_data_ptr(),
                                    token_scales->const_data_ptr<float>(), weight.const_data_ptr(),
                                    weight_scale.const_data_ptr<float>(), scale_stride(*token_scales, -1),
                                    row_stride, column_stride, nullptr, 0, result.mutable_data_ptr()),
            context);
    return result;
}

// ---------------------------------------------------------------------------- E8M0 scales per 32
// Geometry of an E8M0 product: E4M3 weights [outputs, inner] with one scale row per 32 weight rows,
// or packed E2M1 weights [outputs, inner / 2] with one per row; activation scales per 32 inputs, or
// per 128 with packed weights.
struct MxGeometry {
    bool packed;
    int64_t outputs, inner;

    explicit MxGeometry(const Tensor &weight)
        : packed(weight.scalar_type() == E2M1_PAIRS), outputs(weight.size(0)),
          inner(weight.size(1) * (packed ? 2 : 1))
    {
    }
    bool sound() const { return outputs >= 8 && outputs % 8 == 0 && inner >= 32 && inner % 32 == 0; }
    bool accepts_block(int64_t activation_block) const
    {
        return (activation_block == 32 || (packed && activation_block == 128)) && inner % activation_block == 0;
    }
    int64_t scale_rows() const { return packed ? outputs : blocks(outputs, 32); }
    bool scales_fit(const Tensor &scales) const
    {
        return scales.dim() == 2 && scales.size(0) == scale_rows() && scales.size(1) == inner / 32;
    }
};

Tensor quantized_matmul_public(const Tensor &x, const Tensor &x_scale, const Tensor &weight,
                               const Tensor &weight_scale, int activation_block)
{
    same_process();
    require(x.is_cuda(), "Quantized input must be GPU FP8 E4M3");
    const at::Device device = x.device();
    admit("Quantized input", x, device, {{E4M3}, -1, true});
    admit("Quantized weight", weight, device, {{E4M3, E2M1_PAIRS}, 2, true});
    admit("Quantized input scales", x_scale, device, {{E8M0}, -1, true});
    admit("Quantized weight scales", weight_scale, device, {{E8M0}, 2, true});
    const MxGeometry geometry(weight);
    require(geometry.sound() && x.size(-1) == geometry.inner && geometry.accepts_block(activation_block),
            "Invalid quantized matrix dimensions or activation block");
    admit_row_scales("Input scale", x_scale, x, geometry.inner / activation_block);
    require(geometry.scales_fit(weight_scale), "Quantized scale shapes do not match their blocks");
    const int64_t rows = flattened_rows(x, ROW_LIMIT, "Quantized multiplication supports at most 65535 rows");
    c10::DeviceGuard guard(device);
    Tensor result = bf16_like(x, geometry.outputs);
    camblas_cuda_context *context = default_context(x);
    succeed(camblas_cuda_quantized_matmul(context, geometry.packed, int(rows), int(geometry.outputs),
                                          int(geometry.inner), activation_block, x.const_data_ptr(),
                                          x_scale.const_data_ptr(), weight.const_data_ptr(),
                                          weight_scale.const_data_ptr(), result.mutable_data_ptr()),
            context);
    return result;
}

// The weights and scales of a set of experts, kept alive, with their device addresses in a table
// the grouped kernel reads. Values may change in place between calls; storage that has moved since
// construction is refused (the table would point at freed memory).
class QuantizedGroups
{
  public:
    QuantizedGroups(const std::vector<Tensor> &weights, const std::vector<Tensor> &scales)
    {
        same_process();
        require(!weights.empty() && int64_t(weights.size()) <= ROW_LIMIT && weights.size() == scales.size(),
                "Supply matching non-empty weight and scale groups");
        require(weights[0].is_cuda() && weights[0].dim() == 2, "Grouped weights must be GPU matrices");
        const at::Device device = weights[0].device();
        const at::ScalarType storage = weights[0].scalar_type();
        require(storage == E4M3 || storage == E2M1_PAIRS, "Grouped weights require FP8 or packed FP4 storage");
        const MxGeometry geometry(weights[0]);
        require(geometry.sound() && geometry.outputs <= INT_MAX && geometry.inner <= INT_MAX,
                "Invalid grouped weight dimensions");
        packed_ = geometry.packed;
        outputs_ = int(geometry.outputs);
        inner_ = int(geometry.inner);
        host_table_ = at::empty({int64_t(weights.size()), 2}, at::TensorOptions().device(at::kCPU).dtype(at::kLong));
        for (size_t group = 0; group < weights.size(); ++group) {
            const Tensor &w = weights[group], &s = scales[group];
            const bool alike = w.device() == device && w.scalar_type() == storage && w.sizes() == weights[0].sizes() &&
                               w.is_contiguous() && reinterpret_cast<uintptr_t>(w.const_data_ptr()) % 16 == 0 &&
                               s.device() == device && s.scalar_type() == E8M0 && s.is_contiguous() &&
                               geometry.scales_fit(s);
            require(alike, "Grouped weight shapes, dtypes, devices or scales differ");
            trainable_ = trainable_ || w.requires_grad() || s.requires_grad();
            weights_.push_back(w.detach());
            scales_.push_back(s.detach());
            record(group, host_table_.mutable_data_ptr<int64_t>());
        }
        c10::DeviceGuard guard(device);
        device_table_ = host_table_.to(device);
    }

    // input [groups, capacity, inner] E4M3 with scales [groups, capacity, inner / block]; active and
    // counts int32 [groups]: which expert a group uses and how many of its rows are filled
    Tensor matmul(const Tensor &x, const Tensor &x_scale, const Tensor &active, const Tensor &counts,
                  int activation_block)
    {
        same_process();
        require(!c10::GradMode::is_enabled() || (!trainable_ && !x.requires_grad()),
                "Grouped multiplication supports inference only");
        const at::Device device = device_table_.device();
        admit("Grouped input", x, device, {{E4M3}, 3, true});
        admit("Grouped input scales", x_scale, device, {{E8M0}, 3, true});
        admit("Grouped active indices", active, device, {{at::kInt}, 1, true});
        admit("Grouped counts", counts, device, {{at::kInt}, 1, true});
        const int64_t groups = x.size(0), capacity = x.size(1);
        MxGeometry geometry(weights_[0]);
        require(groups <= ROW_LIMIT && capacity <= ROW_LIMIT && x.size(2) == inner_ &&
                    geometry.accepts_block(activation_block),
                "Invalid grouped input dimensions or activation block");
        admit_row_scales("Grouped input scale", x_scale, x, inner_ / activation_block);
        require(active.numel() == groups && counts.numel() == groups,
                "Grouped indices/counts require one GPU int32 value per group");
        std::vector<int64_t> now(2 * weights_.size());
        for (size_t group = 0; group < weights_.size(); ++group)
            record(group, now.data());
        require(std::equal(now.begin(), now.end(), host_table_.const_data_ptr<int64_t>()),
                "Captured weight storage changed; recreate the group");
        c10::DeviceGuard guard(device);
        Tensor result = at::empty({groups, capacity, outputs_}, x.options().dtype(at::kBFloat16));
        camblas_cuda_context *context = default_context(x);
        succeed(camblas_cuda_grouped_quantized_matmul(
                    context, packed_, int(groups), int(weights_.size()), int(capacity), outputs_, inner_,
                    activation_block, x.const_data_ptr(), x_scale.const_data_ptr(), device_table_.const_data_ptr(),
                    active.const_data_ptr(), counts.const_data_ptr(), result.mutable_data_ptr()),
                context);
        return result;
    }

  private:
    // addresses of group `group`'s weight and scale storage into table[2 * group ..]
    void record(size_t group, int64_t *table) const
    {
        table[2 * group] = int64_t(reinterpret_cast<uintptr_t>(weights_[group].const_data_ptr()));
        table[2 * group + 1] = int64_t(reinterpret_cast<uintptr_t>(scales_[group].const_data_ptr()));
    }

    std::vector<Tensor> weights_, scales_;
    Tensor host_table_, device_table_; // int64 [groups, 2]
    int outputs_ = 0, inner_ = 0;
    bool packed_ = false, trainable_ = false;
};

// ---------------------------------------------------------------------------- expert routing
// experts int64 [tokens, choices]; active int32 [groups] (the expert each group serves); returns
// (slots [groups, rows], reverse [tokens, choices], counts [groups])
std::tuple<Tensor, Tensor, Tensor> route_groups_public(const Tensor &experts, const Tensor &active,
                                                       int first_expert, int rows)
{
    same_process();
    const char *refusal = "Invalid expert routing dimensions, indices or devices";
    require(experts.is_cuda(), refusal);
    const at::Device device = experts.device();
    admit("Expert IDs", experts, device, {{at::kLong}, 2, true});
    admit("Active experts", active, device, {{at::kInt}, 1, true});
    const int64_t tokens = experts.size(0), choices = experts.size(1), groups = active.numel();
    require(choices >= 1 && choices <= 64 && experts.numel() <= INT_MAX && groups >= 1 && groups <= ROW_LIMIT &&
                rows >= 1 && rows <= ROW_LIMIT && groups * rows <= INT_MAX && first_expert >= 0,
            refusal);
    c10::DeviceGuard guard(device);
    Tensor counts = at::empty({groups}, active.options());
    Tensor slots = at::empty({groups, rows}, active.options());
    Tensor reverse = at::empty(experts.sizes(), active.options());
    camblas_cuda_context *context = default_context(experts);
    succeed(camblas_cuda_route_groups(context, int(tokens), int(choices), first_expert, int(groups), rows,
                                      experts.const_data_ptr(), active.const_data_ptr(), counts.mutable_data_ptr(),
                                      slots.mutable_data_ptr(), reverse.mutable_data_ptr()),
            context);
    return std::make_tuple(slots, reverse, counts);
}

// input BF16 [groups, rows, width]; returns FP32 [tokens, width], each token's choices summed in
// (expert, choice) order
Tensor reduce_groups_public(const Tensor &input, const Tensor &experts, const Tensor &reverse)
{
    same_process();
    const char *refusal = "Invalid grouped reduction shapes, types, devices or gradients";
    require(input.is_cuda(), refusal);
    const at::Device device = input.device();
    admit("Grouped rows", input, device, {{at::kBFloat16}, 3, true});
    admit("Expert IDs", experts, device, {{at::kLong}, 2, true});
    admit("Reverse map", reverse, device, {{at::kInt}, 2, true});
    const int64_t grouped_rows = input.size(0) * input.size(1), width = input.size(2);
    require(grouped_rows <= INT_MAX && width >= 1 && experts.size(1) >= 1 && experts.size(1) <= 64 &&
                experts.numel() <= INT_MAX && reverse.sizes() == experts.sizes(),
            refusal);
    c10::DeviceGuard guard(device);
    Tensor result = at::empty({experts.size(0), width}, input.options().dtype(at::kFloat));
    camblas_cuda_context *context = default_context(input);
    succeed(camblas_cuda_reduce_groups(context, int(experts.size(0)), int(experts.size(1)), int(width),
                                       int(grouped_rows), experts.const_data_ptr(), reverse.const_data_ptr(),
                                       input.const_data_ptr(), result.mutable_data_ptr()),
            context);
    return result;
}
} // namespace

void register_quantized(py::module_ &module)
{
    module.def("fp8_block_matmul", &fp8_block_matmul_public, py::arg("input"), py::arg("input_scale"),
               py::arg("weight"), py::arg("weight_scale"),
               "Multiply E4M3fn activations (1x128 FP32 scales) by E4M3fn weights (128x128 FP32 "
               "scales), returning BF16.");
    module.attr("quantized_tile_rows") = 16;
    py::class_<QuantizedGroups>(module, "QuantizedGroups",
                                "Capture GPU quantized weight storages and retain their lifetimes. "
                                "In-place value updates are visible; recreate the group after "
                                "storage relocation.")
        .def(py::init<const std::vector<Tensor> &, const std::vector<Tensor> &>(), py::arg("weights"),
             py::arg("scales"))
        .def("matmul", &QuantizedGroups::matmul, py::arg("input"), py::arg("input_scale"), py::arg("active"),
             py::arg("counts"), py::kw_only(), py::arg("activation_block") = 32,
             "Multiply [groups,rows,inner] FP8 input with selected captured weights. Invalid "
             "active indices and padding return zero; counts clip to [0,rows]. Inference only.");
    module.def("route_groups", &route_groups_public, py::arg("experts"), py::arg("active"), py::kw_only(),
               py::arg("first_expert") = 0, py::arg("rows"),
               "Return slots, reverse mapping and counts for expert/choice IDs. Excess rows are "
               "discarded and unassigned slots are -1; execution uses the active stream.");
    module.def("reduce_groups", &reduce_groups_public, py::arg("input"), py::arg("experts"), py::arg("reverse"),
               "Sum BF16 contributions into FP32 in expert/choice order. Invalid IDs/rows are "
               "ignored; requires inference and contiguous GPU tensors.");
    module.def("quantized_matmul", &quantized_matmul_public, py::arg("input"), py::arg("input_scale"),
               py::arg("weight"), py::arg("weight_scale"), py::kw_only(), py::arg("activation_block") = 32,
               "Multiply block-scaled FP8 input by FP8 or packed FP4 weights, returning BF16. "
               "Requires contiguous GPU operands and E8M0 scales.");
    module.def("fp8_decode_supported", &fp8_decode_supported_public, py::arg("device") = -1,
               "Return whether this build and device support the block-32 FP8 decode product.");
    module.def(
        "fp8_decode",
        [](const Tensor &x, const Tensor &x_scale, const Tensor &weight, const Tensor &weight_scale) {
            return block32_token_product(x, &x_scale, weight, weight_scale);
        },
        py::arg("input"), py::arg("input_scale"), py::arg("weight"), py::arg("weight_scale"),
        "Multiply one block32 E4M3 token by E4M3 weights, using FP32 scales and ordered FP32 "
        "accumulation; positive scale strides are allowed.");
    module.def(
        "fp8_linear",
        [](const Tensor &x, const Tensor &weight, const Tensor &weight_scale) {
            return block32_token_product(x, nullptr, weight, weight_scale);
        },
        py::arg("input"), py::arg("weight"), py::arg("weight_scale"),
        "Quantise one finite BF16 token to block32 E4M3 with power-of-two FP32 scales and "
        "multiply E4M3 weights with ordered FP32 accumulation.");
}
} // namespace binding
