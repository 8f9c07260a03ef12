// Inference fusions of the ATen binding: SiLU-multiply, SwiGLU, the RMS normalisation family, the
// gated MLP and the three-way projection (ref for what each computes and where it rounds:
// src/cuda/inference_fusion.cuh:19-51, :136-191 and src/cuda/torch_bindings.cpp:602-736). All of
// them take FP32 or BF16 GPU tensors that do not require gradients.
#include "binding.hpp"

#include <cfloat>
#include <cmath>
#include <tuple>

namespace py = pybind11;

namespace binding
{
namespace
{
camblas_cuda_context *fusion_context(const Tensor &anchor, int algorithm = -1)
{
    return context_for(anchor.get_device(), resolve(algorithm));
}

// the gate / up pair of an activation: same shape, same dtype, same GPU, no gradients
struct GatedPair {
    Tensor gate, up;

    GatedPair(const Tensor &gate_in, const Tensor &up_in, const char *mismatch)
    {
        check_inference(gate_in, gate_in);
        check_inference(up_in, gate_in);
        require(gate_in.sizes().equals(up_in.sizes()), mismatch);
        gate = gate_in.contiguous();
        up = up_in.contiguous();
    }
    int storage() const { return storage_code(gate); }
    uint64_t count() const { return uint64_t(gate.numel()); }
    Tensor like() const { return at::empty(gate.sizes(), gate.options()); }
};

// round(silu(gate)) * up, rounded again: two roundings, as the reference's gated MLP does
Tensor silu_times(const Tensor &gate, const Tensor &up)
{
    const GatedPair pair(gate, up, "SiLU operands must have matching shapes");
    c10::DeviceGuard guard(gate.device());
    Tensor result = pair.like();
    camblas_cuda_context *context = fusion_context(gate);
    succeed(camblas_cuda_silu_multiply(context, pair.storage(), pair.count(), pair.gate.const_data_ptr(),
                                       pair.up.const_data_ptr(), result.mutable_data_ptr()),
            context);
    return result;
}

// silu(min(gate, limit)) * clamp(up, +-limit) in FP32 (limit 0: no clipping), optionally times one
// routing weight per row, one rounding
Tensor swiglu_rows(const Tensor &gate, const Tensor &up, const std::optional<Tensor> &routing, double limit)
{
    const GatedPair pair(gate, up, "Invalid SwiGLU shapes or clipping limit");
    const bool limited = std::isfinite(limit) && limit >= 0 && limit <= FLT_MAX;
    require(gate.dim() >= 1 && gate.size(-1) > 0 && limited, "Invalid SwiGLU shapes or clipping limit");
    c10::DeviceGuard guard(gate.device());
    Tensor weights;
    if (routing) {
        check_inference(*routing, *routing);
        require(routing->scalar_type() == at::kFloat && routing->device() == gate.device(),
                "SwiGLU routing values must be FP32 on the input device");
        // one value per row: shaped like the input without its last dimension, or with it as 1
        const auto rows = gate.sizes().slice(0, gate.dim() - 1);
        const bool flat = routing->sizes().equals(rows);
        const bool column = routing->dim() == gate.dim() && routing->size(-1) == 1 &&
                            routing->sizes().slice(0, gate.dim() - 1).equals(rows);
        require(flat || column, "SwiGLU routing requires one value per input row");
        weights = routing->contiguous();
    }
    Tensor result = pair.like();
    camblas_cuda_context *context = fusion_context(gate);
    succeed(camblas_cuda_swiglu(context, pair.storage(), pair.count(), int(gate.size(-1)), float(limit),
                                pair.gate.const_data_ptr(), pair.up.const_data_ptr(),
                                weights.defined() ? weights.const_data_ptr<float>() : nullptr,
                                result.mutable_data_ptr()),
            context);
    return result;
}

// Row-wise RMS normalisation, optionally after a residual add, in one launch for any number of
// rows: added = round(x + residual), out = round(round(added * rsqrt(mean(added^2) + eps)) * w), or
// with round_before_weight false the weight is applied in FP32 before the single rounding. The
// reference composes the multi-row case from a square kernel, ATen's mean and a scale kernel
// (src/cuda/torch_bindings.cpp:602-673); the mean here is the library's own fixed-order sum.
struct Normalised {
    Tensor added, output; // `added` is undefined without a residual
};

Normalised normalise_rows(const Tensor &x, const Tensor *residual, const Tensor &weight, double epsilon,
                          bool round_before_weight)
{
    check_inference(x, x);
    if (round_before_weight) {
        check_inference(weight, x);
    } else { // a final-round weight may also be FP32 for BF16 rows
        check_inference(weight, weight);
        const bool fp32_for_bf16 = x.scalar_type() == at::kBFloat16 && weight.scalar_type() == at::kFloat;
        require(weight.device() == x.device() && (weight.scalar_type() == x.scalar_type() || fp32_for_bf16),
                "Final-round RMS weight must match input dtype or use FP32 with BF16 input");
    }
    require(x.dim() >= 1 && weight.dim() == 1 && weight.size(0) == x.size(-1),
            "RMS norm weight must match the input's last dimension");
    require(std::isfinite(epsilon) && epsilon >= 0 && epsilon <= FLT_MAX,
            "RMS norm epsilon must be finite and nonnegative");
    if (residual) {
        check_inference(*residual, x);
        require(residual->sizes().equals(x.sizes()), "Residual RMS dimensions must match");
    }
    const int64_t rows = flattened_rows(x, INT_MAX, "LP64 flattened row overflow");
    c10::DeviceGuard guard(x.device());
    const Tensor rows_in = x.contiguous(), scale = weight.contiguous();
    const Tensor skip = residual ? residual->contiguous() : Tensor();
    Normalised result{residual ? at::empty(x.sizes(), x.options()) : Tensor(), at::empty(x.sizes(), x.options())};
    if (x.numel() == 0)
        return result;
    camblas_cuda_context *context = fusion_context(x);
    succeed(camblas_cuda_add_rms_norm_rows(context, storage_code(x), storage_code(weight), int(rows),
                                           int(weight.size(0)), float(epsilon), round_before_weight ? 1 : 0,
                                           rows_in.const_data_ptr(), residual ? skip.const_data_ptr() : nullptr,
                                           scale.const_data_ptr(),
                                           residual ? result.added.mutable_data_ptr() : nullptr,
                                           result.output.mutable_data_ptr()),
            context);
    return result;
}

// down(silu(gate(x)) * up(x)), the activation written over the gate projection
Tensor gated_perceptron(const Tensor &x, const Tensor &gate_weight, const Tensor &up_weight,
                        const Tensor &down_weight, int algorithm)
{
    check_inference(x, x);
    for (const Tensor *weight : {&gate_weight, &up_weight, &down_weight}) {
        check_inference(*weight, x);
        require(weight->dim() == 2, "Invalid gated MLP dimensions");
    }
    const bool chained = x.dim() >= 1 && gate_weight.sizes().equals(up_weight.sizes()) &&
                         gate_weight.size(1) == x.size(-1) && down_weight.size(1) == gate_weight.size(0);
    require(chained, "Invalid gated MLP dimensions");
    Tensor activation = linear_public(x, gate_weight, std::nullopt, algorithm);
    const Tensor raised = linear_public(x, up_weight, std::nullopt, algorithm);
    c10::DeviceGuard guard(x.device());
    camblas_cuda_context *context = fusion_context(x, algorithm);
    succeed(camblas_cuda_silu_multiply(context, storage_code(x), uint64_t(activation.numel()),
                                       activation.const_data_ptr(), raised.const_data_ptr(),
                                       activation.mutable_data_ptr()),
            context);
    return linear_public(activation, down_weight, std::nullopt, algorithm);
}

// three independent bias-free projections of one input
std::tuple<Tensor, Tensor, Tensor> three_projections(const Tensor &x, const Tensor &q_weight, const Tensor &k_weight,
                                                     const Tensor &v_weight, int algorithm)
{
    check_inference(x, x);
    Tensor projected[3];
    const Tensor *weights[3] = {&q_weight, &k_weight, &v_weight};
    for (int index = 0; index < 3; ++index) {
        check_inference(*weights[index], x);
        projected[index] = linear_public(x, *weights[index], std::nullopt, algorithm);
    }
    return std::make_tuple(projected[0], projected[1], projected[2]);
}
} // namespace

void register_fusion(py::module_ &module)
{
    module.def("qkv_linear", &three_projections, py::arg("input"), py::arg("q_weight"), py::arg("k_weight"),
               py::arg("v_weight"), py::kw_only(), py::arg("algorithm") = -1,
               "Apply three bias-free linear projections for inference.");
    module.def("silu_multiply", &silu_times, py::arg("gate"), py::arg("up"),
               "Compute SiLU(gate)*up with storage rounding, for inference.");
    module.def("swiglu", &swiglu_rows, py::arg("gate"), py::arg("up"), py::kw_only(), py::arg("routing") = py::none(),
               py::arg("limit") = 0., "Compute SiLU(gate)*up in FP32 with one final storage rounding.");
    module.def(
        "rms_norm",
        [](const Tensor &x, const Tensor &weight, double epsilon, bool round_before_weight) {
            return normalise_rows(x, nullptr, weight, epsilon, round_before_weight).output;
        },
        py::arg("input"), py::arg("weight"), py::arg("epsilon") = 1e-6, py::kw_only(),
        py::arg("round_before_weight") = true, "Apply RMS normalisation in FP32.");
    module.def(
        "add_rms_norm",
        [](const Tensor &x, const Tensor &residual, const Tensor &weight, double epsilon) {
            Normalised result = normalise_rows(x, &residual, weight, epsilon, true);
            return std::make_tuple(result.added, result.output);
        },
        py::arg("x"), py::arg("residual"), py::arg("weight"), py::arg("epsilon") = 1e-6,
        "Return fresh residual sum and RMS-normalised output.");
    module.def("gated_mlp", &gated_perceptron, py::arg("input"), py::arg("gate_weight"), py::arg("up_weight"),
               py::arg("down_weight"), py::kw_only(), py::arg("algorithm") = -1,
               "Apply a bias-free SiLU gated MLP for inference.");
}
} // namespace binding
