// FP32 / FP64 dense helpers of the ATen binding: affine layer, two-layer perceptron with its backward
// pass, dense single-head attention, each with autograd where the reference offers it
// (ref for the semantics: src/cuda/torch_bindings.cpp:737-1002; the C entry points they call are
// declared in include/camblas_hip.h).
//
// Every function here follows one pattern: describe the operands as a list of (name, tensor,
// expected shape), let `Operands` check them and make them contiguous, then hand raw pointers to the C
// ABI. Shapes are written with named extents so that a mismatch is reported by name.
#include "binding.hpp"

#include <array>
#include <cmath>
#include <deque>
#include <map>
#include <string>

namespace py = pybind11;

namespace binding
{
namespace
{
// The dense operands of one call: FP32 or FP64, one GPU, one dtype. `add` checks an operand
// against a shape given as extent names; an extent is bound by its first use and must agree with
// every later one. Operands are kept contiguous for the lifetime of the call.
class Operands
{
  public:
    explicit Operands(const char *operation, const Tensor &anchor) : operation_(operation), anchor_(anchor) {}

    const Tensor &add(const char *name, const Tensor &tensor, std::initializer_list<const char *> shape)
    {
        check_tensor(tensor, anchor_, false);
        require(tensor.dim() == int64_t(shape.size()), mismatch(name));
        int64_t axis = 0;
        for (const char *extent : shape) {
            auto known = extents_.find(extent);
            if (known == extents_.end())
                extents_[extent] = tensor.size(axis);
            else
                require(known->second == tensor.size(axis), mismatch(name));
            ++axis;
        }
        kept_.push_back(tensor.contiguous());
        return kept_.back();
    }
    int extent(const char *name) const { return int(extents_.at(name)); }
    Tensor fresh(const std::vector<const char *> &shape) const
    {
        std::vector<int64_t> sizes;
        for (const char *name : shape)
            sizes.push_back(extents_.at(name));
        return at::empty(sizes, anchor_.options());
    }
    int wide() const { return anchor_.scalar_type() == at::kDouble ? 1 : 0; } // the ABI's dtype code
    camblas_cuda_context *context(int algorithm) const { return context_for(anchor_.get_device(), algorithm); }

  private:
    std::string mismatch(const char *name) const
    {
        return std::string("Invalid ") + operation_ + " operand shapes (" + name + ")";
    }
    const char *operation_;
    const Tensor &anchor_;
    std::map<std::string, int64_t> extents_;
    std::deque<Tensor> kept_; // (a deque: references handed out stay valid as operands are added)
};

bool any_recording(std::initializer_list<const Tensor *> tensors)
{
    for (const Tensor *tensor : tensors)
        if (recording(*tensor))
            return true;
    return false;
}

// ---------------------------------------------------------------------------- affine
// x W + bias with optional ReLU
Tensor affine(const Tensor &x, const Tensor &weight, const Tensor &bias, bool relu,
              const std::optional<Tensor> &output, int algorithm)
{
    Operands operands("affine", x);
    const Tensor &xc = operands.add("x", x, {"rows", "inner"});
    const Tensor &wc = operands.add("weight", weight, {"inner", "columns"});
    const Tensor &bc = operands.add("bias", bias, {"columns"});
    c10::DeviceGuard guard(x.device());
    Tensor result;
    if (output) {
        result = *output;
        check_tensor(result, x, false);
        require(!recording(result), "Autograd affine does not support an out tensor requiring gradients");
        require(result.dim() == 2 && result.size(0) == operands.extent("rows") &&
                    result.size(1) == operands.extent("columns") && result.is_contiguous(),
                "Invalid affine output shape or strides");
        require(!result.is_alias_of(x) && !result.is_alias_of(weight) && !result.is_alias_of(bias),
                "Affine output cannot alias an input");
    } else {
        result = operands.fresh({"rows", "columns"});
    }
    camblas_cuda_context *context = operands.context(algorithm);
    succeed(camblas_cuda_affine(context, operands.wide(), operands.extent("rows"), operands.extent("inner"),
                                operands.extent("columns"), xc.const_data_ptr(), wc.const_data_ptr(),
                                bc.const_data_ptr(), relu, result.mutable_data_ptr()),
            context);
    if (output && !result.is_inference())
        torch::autograd::impl::bump_version(result);
    return result;
}

// Gradients are products through matmul_public, so higher derivatives build a graph; with ReLU the
// incoming gradient is zeroed where the output is not positive.
struct AffineFunction : torch::autograd::Function<AffineFunction> {
    static Tensor forward(torch::autograd::AutogradContext *state, const Tensor &x, const Tensor &weight,
                          const Tensor &bias, bool relu, int64_t algorithm)
    {
        Tensor output = affine(x, weight, bias, relu, std::nullopt, int(algorithm));
        state->save_for_backward({x, weight, output});
        state->saved_data["relu"] = relu;
        state->saved_data["algorithm"] = algorithm;
        return output;
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *state,
                                                   torch::autograd::variable_list incoming)
    {
        const auto saved = state->get_saved_variables();
        const int algorithm = int(state->saved_data["algorithm"].toInt());
        Tensor gradient = incoming[0];
        if (state->saved_data["relu"].toBool())
            gradient = at::where(saved[2].le(0), 0, gradient);
        torch::autograd::variable_list result(5);
        if (state->needs_input_grad(0))
            result[0] = matmul_public(gradient, saved[1].t(), std::nullopt, 1, 0, algorithm);
        if (state->needs_input_grad(1))
            result[1] = matmul_public(saved[0].t(), gradient, std::nullopt, 1, 0, algorithm);
        if (state->needs_input_grad(2))
            result[2] = gradient.sum(at::IntArrayRef{0});
        return result;
    }
};

Tensor affine_public(const Tensor &x, const Tensor &weight, const Tensor &bias, bool relu, int algorithm)
{
    same_process();
    algorithm = resolve(algorithm);
    if (any_recording({&x, &weight, &bias}))
        return AffineFunction::apply(x, weight, bias, relu, int64_t(algorithm));
    return affine(x, weight, bias, relu, std::nullopt, algorithm);
}

// ---------------------------------------------------------------------------- two-layer perceptron
struct Perceptron {
    Tensor output, hidden;
};

// relu(x w1 + b1) w2 + b2 with the hidden activations kept for the backward pass
Perceptron mlp(const Tensor &x, const Tensor &w1, const Tensor &b1, const Tensor &w2, const Tensor &b2,
               int algorithm)
{
    Operands operands("MLP", x);
    const Tensor &xc = operands.add("x", x, {"rows", "inputs"});
    const Tensor &w1c = operands.add("w1", w1, {"inputs", "hidden"});
    const Tensor &b1c = operands.add("b1", b1, {"hidden"});
    const Tensor &w2c = operands.add("w2", w2, {"hidden", "outputs"});
    const Tensor &b2c = operands.add("b2", b2, {"outputs"});
    c10::DeviceGuard guard(x.device());
    Perceptron result{operands.fresh({"rows", "outputs"}), operands.fresh({"rows", "hidden"})};
    camblas_cuda_context *context = operands.context(algorithm);
    succeed(camblas_cuda_mlp(context, operands.wide(), operands.extent("rows"), operands.extent("inputs"),
                             operands.extent("hidden"), operands.extent("outputs"), xc.const_data_ptr(),
                             w1c.const_data_ptr(), b1c.const_data_ptr(), w2c.const_data_ptr(),
                             b2c.const_data_ptr(), result.hidden.mutable_data_ptr(),
                             result.output.mutable_data_ptr()),
            context);
    return result;
}

// Gradients in the order (x, w1, b1, w2, b2); entries that are not wanted stay undefined. The C
// entry point takes a null pointer for a gradient it should skip, and scratch for the hidden
// gradient whenever anything of the first layer is wanted.
std::array<Tensor, 5> mlp_backward(const Tensor &x, const Tensor &w1, const Tensor &w2, const Tensor &hidden,
                                   const Tensor &gradient, const std::array<bool, 5> &wanted, int algorithm)
{
    Operands operands("backward", x);
    const Tensor &xc = operands.add("x", x, {"rows", "inputs"});
    const Tensor &w1c = operands.add("w1", w1, {"inputs", "hidden"});
    const Tensor &w2c = operands.add("w2", w2, {"hidden", "outputs"});
    const Tensor &hc = operands.add("hidden", hidden, {"rows", "hidden"});
    const Tensor &gc = operands.add("gradient", gradient, {"rows", "outputs"});
    c10::DeviceGuard guard(x.device());
    static const std::vector<const char *> shapes[5] = {
        {"rows", "inputs"}, {"inputs", "hidden"}, {"hidden"}, {"hidden", "outputs"}, {"outputs"}};
    std::array<Tensor, 5> gradients;
    void *targets[5] = {};
    for (int index = 0; index < 5; ++index) {
        if (!wanted[index])
            continue;
        gradients[index] = operands.fresh(shapes[index]);
        targets[index] = gradients[index].mutable_data_ptr();
    }
    Tensor hidden_gradient;
    if (wanted[0] || wanted[1] || wanted[2])
        hidden_gradient = operands.fresh({"rows", "hidden"});
    camblas_cuda_context *context = operands.context(algorithm);
    succeed(camblas_cuda_mlp_backward(context, operands.wide(), operands.extent("rows"), operands.extent("inputs"),
                                      operands.extent("hidden"), operands.extent("outputs"),
                                      xc.const_data_ptr(), w1c.const_data_ptr(), w2c.const_data_ptr(),
                                      hc.const_data_ptr(), gc.const_data_ptr(),
                                      hidden_gradient.defined() ? hidden_gradient.mutable_data_ptr() : nullptr,
                                      targets[0], targets[1], targets[2], targets[3], targets[4]),
            context);
    return gradients;
}

py::tuple mlp_backward_public(const Tensor &x, const Tensor &w1, const Tensor &w2, const Tensor &hidden,
                              const Tensor &gradient, const std::array<bool, 5> &wanted, int algorithm)
{
    same_process();
    const auto gradients = mlp_backward(x, w1, w2, hidden, gradient, wanted, resolve(algorithm));
    py::tuple result(5);
    for (int index = 0; index < 5; ++index)
        result[index] = wanted[index] ? py::cast(gradients[index]) : py::none();
    return result;
}

// first derivatives only: the backward pass is one fused C call, not a graph of products
struct MlpFunction : torch::autograd::Function<MlpFunction> {
    static Tensor forward(torch::autograd::AutogradContext *state, const Tensor &x, const Tensor &w1,
                          const Tensor &b1, const Tensor &w2, const Tensor &b2, int64_t algorithm)
    {
        Perceptron result = mlp(x, w1, b1, w2, b2, int(algorithm));
        state->save_for_backward({x, w1, w2, result.hidden});
        state->saved_data["algorithm"] = algorithm;
        return result.output;
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *state,
                                                   torch::autograd::variable_list incoming)
    {
        TORCH_CHECK(!c10::GradMode::is_enabled(),
                    "MLP supports first derivatives; use two affine calls for higher derivatives");
        const auto saved = state->get_saved_variables();
        std::array<bool, 5> wanted;
        for (int index = 0; index < 5; ++index)
            wanted[index] = state->needs_input_grad(index);
        const auto gradients = mlp_backward(saved[0], saved[1], saved[2], saved[3], incoming[0], wanted,
                                            int(state->saved_data["algorithm"].toInt()));
        torch::autograd::variable_list result(gradients.begin(), gradients.end());
        result.emplace_back(); // the algorithm argument
        return result;
    }
};

Tensor mlp_public(const Tensor &x, const Tensor &w1, const Tensor &b1, const Tensor &w2, const Tensor &b2,
                  int algorithm)
{
    same_process();
    algorithm = resolve(algorithm);
    if (any_recording({&x, &w1, &b1, &w2, &b2}))
        return MlpFunction::apply(x, w1, b1, w2, b2, int64_t(algorithm));
    return mlp(x, w1, b1, w2, b2, algorithm).output;
}

// ---------------------------------------------------------------------------- dense attention
// softmax(scale q k^T) v, single head; under autograd it is composed from differentiable products
Tensor attention_public(const Tensor &q, const Tensor &k, const Tensor &v, const std::optional<double> &scale,
                        int algorithm)
{
    same_process();
    require(q.dim() == 2 && (scale || q.size(1) > 0),
            "Attention requires a rank-two query and positive depth for the default scale");
    const double factor = scale ? *scale : 1 / std::sqrt(double(q.size(1)));
    algorithm = resolve(algorithm);
    if (any_recording({&q, &k, &v})) {
        const Tensor scores = matmul_public(q, k.t(), std::nullopt, 1, 0, algorithm).mul(factor);
        return matmul_public(at::softmax(scores, -1, std::nullopt), v, std::nullopt, 1, 0, algorithm);
    }
    Operands operands("attention", q);
    const Tensor &qc = operands.add("q", q, {"queries", "depth"});
    const Tensor &kc = operands.add("k", k, {"keys", "depth"});
    const Tensor &vc = operands.add("v", v, {"keys", "values"});
    c10::DeviceGuard guard(q.device());
    Tensor output = operands.fresh({"queries", "values"});
    camblas_cuda_context *context = operands.context(algorithm);
    succeed(camblas_cuda_attention(context, operands.wide(), operands.extent("queries"), operands.extent("keys"),
                                   operands.extent("depth"), operands.extent("values"), factor,
                                   qc.const_data_ptr(), kc.const_data_ptr(), vc.const_data_ptr(),
                                   output.mutable_data_ptr()),
            context);
    return output;
}
} // namespace

void register_dense(py::module_ &module)
{
    module.def("affine", [](const Tensor &x, const Tensor &weight, const Tensor &bias, bool relu,
                            const std::optional<Tensor> &output, int algorithm) {
        return affine(x, weight, bias, relu, output, resolve(algorithm));
    });
    module.def("affine_public", &affine_public, py::arg("x"), py::arg("weight"), py::arg("bias"),
               py::kw_only(), py::arg("relu") = false, py::arg("algorithm") = -1);
    module.def("mlp_public", &mlp_public, py::arg("x"), py::arg("w1"), py::arg("b1"), py::arg("w2"),
               py::arg("b2"), py::kw_only(), py::arg("algorithm") = -1);
    module.def("mlp_backward", &mlp_backward_public, py::arg("x"), py::arg("w1"), py::arg("w2"),
               py::arg("hidden"), py::arg("gradient"), py::arg("needed"), py::arg("algorithm") = -1);
    module.def(
        "mlp",
        [](const Tensor &x, const Tensor &w1, const Tensor &b1, const Tensor &w2, const Tensor &b2,
           int algorithm) {
            same_process();
            Perceptron result = mlp(x, w1, b1, w2, b2, resolve(algorithm));
            return std::make_pair(result.output, result.hidden);
        },
        py::arg("x"), py::arg("w1"), py::arg("b1"), py::arg("w2"), py::arg("b2"), py::arg("algorithm") = -1);
    module.def(
        "attention",
        [](const Tensor &q, const Tensor &k, const Tensor &v, double scale, int algorithm) {
            c10::AutoGradMode inference(false);
            return attention_public(q, k, v, scale, algorithm);
        },
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("scale"), py::arg("algorithm") = -1);
    module.def("attention_public", &attention_public, py::arg("q"), py::arg("k"), py::arg("v"),
               py::kw_only(), py::arg("scale") = py::none(), py::arg("algorithm") = -1);
}
} // namespace binding
