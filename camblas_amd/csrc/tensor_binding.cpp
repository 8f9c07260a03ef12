// ATen binding for libcamblas_hip.so, built as _camblas_cuda_torch*.so beside the core library: the
// module name and function surface are the ones the reference's Python layer imports
// (ref: src/cuda/torch_bindings.cpp:1194-1294 for the exported names, camblas/_native.py:40-66 for
// how it is found). Row-major tensors are handed to the column-major C ABI as the swapped product
// (ref: src/cuda/torch_bindings.cpp:146-199), and `install_torch_backend` re-routes aten::mm,
// aten::mm.out and aten::addmm for the GPU dispatch key (ref: src/cuda/torch_backend.cuh:7-88).
//
// PyTorch is used for device memory, the current stream and dispatch only; every product runs in
// the library's own kernels. One library context exists per (thread, device, stream); a global
// table lets `stats_all` and `close` reach the contexts of every thread.
#include <torch/extension.h>
#include <torch/library.h>

#include <ATen/CUDAFunctions.h>
#include <ATen/Context.h>
#include <c10/core/DeviceGuard.h>
#include <c10/core/GradMode.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>

#include <hip/hip_runtime_api.h>
#include <unistd.h>

#include <array>
#include <cfloat>
#include <climits>
#include <cmath>
#include <map>
#include <memory>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "camblas_hip.h"

namespace py = pybind11;
using at::Tensor;

namespace
{
constexpr const char *COUNTER_NAMES[8] = {"classical", "strassen",       "gram",      "affine",
                                          "lt",        "guard_fallback", "attention", "backward"};
const pid_t creator_process = getpid();
thread_local int default_algorithm = CAMBLAS_CUDA_AUTO;

void require(bool condition, const char *message)
{
    if (!condition)
        throw std::invalid_argument(message);
}

void same_process()
{
    require(creator_process == getpid(), "GPU bindings cannot be reused after fork; use spawn");
}

void succeed(int status, camblas_cuda_context *context)
{
    if (status != 0)
        throw std::runtime_error(camblas_cuda_error(context));
}

// ---------------------------------------------------------------------------- contexts
struct Slot; // one library context owned by one thread

struct ContextTable {
    std::mutex mutex;
    std::unordered_map<camblas_cuda_context *, std::pair<int, Slot *>> live; // -> (device, owner)
};

ContextTable &table()
{
    // never destroyed: worker threads may release their slots after static destruction began
    static ContextTable *instance = new ContextTable;
    return *instance;
}

struct Slot {
    camblas_cuda_context *context = nullptr;

    Slot(int device, hipStream_t stream)
    {
        succeed(camblas_cuda_create(device, static_cast<void *>(stream), &context), nullptr);
        std::lock_guard<std::mutex> lock(table().mutex);
        table().live[context] = {device, this};
    }
    Slot(const Slot &) = delete;
    Slot &operator=(const Slot &) = delete;
    ~Slot()
    {
        if (creator_process != getpid())
            return;
        camblas_cuda_context *mine = nullptr;
        {
            // `close` may already have taken the context away from this slot
            std::lock_guard<std::mutex> lock(table().mutex);
            mine = context;
            if (mine)
                table().live.erase(mine);
            context = nullptr;
        }
        if (mine)
            camblas_cuda_destroy(mine);
    }
};

thread_local std::map<std::pair<int, hipStream_t>, std::unique_ptr<Slot>> thread_slots;

camblas_cuda_context *context_for(int device, int algorithm)
{
    same_process();
    hipStream_t stream = c10::hip::getCurrentHIPStream(c10::DeviceIndex(device)).stream();
    auto key = std::make_pair(device, stream);
    auto found = thread_slots.find(key);
    bool usable = false;
    if (found != thread_slots.end()) {
        std::lock_guard<std::mutex> lock(table().mutex);
        usable = found->second->context != nullptr;
    }
    if (!usable) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        hipError_t error = hipStreamIsCapturing(stream, &capture);
        require(error == hipSuccess && capture == hipStreamCaptureStatusNone,
                "Warm up CAMBLAS on this stream before graph capture");
        thread_slots[key] = std::make_unique<Slot>(device, stream);
        found = thread_slots.find(key);
    }
    camblas_cuda_context *context = found->second->context;
    succeed(camblas_cuda_set_algorithm(context, algorithm), context);
    return context;
}

void close_all()
{
    if (creator_process != getpid())
        return;
    std::vector<camblas_cuda_context *> pending;
    {
        std::lock_guard<std::mutex> lock(table().mutex);
        for (auto &entry : table().live) {
            pending.push_back(entry.first);
            entry.second.second->context = nullptr;
        }
        table().live.clear();
    }
    for (camblas_cuda_context *context : pending)
        camblas_cuda_destroy(context);
    thread_slots.clear();
}

py::dict counters_to_dict(const uint64_t (&counts)[8])
{
    py::dict result;
    for (int index = 0; index < 8; ++index)
        result[COUNTER_NAMES[index]] = counts[index];
    return result;
}

py::dict stats(int device, bool reset, int algorithm)
{
    same_process();
    c10::DeviceGuard guard(c10::Device(c10::kCUDA, c10::DeviceIndex(device)));
    camblas_cuda_context *context = context_for(device, algorithm);
    uint64_t counts[8];
    succeed(camblas_cuda_stats(context, counts, 8), context);
    if (reset)
        succeed(camblas_cuda_reset_stats(context), context);
    return counters_to_dict(counts);
}

py::dict stats_all(int device, bool reset)
{
    same_process();
    uint64_t totals[8] = {};
    std::lock_guard<std::mutex> lock(table().mutex);
    for (auto &entry : table().live) {
        if (entry.second.first != device)
            continue;
        uint64_t counts[8];
        succeed(camblas_cuda_stats(entry.first, counts, 8), entry.first);
        for (int index = 0; index < 8; ++index)
            totals[index] += counts[index];
        if (reset)
            succeed(camblas_cuda_reset_stats(entry.first), entry.first);
    }
    return counters_to_dict(totals);
}

// ---------------------------------------------------------------------------- operands
void check_tensor(const Tensor &tensor, const Tensor &like, bool allow_bf16)
{
    same_process();
    const auto type = tensor.scalar_type();
    require(tensor.is_cuda() && (type == at::kFloat || type == at::kDouble ||
                                 (allow_bf16 && type == at::kBFloat16)),
            allow_bf16 ? "CAMBLAS matmul requires GPU FP32, FP64 or BF16 tensors"
                       : "CAMBLAS requires GPU FP32 or FP64 tensors");
    require(tensor.device() == like.device() && type == like.scalar_type(),
            "All operands must have the same device and dtype");
    for (int64_t size : tensor.sizes())
        require(size <= INT_MAX, "LP64 dimension overflow");
    for (int64_t stride : tensor.strides())
        require(stride <= INT_MAX, "LP64 stride overflow");
}

void check_inference(const Tensor &tensor, const Tensor &like)
{
    check_tensor(tensor, like, true);
    require(tensor.scalar_type() != at::kDouble, "Native fusion requires FP32 or BF16 storage");
    require(!c10::GradMode::is_enabled() || !tensor.requires_grad(),
            "Native fusion supports inference only");
}

int storage_code(const Tensor &tensor) { return tensor.scalar_type() == at::kFloat ? 0 : 2; }

// A row-major [r, c] tensor is a column-major [c, r] matrix: unit stride along columns means the
// C ABI sees it untransposed with ld = row pitch, unit stride along rows means transposed with
// ld = column pitch, anything else is copied (ref: src/cuda/torch_bindings.cpp:146-154).
struct ColumnMajorView {
    Tensor keep;
    char transpose;
    int ld;
};

ColumnMajorView column_major(const Tensor &tensor)
{
    const int64_t rows = tensor.size(0), columns = tensor.size(1);
    if (tensor.stride(1) == 1 && tensor.stride(0) >= std::max<int64_t>(1, columns))
        return {tensor, 'N', int(tensor.stride(0))};
    if (tensor.stride(0) == 1 && tensor.stride(1) >= std::max<int64_t>(1, rows))
        return {tensor, 'T', int(tensor.stride(1))};
    return {tensor.contiguous(), 'N', int(std::max<int64_t>(1, columns))};
}

int64_t leading_rows(const Tensor &x)
{
    int64_t rows = 1;
    for (int64_t index = 0; index + 1 < x.dim(); ++index) {
        int64_t size = x.size(index);
        require(rows <= INT_MAX / std::max<int64_t>(1, size), "LP64 flattened row overflow");
        rows *= size;
    }
    return rows;
}

// ---------------------------------------------------------------------------- products
// C[m, n] = alpha * A[m, k] B[k, n] + beta * C, all row-major: the library computes the
// column-major product C^T = B^T A^T (ref: src/cuda/torch_bindings.cpp:156-199).
Tensor matmul(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output, double alpha,
              double beta, int algorithm, bool update_version = true)
{
    check_tensor(a, a, true);
    check_tensor(b, a, true);
    require(a.dim() == 2 && b.dim() == 2 && a.size(1) == b.size(0),
            "matmul requires compatible rank-two operands");
    c10::DeviceGuard guard(a.device());
    const int m = int(a.size(0)), k = int(a.size(1)), n = int(b.size(1));
    Tensor c;
    if (output) {
        c = *output;
        check_tensor(c, a, true);
        require(!c10::GradMode::is_enabled() || !c.requires_grad(),
                "Autograd matmul does not support an out tensor requiring gradients");
        require(c.dim() == 2 && c.size(0) == m && c.size(1) == n && c.is_contiguous(),
                "Output must have the product shape and contiguous row storage");
        require(!c.is_alias_of(a) && !c.is_alias_of(b), "GEMM output cannot alias an input");
    } else {
        require(beta == 0, "beta requires an existing output tensor");
        c = at::empty({m, n}, a.options());
    }
    ColumnMajorView left = column_major(b), right = column_major(a);
    camblas_cuda_context *context = context_for(a.get_device(), algorithm);
    const int ldc = std::max(1, n);
    int status;
    switch (a.scalar_type()) {
    case at::kFloat:
        status = camblas_cuda_sgemm(context, left.transpose, right.transpose, n, m, k, float(alpha),
                                    left.keep.const_data_ptr<float>(), left.ld,
                                    right.keep.const_data_ptr<float>(), right.ld, float(beta),
                                    c.mutable_data_ptr<float>(), ldc);
        break;
    case at::kDouble:
        status = camblas_cuda_dgemm(context, left.transpose, right.transpose, n, m, k, alpha,
                                    left.keep.const_data_ptr<double>(), left.ld,
                                    right.keep.const_data_ptr<double>(), right.ld, beta,
                                    c.mutable_data_ptr<double>(), ldc);
        break;
    default:
        status = camblas_cuda_bgemm(context, left.transpose, right.transpose, n, m, k, float(alpha),
                                    left.keep.const_data_ptr(), left.ld, right.keep.const_data_ptr(),
                                    right.ld, float(beta), c.mutable_data_ptr(), ldc);
    }
    succeed(status, context);
    if (output && update_version && !c.is_inference())
        torch::autograd::impl::bump_version(c);
    return c;
}

Tensor matmul_public(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output,
                     double alpha, double beta, int algorithm);

// d(AB)/dA = G B^T, d(AB)/dB = A^T G, both through the same entry so that higher derivatives
// build a graph (ref: src/cuda/torch_bindings.cpp:203-228).
struct MatmulFunction : torch::autograd::Function<MatmulFunction> {
    static Tensor forward(torch::autograd::AutogradContext *state, const Tensor &a, const Tensor &b,
                          int64_t algorithm)
    {
        state->save_for_backward({a, b});
        state->saved_data["algorithm"] = algorithm;
        return matmul(a, b, std::nullopt, 1, 0, int(algorithm));
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *state,
                                                   torch::autograd::variable_list gradients)
    {
        auto saved = state->get_saved_variables();
        const int algorithm = int(state->saved_data["algorithm"].toInt());
        Tensor grad_a, grad_b;
        if (state->needs_input_grad(0))
            grad_a = matmul_public(gradients[0], saved[1].t(), std::nullopt, 1, 0, algorithm);
        if (state->needs_input_grad(1))
            grad_b = matmul_public(saved[0].t(), gradients[0], std::nullopt, 1, 0, algorithm);
        return {grad_a, grad_b, Tensor()};
    }
};

Tensor matmul_public(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output,
                     double alpha, double beta, int algorithm)
{
    same_process();
    if (algorithm < 0)
        algorithm = default_algorithm;
    if (c10::GradMode::is_enabled() && (a.requires_grad() || b.requires_grad())) {
        require(!output && alpha == 1 && beta == 0,
                "Autograd matmul requires alpha=1, beta=0 and no out");
        return MatmulFunction::apply(a, b, int64_t(algorithm));
    }
    return matmul(a, b, output, alpha, beta, algorithm);
}

// ---------------------------------------------------------------------------- dense helpers
// x W + bias with optional ReLU, FP32 / FP64 (ref: src/cuda/torch_bindings.cpp:737-771).
Tensor affine(const Tensor &x, const Tensor &weight, const Tensor &bias, bool relu,
              const std::optional<Tensor> &output, int algorithm)
{
    check_tensor(x, x, false);
    check_tensor(weight, x, false);
    check_tensor(bias, x, false);
    require(x.dim() == 2 && weight.dim() == 2 && bias.dim() == 1 && x.size(1) == weight.size(0) &&
                weight.size(1) == bias.size(0),
            "Invalid affine operand shapes");
    c10::DeviceGuard guard(x.device());
    const int rows = int(x.size(0)), inner = int(x.size(1)), columns = int(weight.size(1));
    Tensor c;
    if (output) {
        c = *output;
        check_tensor(c, x, false);
        require(!c10::GradMode::is_enabled() || !c.requires_grad(),
                "Autograd affine does not support an out tensor requiring gradients");
        require(c.dim() == 2 && c.size(0) == rows && c.size(1) == columns && c.is_contiguous(),
                "Invalid affine output shape or strides");
        require(!c.is_alias_of(x) && !c.is_alias_of(weight) && !c.is_alias_of(bias),
                "Affine output cannot alias an input");
    } else {
        c = at::empty({rows, columns}, x.options());
    }
    Tensor xc = x.contiguous(), wc = weight.contiguous(), bc = bias.contiguous();
    camblas_cuda_context *context = context_for(x.get_device(), algorithm);
    succeed(camblas_cuda_affine(context, x.scalar_type() == at::kDouble, rows, inner, columns,
                                xc.const_data_ptr(), wc.const_data_ptr(), bc.const_data_ptr(), relu,
                                c.mutable_data_ptr()),
            context);
    if (output && !c.is_inference())
        torch::autograd::impl::bump_version(c);
    return c;
}

// Gradients as products through matmul_public, so higher derivatives build a graph; with ReLU
// the incoming gradient is zeroed where the output is not positive
// (ref: src/cuda/torch_bindings.cpp:773-801).
struct AffineFunction : torch::autograd::Function<AffineFunction> {
    static Tensor forward(torch::autograd::AutogradContext *state, const Tensor &x,
                          const Tensor &weight, const Tensor &bias, bool relu, int64_t algorithm)
    {
        Tensor output = affine(x, weight, bias, relu, std::nullopt, int(algorithm));
        state->save_for_backward({x, weight, output});
        state->saved_data["relu"] = relu;
        state->saved_data["algorithm"] = algorithm;
        return output;
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *state,
                                                   torch::autograd::variable_list gradients)
    {
        auto saved = state->get_saved_variables();
        const int algorithm = int(state->saved_data["algorithm"].toInt());
        Tensor gradient = gradients[0], dx, dw, db;
        if (state->saved_data["relu"].toBool())
            gradient = at::where(saved[2].le(0), 0, gradient);
        if (state->needs_input_grad(0))
            dx = matmul_public(gradient, saved[1].t(), std::nullopt, 1, 0, algorithm);
        if (state->needs_input_grad(1))
            dw = matmul_public(saved[0].t(), gradient, std::nullopt, 1, 0, algorithm);
        if (state->needs_input_grad(2))
            db = gradient.sum(at::IntArrayRef{0});
        return {dx, dw, db, Tensor(), Tensor()};
    }
};

Tensor affine_public(const Tensor &x, const Tensor &weight, const Tensor &bias, bool relu,
                     int algorithm)
{
    same_process();
    if (algorithm < 0)
        algorithm = default_algorithm;
    if (c10::GradMode::is_enabled() &&
        (x.requires_grad() || weight.requires_grad() || bias.requires_grad()))
        return AffineFunction::apply(x, weight, bias, relu, int64_t(algorithm));
    return affine(x, weight, bias, relu, std::nullopt, algorithm);
}

// relu(x w1 + b1) w2 + b2; returns (output, hidden activations)
// (ref: src/cuda/torch_bindings.cpp:815-841).
std::pair<Tensor, Tensor> mlp(const Tensor &x, const Tensor &w1, const Tensor &b1, const Tensor &w2,
                              const Tensor &b2, int algorithm)
{
    for (const Tensor *tensor : {&x, &w1, &b1, &w2, &b2})
        check_tensor(*tensor, x, false);
    require(x.dim() == 2 && w1.dim() == 2 && w2.dim() == 2 && b1.dim() == 1 && b2.dim() == 1 &&
                x.size(1) == w1.size(0) && w1.size(1) == w2.size(0) && b1.size(0) == w1.size(1) &&
                b2.size(0) == w2.size(1),
            "Invalid MLP operand shapes");
    c10::DeviceGuard guard(x.device());
    const int rows = int(x.size(0)), inputs = int(x.size(1));
    const int hidden = int(w1.size(1)), outputs = int(w2.size(1));
    Tensor h = at::empty({rows, hidden}, x.options()), c = at::empty({rows, outputs}, x.options());
    Tensor xc = x.contiguous(), w1c = w1.contiguous(), b1c = b1.contiguous();
    Tensor w2c = w2.contiguous(), b2c = b2.contiguous();
    camblas_cuda_context *context = context_for(x.get_device(), algorithm);
    succeed(camblas_cuda_mlp(context, x.scalar_type() == at::kDouble, rows, inputs, hidden, outputs,
                             xc.const_data_ptr(), w1c.const_data_ptr(), b1c.const_data_ptr(),
                             w2c.const_data_ptr(), b2c.const_data_ptr(), h.mutable_data_ptr(),
                             c.mutable_data_ptr()),
            context);
    return {c, h};
}

// (dx, dw1, db1, dw2, db2); entries not needed stay undefined
// (ref: src/cuda/torch_bindings.cpp:925-966).
std::array<Tensor, 5> mlp_backward_tensors(const Tensor &x, const Tensor &w1, const Tensor &w2,
                                           const Tensor &h, const Tensor &gradient,
                                           const std::array<bool, 5> &needed, int algorithm)
{
    for (const Tensor *tensor : {&x, &w1, &w2, &h, &gradient})
        check_tensor(*tensor, x, false);
    require(x.dim() == 2 && w1.dim() == 2 && w2.dim() == 2 && h.dim() == 2 && gradient.dim() == 2 &&
                x.size(1) == w1.size(0) && w1.size(1) == w2.size(0) && h.size(0) == x.size(0) &&
                h.size(1) == w1.size(1) && gradient.size(0) == x.size(0) &&
                gradient.size(1) == w2.size(1),
            "Invalid backward operand shapes");
    c10::DeviceGuard guard(x.device());
    const int rows = int(x.size(0)), inputs = int(x.size(1));
    const int hidden = int(w1.size(1)), outputs = int(w2.size(1));
    Tensor xc = x.contiguous(), w1c = w1.contiguous(), w2c = w2.contiguous();
    Tensor hc = h.contiguous(), gc = gradient.contiguous();
    Tensor dh, dx, dw1, db1, dw2, db2;
    if (needed[0] || needed[1] || needed[2])
        dh = at::empty({rows, hidden}, x.options());
    if (needed[0])
        dx = at::empty({rows, inputs}, x.options());
    if (needed[1])
        dw1 = at::empty({inputs, hidden}, x.options());
    if (needed[2])
        db1 = at::empty({hidden}, x.options());
    if (needed[3])
        dw2 = at::empty({hidden, outputs}, x.options());
    if (needed[4])
        db2 = at::empty({outputs}, x.options());
    auto pointer = [](Tensor &tensor) { return tensor.defined() ? tensor.mutable_data_ptr() : nullptr; };
    camblas_cuda_context *context = context_for(x.get_device(), algorithm);
    succeed(camblas_cuda_mlp_backward(context, x.scalar_type() == at::kDouble, rows, inputs, hidden,
                                      outputs, xc.const_data_ptr(), w1c.const_data_ptr(),
                                      w2c.const_data_ptr(), hc.const_data_ptr(), gc.const_data_ptr(),
                                      pointer(dh), pointer(dx), pointer(dw1), pointer(db1),
                                      pointer(dw2), pointer(db2)),
            context);
    return {dx, dw1, db1, dw2, db2};
}

py::tuple mlp_backward_public(const Tensor &x, const Tensor &w1, const Tensor &w2, const Tensor &h,
                              const Tensor &gradient, const std::array<bool, 5> &needed,
                              int algorithm)
{
    same_process();
    auto gradients = mlp_backward_tensors(x, w1, w2, h, gradient, needed,
                                          algorithm < 0 ? default_algorithm : algorithm);
    py::tuple result(5);
    for (int i = 0; i < 5; ++i)
        result[i] = needed[i] ? py::cast(gradients[i]) : py::none();
    return result;
}

// First derivatives only (ref: src/cuda/torch_bindings.cpp:978-1002).
struct MlpFunction : torch::autograd::Function<MlpFunction> {
    static Tensor forward(torch::autograd::AutogradContext *state, const Tensor &x, const Tensor &w1,
                          const Tensor &b1, const Tensor &w2, const Tensor &b2, int64_t algorithm)
    {
        auto output = mlp(x, w1, b1, w2, b2, int(algorithm));
        state->save_for_backward({x, w1, w2, output.second});
        state->saved_data["algorithm"] = algorithm;
        return output.first;
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *state,
                                                   torch::autograd::variable_list gradients)
    {
        TORCH_CHECK(!c10::GradMode::is_enabled(),
                    "MLP supports first derivatives; use two affine calls for higher derivatives");
        auto saved = state->get_saved_variables();
        const int algorithm = int(state->saved_data["algorithm"].toInt());
        std::array<bool, 5> needed;
        for (int i = 0; i < 5; ++i)
            needed[i] = state->needs_input_grad(i);
        auto result =
            mlp_backward_tensors(saved[0], saved[1], saved[2], saved[3], gradients[0], needed, algorithm);
        return {result[0], result[1], result[2], result[3], result[4], Tensor()};
    }
};

Tensor mlp_public(const Tensor &x, const Tensor &w1, const Tensor &b1, const Tensor &w2,
                  const Tensor &b2, int algorithm)
{
    same_process();
    if (algorithm < 0)
        algorithm = default_algorithm;
    if (c10::GradMode::is_enabled() && (x.requires_grad() || w1.requires_grad() || b1.requires_grad() ||
                                        w2.requires_grad() || b2.requires_grad()))
        return MlpFunction::apply(x, w1, b1, w2, b2, int64_t(algorithm));
    return mlp(x, w1, b1, w2, b2, algorithm).first;
}

// softmax(scale q k^T) v, dense and single-head; with gradients enabled it is composed from
// differentiable products (ref: src/cuda/torch_bindings.cpp:880-923).
Tensor attention_public(const Tensor &q, const Tensor &k, const Tensor &v,
                        const std::optional<double> &scale, int algorithm)
{
    same_process();
    require(q.dim() == 2 && (scale || q.size(1) > 0),
            "Attention requires a rank-two query and positive depth for the default scale");
    const double value = scale ? *scale : 1 / std::sqrt(double(q.size(1)));
    if (algorithm < 0)
        algorithm = default_algorithm;
    if (c10::GradMode::is_enabled() && (q.requires_grad() || k.requires_grad() || v.requires_grad())) {
        Tensor scores = matmul_public(q, k.t(), std::nullopt, 1, 0, algorithm).mul(value);
        return matmul_public(at::softmax(scores, -1, std::nullopt), v, std::nullopt, 1, 0, algorithm);
    }
    check_tensor(q, q, false);
    check_tensor(k, q, false);
    check_tensor(v, q, false);
    require(k.dim() == 2 && v.dim() == 2 && q.size(1) == k.size(1) && k.size(0) == v.size(0),
            "Invalid attention operand shapes");
    c10::DeviceGuard guard(q.device());
    const int queries = int(q.size(0)), keys = int(k.size(0)), depth = int(q.size(1)),
              values = int(v.size(1));
    Tensor qc = q.contiguous(), kc = k.contiguous(), vc = v.contiguous();
    Tensor output = at::empty({queries, values}, q.options());
    camblas_cuda_context *context = context_for(q.get_device(), algorithm);
    succeed(camblas_cuda_attention(context, q.scalar_type() == at::kDouble, queries, keys, depth, values,
                                   value, qc.const_data_ptr(), kc.const_data_ptr(), vc.const_data_ptr(),
                                   output.mutable_data_ptr()),
            context);
    return output;
}

// y = x W^T (+ bias) for W [outputs, inputs]; leading dimensions of x are flattened
// (ref: src/cuda/torch_bindings.cpp:244-271).
Tensor linear_public(const Tensor &x, const Tensor &weight, const std::optional<Tensor> &bias,
                     int algorithm)
{
    check_tensor(x, x, true);
    check_tensor(weight, x, true);
    require(x.dim() >= 1 && weight.dim() == 2 && x.size(-1) == weight.size(1),
            "linear requires matching input and [outputs, inputs] weight dimensions");
    const int64_t rows = leading_rows(x);
    if (bias) {
        check_tensor(*bias, x, true);
        require(bias->dim() == 1 && bias->size(0) == weight.size(0),
                "linear bias must have the output width");
    }
    Tensor result = matmul_public(x.reshape({rows, x.size(-1)}), weight.t(), std::nullopt, 1., 0.,
                                  algorithm);
    if (bias)
        result = result.add(*bias);
    auto shape = x.sizes().vec();
    shape.back() = weight.size(0);
    return result.reshape(shape);
}

std::tuple<Tensor, Tensor, Tensor> qkv_linear_public(const Tensor &x, const Tensor &q_weight,
                                                     const Tensor &k_weight, const Tensor &v_weight,
                                                     int algorithm)
{
    check_inference(x, x);
    for (const Tensor *weight : {&q_weight, &k_weight, &v_weight})
        check_inference(*weight, x);
    return std::make_tuple(linear_public(x, q_weight, std::nullopt, algorithm),
                           linear_public(x, k_weight, std::nullopt, algorithm),
                           linear_public(x, v_weight, std::nullopt, algorithm));
}

// ---------------------------------------------------------------------------- epilogues
Tensor silu_multiply_public(const Tensor &gate, const Tensor &up)
{
    check_inference(gate, gate);
    check_inference(up, gate);
    require(gate.sizes() == up.sizes(), "SiLU operands must have matching shapes");
    c10::DeviceGuard guard(gate.device());
    Tensor g = gate.contiguous(), u = up.contiguous();
    Tensor result = at::empty(gate.sizes(), gate.options());
    camblas_cuda_context *context = context_for(gate.get_device(), default_algorithm);
    succeed(camblas_cuda_silu_multiply(context, storage_code(gate), uint64_t(gate.numel()),
                                       g.const_data_ptr(), u.const_data_ptr(),
                                       result.mutable_data_ptr()),
            context);
    return result;
}

Tensor swiglu_public(const Tensor &gate, const Tensor &up, const std::optional<Tensor> &routing,
                     double limit)
{
    check_inference(gate, gate);
    check_inference(up, gate);
    require(gate.dim() >= 1 && gate.sizes() == up.sizes() && gate.size(-1) > 0 &&
                gate.size(-1) <= INT_MAX && std::isfinite(limit) && limit >= 0 && limit <= FLT_MAX,
            "Invalid SwiGLU shapes or clipping limit");
    c10::DeviceGuard guard(gate.device());
    Tensor g = gate.contiguous(), u = up.contiguous(), r;
    if (routing) {
        check_inference(*routing, *routing);
        require(routing->device() == gate.device() && routing->scalar_type() == at::kFloat,
                "SwiGLU routing values must be FP32 on the input device");
        auto rows = gate.sizes().vec();
        rows.pop_back();
        auto column = rows;
        column.push_back(1);
        require(routing->sizes().vec() == rows || routing->sizes().vec() == column,
                "SwiGLU routing requires one value per input row");
        r = routing->contiguous();
    }
    Tensor result = at::empty(gate.sizes(), gate.options());
    camblas_cuda_context *context = context_for(gate.get_device(), default_algorithm);
    succeed(camblas_cuda_swiglu(context, storage_code(gate), uint64_t(gate.numel()),
                                int(gate.size(-1)), float(limit), g.const_data_ptr(),
                                u.const_data_ptr(), routing ? r.const_data_ptr<float>() : nullptr,
                                result.mutable_data_ptr()),
            context);
    return result;
}

// Row-wise RMS normalisation, optionally after a residual add, in one launch for any number of
// rows. Arithmetic: ref src/cuda/inference_fusion.cuh:136-191 (round the normalised value to the
// storage type before the weight unless round_before_weight is false). The reference composes
// the multi-row case from a square kernel, ATen's mean and a scale kernel
// (src/cuda/torch_bindings.cpp:602-673); the mean here is the library's own fixed-order sum.
std::tuple<Tensor, Tensor> normalise_rows(const Tensor &x, const std::optional<Tensor> &residual,
                                          const Tensor &weight, double epsilon,
                                          bool round_before_weight)
{
    check_inference(x, x);
    if (round_before_weight) {
        check_inference(weight, x);
    } else {
        check_inference(weight, weight);
        require(weight.device() == x.device() &&
                    (weight.scalar_type() == x.scalar_type() ||
                     (x.scalar_type() == at::kBFloat16 && weight.scalar_type() == at::kFloat)),
                "Final-round RMS weight must match input dtype or use FP32 with BF16 input");
    }
    require(x.dim() >= 1 && weight.dim() == 1 && x.size(-1) == weight.size(0),
            "RMS norm weight must match the input's last dimension");
    require(std::isfinite(epsilon) && epsilon >= 0 && epsilon <= FLT_MAX,
            "RMS norm epsilon must be finite and nonnegative");
    if (residual) {
        check_inference(*residual, x);
        require(residual->sizes() == x.sizes(), "Residual RMS dimensions must match");
    }
    const int64_t rows = leading_rows(x);
    c10::DeviceGuard guard(x.device());
    Tensor xc = x.contiguous(), wc = weight.contiguous(), rc, added;
    Tensor output = at::empty(x.sizes(), x.options());
    if (residual) {
        rc = residual->contiguous();
        added = at::empty(x.sizes(), x.options());
    }
    if (x.numel() == 0)
        return std::make_tuple(added, output);
    camblas_cuda_context *context = context_for(x.get_device(), default_algorithm);
    succeed(camblas_cuda_add_rms_norm_rows(
                context, storage_code(x), storage_code(weight), int(rows), int(weight.size(0)),
                float(epsilon), round_before_weight ? 1 : 0, xc.const_data_ptr(),
                residual ? rc.const_data_ptr() : nullptr, wc.const_data_ptr(),
                residual ? added.mutable_data_ptr() : nullptr, output.mutable_data_ptr()),
            context);
    return std::make_tuple(added, output);
}

Tensor rms_norm_public(const Tensor &x, const Tensor &weight, double epsilon,
                       bool round_before_weight)
{
    return std::get<1>(normalise_rows(x, std::nullopt, weight, epsilon, round_before_weight));
}

std::tuple<Tensor, Tensor> add_rms_norm_public(const Tensor &x, const Tensor &residual,
                                               const Tensor &weight, double epsilon)
{
    return normalise_rows(x, residual, weight, epsilon, true);
}

// down(silu(gate(x)) * up(x)) with the SiLU product written over the gate activation
// (ref: src/cuda/torch_bindings.cpp:703-723).
Tensor gated_mlp_public(const Tensor &x, const Tensor &gate_weight, const Tensor &up_weight,
                        const Tensor &down_weight, int algorithm)
{
    check_inference(x, x);
    for (const Tensor *weight : {&gate_weight, &up_weight, &down_weight})
        check_inference(*weight, x);
    require(x.dim() >= 1 && gate_weight.dim() == 2 && up_weight.dim() == 2 &&
                down_weight.dim() == 2 && gate_weight.sizes() == up_weight.sizes() &&
                x.size(-1) == gate_weight.size(1) && down_weight.size(1) == gate_weight.size(0),
            "Invalid gated MLP dimensions");
    Tensor gate = linear_public(x, gate_weight, std::nullopt, algorithm);
    Tensor up = linear_public(x, up_weight, std::nullopt, algorithm);
    c10::DeviceGuard guard(x.device());
    camblas_cuda_context *context =
        context_for(x.get_device(), algorithm < 0 ? default_algorithm : algorithm);
    succeed(camblas_cuda_silu_multiply(context, storage_code(x), uint64_t(gate.numel()),
                                       gate.const_data_ptr(), up.const_data_ptr(),
                                       gate.mutable_data_ptr()),
            context);
    return linear_public(gate, down_weight, std::nullopt, algorithm);
}

// FP8 E4M3fn block-scaled linear (1x128 activation groups, 128x128 weight blocks), any row count.
Tensor fp8_block_matmul_public(const Tensor &a, const Tensor &a_scale, const Tensor &weight,
                               const Tensor &weight_scale)
{
    same_process();
    require(a.is_cuda() && weight.is_cuda() && a_scale.is_cuda() && weight_scale.is_cuda() &&
                a.device() == weight.device() && a_scale.device() == a.device() &&
                weight_scale.device() == a.device(),
            "FP8 operands must live on one GPU");
    require(a.scalar_type() == at::kFloat8_e4m3fn && weight.scalar_type() == at::kFloat8_e4m3fn &&
                a_scale.scalar_type() == at::kFloat && weight_scale.scalar_type() == at::kFloat,
            "FP8 block matmul takes E4M3fn values and FP32 scales");
    require(a.dim() == 2 && weight.dim() == 2 && a.size(1) == weight.size(1) && a.size(1) > 0 &&
                a.size(1) % 128 == 0 && a.size(0) <= 65535 && weight.size(0) <= INT_MAX &&
                a.size(1) <= INT_MAX,
            "FP8 block matmul needs [rows, inner] x [outputs, inner] with inner a multiple of 128");
    const int64_t rows = a.size(0), outputs = weight.size(0), groups = a.size(1) / 128;
    require(a_scale.dim() == 2 && a_scale.size(0) == rows && a_scale.size(1) == groups &&
                weight_scale.dim() == 2 && weight_scale.size(0) == (outputs + 127) / 128 &&
                weight_scale.size(1) == groups,
            "FP8 scale shapes must be [rows, inner/128] and [ceil(outputs/128), inner/128]");
    require(!c10::GradMode::is_enabled() || !(a_scale.requires_grad() || weight_scale.requires_grad()),
            "FP8 block matmul supports inference only");
    c10::DeviceGuard guard(a.device());
    Tensor ac = a.contiguous(), wc = weight.contiguous(), as = a_scale.contiguous(),
           ws = weight_scale.contiguous();
    Tensor result = at::empty({rows, outputs}, a.options().dtype(at::kBFloat16));
    if (rows == 0 || outputs == 0)
        return result;
    camblas_cuda_context *context = context_for(a.get_device(), default_algorithm);
    succeed(camblas_cuda_fp8_block_matmul(context, int(rows), int(outputs), int(a.size(1)),
                                          ac.const_data_ptr(), as.const_data_ptr<float>(),
                                          wc.const_data_ptr(), ws.const_data_ptr<float>(),
                                          result.mutable_data_ptr()),
            context);
    return result;
}

// Single-token FP8 product with 32-wide FP32 scale blocks; without input scales the BF16 token is
// quantised on the fly (ref: src/cuda/torch_bindings.cpp:380-458).
bool fp8_decode_supported_public(int device)
{
    same_process();
    if (device < 0)
        device = int(c10::hip::current_device());
    c10::DeviceGuard guard(c10::Device(c10::kCUDA, c10::DeviceIndex(device)));
    return camblas_cuda_fp8_decode_supported(context_for(device, default_algorithm)) != 0;
}

Tensor fp8_block32_product(const Tensor &x, const std::optional<Tensor> &x_scale,
                           const Tensor &weight, const Tensor &weight_scale)
{
    same_process();
    const bool quantise = !x_scale.has_value();
    require(x.is_cuda() && x.scalar_type() == (quantise ? at::kBFloat16 : at::kFloat8_e4m3fn) &&
                weight.scalar_type() == at::kFloat8_e4m3fn,
            "FP8 linear requires GPU BF16/FP8 input and E4M3 weight");
    require(x.dim() >= 1 && weight.dim() == 2 && weight_scale.dim() == 2 && x.is_contiguous() &&
                weight.is_contiguous(),
            "FP8 linear requires contiguous matrices and rank-two weight scales");
    require(weight_scale.scalar_type() == at::kFloat, "FP8 weight scales must be FP32");
    for (const Tensor *tensor : {&x, &weight, &weight_scale}) {
        require(tensor->device() == x.device() &&
                    (!c10::GradMode::is_enabled() || !tensor->requires_grad()),
                "FP8 operands must share a GPU and support inference only");
        for (int64_t size : tensor->sizes())
            require(size <= INT_MAX, "LP64 dimension overflow");
    }
    const int64_t inner = x.size(-1), outputs = weight.size(0);
    require(inner >= 32 && inner <= 8192 && inner % 32 == 0 && outputs >= 16 && outputs % 16 == 0 &&
                x.numel() == inner && weight.size(1) == inner,
            "Invalid FP8 linear matrix dimensions");
    require(weight_scale.size(0) == (outputs + 31) / 32 && weight_scale.size(1) == inner / 32,
            "FP8 weight scale shape does not match its blocks");
    int64_t sx = 1;
    const int64_t sn = weight_scale.stride(0), sk = weight_scale.stride(1);
    if (!quantise) {
        require(x_scale->device() == x.device() && x_scale->scalar_type() == at::kFloat &&
                    x_scale->dim() == x.dim() &&
                    (!c10::GradMode::is_enabled() || !x_scale->requires_grad()),
                "FP8 input scales require matching device/rank and FP32 inference storage");
        for (int64_t index = 0; index + 1 < x.dim(); ++index)
            require(x_scale->size(index) == x.size(index), "FP8 input scale shape mismatch");
        require(x_scale->size(-1) == inner / 32, "FP8 input scale shape mismatch");
        sx = x_scale->stride(-1);
    }
    require(sx > 0 && sx <= INT_MAX && sn > 0 && sn <= INT_MAX && sk > 0 && sk <= INT_MAX,
            "FP8 scale strides must be positive LP64 values");
    c10::DeviceGuard guard(x.device());
    camblas_cuda_context *context = context_for(x.get_device(), default_algorithm);
    auto shape = x.sizes().vec();
    shape.back() = outputs;
    Tensor result = at::empty(shape, x.options().dtype(at::kBFloat16));
    const int status =
        quantise ? camblas_cuda_fp8_linear(context, int(outputs), int(inner), x.const_data_ptr(),
                                           weight.const_data_ptr(),
                                           weight_scale.const_data_ptr<float>(), int(sn), int(sk),
                                           nullptr, 0, result.mutable_data_ptr())
                 : camblas_cuda_fp8_decode(context, int(outputs), int(inner), x.const_data_ptr(),
                                           x_scale->const_data_ptr<float>(), weight.const_data_ptr(),
                                           weight_scale.const_data_ptr<float>(), int(sx), int(sn),
                                           int(sk), nullptr, 0, result.mutable_data_ptr());
    succeed(status, context);
    return result;
}

// E8M0 block-scaled products and mixture-of-experts routing
// (ref: src/cuda/torch_bindings.cpp:328-378, :462-600).
void check_quantized_operand(const Tensor &tensor, const Tensor &like)
{
    require(tensor.device() == like.device() && tensor.is_contiguous(),
            "Quantized operands must be contiguous and on the same GPU");
    require(!c10::GradMode::is_enabled() || !tensor.requires_grad(),
            "Quantized multiplication supports inference only");
    for (int64_t size : tensor.sizes())
        require(size <= INT_MAX, "LP64 dimension overflow");
}

Tensor quantized_matmul_public(const Tensor &x, const Tensor &x_scale, const Tensor &weight,
                               const Tensor &weight_scale, int activation_block)
{
    same_process();
    require(x.is_cuda() && x.scalar_type() == at::kFloat8_e4m3fn, "Quantized input must be GPU FP8 E4M3");
    const bool packed = weight.scalar_type() == at::ScalarType::Float4_e2m1fn_x2;
    require(packed || weight.scalar_type() == at::kFloat8_e4m3fn,
            "Quantized weight must be FP8 E4M3 or packed FP4 E2M1");
    require(x_scale.scalar_type() == at::ScalarType::Float8_e8m0fnu &&
                weight_scale.scalar_type() == at::ScalarType::Float8_e8m0fnu,
            "Quantized scales must be E8M0");
    for (const Tensor *tensor : {&x, &x_scale, &weight, &weight_scale})
        check_quantized_operand(*tensor, x);
    require(x.dim() >= 1 && weight.dim() == 2 && x_scale.dim() == x.dim() && weight_scale.dim() == 2,
            "Quantized matrix and scale ranks do not match");
    const int64_t inner = x.size(-1), outputs = weight.size(0);
    int64_t rows = 1;
    require(inner >= 32 && inner % 32 == 0 && outputs >= 8 && outputs % 8 == 0 &&
                weight.size(1) == inner / (packed ? 2 : 1) &&
                (activation_block == 32 || (packed && activation_block == 128)) &&
                inner % activation_block == 0,
            "Invalid quantized matrix dimensions or activation block");
    for (int64_t index = 0; index + 1 < x.dim(); ++index) {
        require(x_scale.size(index) == x.size(index), "Input scale shape mismatch");
        require(rows <= 65535 / std::max<int64_t>(1, x.size(index)),
                "Quantized multiplication supports at most 65535 rows");
        rows *= x.size(index);
    }
    require(x_scale.size(-1) == inner / activation_block &&
                weight_scale.size(0) == (packed ? outputs : (outputs + 31) / 32) &&
                weight_scale.size(1) == inner / 32,
            "Quantized scale shapes do not match their blocks");
    c10::DeviceGuard guard(x.device());
    auto shape = x.sizes().vec();
    shape.back() = outputs;
    Tensor result = at::empty(shape, x.options().dtype(at::kBFloat16));
    camblas_cuda_context *context = context_for(x.get_device(), default_algorithm);
    succeed(camblas_cuda_quantized_matmul(context, packed, int(rows), int(outputs), int(inner),
                                          activation_block, x.const_data_ptr(),
                                          x_scale.const_data_ptr(), weight.const_data_ptr(),
                                          weight_scale.const_data_ptr(), result.mutable_data_ptr()),
            context);
    return result;
}

// Keeps the weight and scale tensors of every expert alive and their addresses in a device table;
// in-place updates of the values are seen by later calls, a relocated storage is refused.
struct QuantizedGroups {
    std::vector<Tensor> weights, scales;
    Tensor table; // int64 [groups, 2] on the device
    int outputs = 0, inner = 0;
    bool packed = false, trainable = false;

    QuantizedGroups(const std::vector<Tensor> &group_weights, const std::vector<Tensor> &group_scales)
    {
        same_process();
        require(!group_weights.empty() && group_weights.size() <= 65535 &&
                    group_weights.size() == group_scales.size(),
                "Supply matching non-empty weight and scale groups");
        const Tensor &first = group_weights[0];
        require(first.is_cuda() && first.dim() == 2, "Grouped weights must be GPU matrices");
        packed = first.scalar_type() == at::ScalarType::Float4_e2m1fn_x2;
        require(packed || first.scalar_type() == at::kFloat8_e4m3fn,
                "Grouped weights require FP8 or packed FP4 storage");
        require(first.size(0) >= 8 && first.size(0) <= INT_MAX && first.size(0) % 8 == 0 &&
                    first.size(1) >= (packed ? 16 : 32) && first.size(1) <= INT_MAX / (packed ? 2 : 1),
                "Invalid grouped weight dimensions");
        outputs = int(first.size(0));
        inner = int(first.size(1)) * (packed ? 2 : 1);
        require(inner % 32 == 0, "Grouped inner dimension must be a multiple of 32");
        Tensor host = at::empty({int64_t(group_weights.size()), 2},
                                at::TensorOptions().device(at::kCPU).dtype(at::kLong));
        int64_t *addresses = host.mutable_data_ptr<int64_t>();
        for (size_t index = 0; index < group_weights.size(); ++index) {
            const Tensor &w = group_weights[index], &s = group_scales[index];
            require(w.device() == first.device() && w.scalar_type() == first.scalar_type() &&
                        w.sizes() == first.sizes() && w.is_contiguous() &&
                        uintptr_t(w.const_data_ptr()) % 16 == 0 && s.device() == first.device() &&
                        s.scalar_type() == at::ScalarType::Float8_e8m0fnu && s.dim() == 2 &&
                        s.size(0) == (packed ? outputs : (outputs + 31LL) / 32) &&
                        s.size(1) == inner / 32 && s.is_contiguous(),
                    "Grouped weight shapes, dtypes, devices or scales differ");
            trainable |= w.requires_grad() || s.requires_grad();
            weights.push_back(w.detach());
            scales.push_back(s.detach());
            addresses[2 * index] = int64_t(uintptr_t(w.const_data_ptr()));
            addresses[2 * index + 1] = int64_t(uintptr_t(s.const_data_ptr()));
        }
        c10::DeviceGuard guard(first.device());
        table = host.to(first.device());
        host_table = host;
    }

    Tensor matmul(const Tensor &x, const Tensor &x_scale, const Tensor &active, const Tensor &counts,
                  int activation_block)
    {
        same_process();
        require(!c10::GradMode::is_enabled() || (!trainable && !x.requires_grad()),
                "Grouped multiplication supports inference only");
        require(x.device() == table.device() && x.scalar_type() == at::kFloat8_e4m3fn &&
                    x.dim() == 3 && x.size(0) <= 65535 && x.size(1) <= 65535 && x.size(2) == inner &&
                    (activation_block == 32 || (packed && activation_block == 128)) &&
                    inner % activation_block == 0,
                "Invalid grouped input dimensions or activation block");
        require(x_scale.device() == x.device() &&
                    x_scale.scalar_type() == at::ScalarType::Float8_e8m0fnu && x_scale.dim() == 3 &&
                    x_scale.size(0) == x.size(0) && x_scale.size(1) == x.size(1) &&
                    x_scale.size(2) == inner / activation_block,
                "Grouped input scale shape or dtype mismatch");
        for (const Tensor *index : {&active, &counts})
            require(index->device() == x.device() && index->scalar_type() == at::kInt &&
                        index->dim() == 1 && index->numel() == x.size(0),
                    "Grouped indices/counts require one GPU int32 value per group");
        for (const Tensor *value : {&x, &x_scale, &active, &counts})
            require(value->is_contiguous(), "Grouped operands must be contiguous");
        const int64_t *addresses = host_table.const_data_ptr<int64_t>();
        for (size_t index = 0; index < weights.size(); ++index)
            require(int64_t(uintptr_t(weights[index].const_data_ptr())) == addresses[2 * index] &&
                        int64_t(uintptr_t(scales[index].const_data_ptr())) == addresses[2 * index + 1],
                    "Captured weight storage changed; recreate the group");
        c10::DeviceGuard guard(x.device());
        Tensor result = at::empty({x.size(0), x.size(1), outputs}, x.options().dtype(at::kBFloat16));
        camblas_cuda_context *context = context_for(x.get_device(), default_algorithm);
        succeed(camblas_cuda_grouped_quantized_matmul(
                    context, packed, int(x.size(0)), int(weights.size()), int(x.size(1)), outputs,
                    inner, activation_block, x.const_data_ptr(), x_scale.const_data_ptr(),
                    table.const_data_ptr(), active.const_data_ptr(), counts.const_data_ptr(),
                    result.mutable_data_ptr()),
                context);
        return result;
    }

  private:
    Tensor host_table;
};

std::tuple<Tensor, Tensor, Tensor> route_groups_public(const Tensor &experts, const Tensor &active,
                                                       int first_expert, int rows)
{
    same_process();
    require(experts.is_cuda() && experts.scalar_type() == at::kLong && experts.dim() == 2 &&
                experts.is_contiguous() && experts.size(0) <= INT_MAX && experts.size(1) >= 1 &&
                experts.size(1) <= 64 && experts.numel() <= INT_MAX &&
                active.device() == experts.device() && active.scalar_type() == at::kInt &&
                active.dim() == 1 && active.is_contiguous() && active.numel() >= 1 &&
                active.numel() <= 65535 && rows >= 1 && rows <= 65535 &&
                active.numel() * rows <= INT_MAX && first_expert >= 0,
            "Invalid expert routing dimensions, indices or devices");
    c10::DeviceGuard guard(experts.device());
    Tensor counts = at::empty({active.numel()}, active.options());
    Tensor slots = at::empty({active.numel(), rows}, active.options());
    Tensor reverse = at::empty(experts.sizes(), active.options());
    camblas_cuda_context *context = context_for(experts.get_device(), default_algorithm);
    succeed(camblas_cuda_route_groups(context, int(experts.size(0)), int(experts.size(1)),
                                      first_expert, int(active.numel()), rows,
                                      experts.const_data_ptr(), active.const_data_ptr(),
                                      counts.mutable_data_ptr(), slots.mutable_data_ptr(),
                                      reverse.mutable_data_ptr()),
            context);
    return std::make_tuple(slots, reverse, counts);
}

Tensor reduce_groups_public(const Tensor &input, const Tensor &experts, const Tensor &reverse)
{
    same_process();
    require(input.is_cuda() && input.scalar_type() == at::kBFloat16 && input.dim() == 3 &&
                input.is_contiguous() && input.size(0) * input.size(1) <= INT_MAX &&
                input.size(2) >= 1 && input.size(2) <= INT_MAX &&
                experts.device() == input.device() && experts.scalar_type() == at::kLong &&
                experts.dim() == 2 && experts.is_contiguous() && experts.size(0) <= INT_MAX &&
                experts.size(1) >= 1 && experts.size(1) <= 64 && experts.numel() <= INT_MAX &&
                reverse.device() == input.device() && reverse.scalar_type() == at::kInt &&
                reverse.sizes() == experts.sizes() && reverse.is_contiguous() &&
                (!c10::GradMode::is_enabled() || !input.requires_grad()),
            "Invalid grouped reduction shapes, types, devices or gradients");
    c10::DeviceGuard guard(input.device());
    Tensor result = at::empty({experts.size(0), input.size(2)}, input.options().dtype(at::kFloat));
    camblas_cuda_context *context = context_for(input.get_device(), default_algorithm);
    succeed(camblas_cuda_reduce_groups(context, int(experts.size(0)), int(experts.size(1)),
                                       int(input.size(2)), int(input.size(0) * input.size(1)),
                                       experts.const_data_ptr(), reverse.const_data_ptr(),
                                       input.const_data_ptr(), result.mutable_data_ptr()),
            context);
    return result;
}

// ---------------------------------------------------------------------------- ATen backend
// Re-route aten::mm / mm.out / addmm on the GPU dispatch key. Anything the library does not take
// goes to ATen's own GPU implementation through the at::cuda:: entry points, which bypass the
// dispatcher and therefore cannot recurse into these functions
// (ref: src/cuda/torch_backend.cuh:1-88).
std::unique_ptr<torch::Library> backend_registration;
int backend_algorithm = CAMBLAS_CUDA_LT;

bool product_supported(const Tensor &a, const Tensor &b)
{
    if (!a.is_cuda() || !b.is_cuda() || a.layout() != at::kStrided || b.layout() != at::kStrided ||
        a.dim() != 2 || b.dim() != 2 || a.device() != b.device() ||
        a.scalar_type() != b.scalar_type() || a.size(1) != b.size(0) || a.is_conj() ||
        b.is_conj() || a.is_neg() || b.is_neg())
        return false;
    const auto type = a.scalar_type();
    if (type != at::kFloat && type != at::kDouble && type != at::kBFloat16)
        return false;
    // a caller that allowed reduced-precision FP32 products keeps ATen's behaviour
    if (type == at::kFloat && at::globalContext().allowTF32CuBLAS())
        return false;
    for (const Tensor *tensor : {&a, &b}) {
        for (int64_t size : tensor->sizes())
            if (size == 0 || size > INT_MAX)
                return false;
        for (int64_t stride : tensor->strides())
            if (stride < 0 || stride > INT_MAX)
                return false;
    }
    return true;
}

bool bias_supported(const Tensor &bias, const Tensor &a, const Tensor &b)
{
    if (bias.device() != a.device() || bias.scalar_type() != a.scalar_type() ||
        bias.layout() != at::kStrided || bias.dim() > 2 || bias.is_conj() || bias.is_neg())
        return false;
    if (bias.dim() >= 1 && bias.size(-1) != 1 && bias.size(-1) != b.size(1))
        return false;
    return bias.dim() < 2 || bias.size(0) == 1 || bias.size(0) == a.size(0);
}

Tensor backend_mm(const Tensor &a, const Tensor &b)
{
    if (!product_supported(a, b))
        return at::cuda::mm(a, b);
    return matmul(a, b, std::nullopt, 1., 0., backend_algorithm, false);
}

Tensor &backend_mm_out(const Tensor &a, const Tensor &b, Tensor &out)
{
    if (!product_supported(a, b) || out.device() != a.device() ||
        out.scalar_type() != a.scalar_type() || out.layout() != at::kStrided || out.dim() != 2 ||
        out.size(0) != a.size(0) || out.size(1) != b.size(1) || !out.is_contiguous() ||
        out.is_conj() || out.is_neg() || out.is_alias_of(a) || out.is_alias_of(b))
        return at::cuda::mm_out(out, a, b);
    matmul(a, b, out, 1., 0., backend_algorithm, false); // the dispatcher bumps the version
    return out;
}

Tensor backend_addmm(const Tensor &bias, const Tensor &a, const Tensor &b, const at::Scalar &beta,
                     const at::Scalar &alpha)
{
    if (!product_supported(a, b) || !bias_supported(bias, a, b) || beta.isComplex() ||
        alpha.isComplex())
        return at::cuda::addmm(bias, a, b, beta, alpha);
    c10::DeviceGuard guard(a.device());
    const double beta_value = beta.toDouble();
    Tensor out = beta_value == 0
                     ? at::empty({a.size(0), b.size(1)}, a.options())
                     : bias.expand({a.size(0), b.size(1)}).clone(at::MemoryFormat::Contiguous);
    return matmul(a, b, out, alpha.toDouble(), beta_value, backend_algorithm, false);
}

void install_torch_backend(int algorithm)
{
    static std::mutex install_mutex;
    std::lock_guard<std::mutex> lock(install_mutex);
    if (backend_registration)
        return;
    TORCH_CHECK(algorithm >= CAMBLAS_CUDA_AUTO && algorithm <= CAMBLAS_CUDA_STRASSEN_FOUR,
                "Invalid CAMBLAS algorithm");
    backend_algorithm = algorithm;
    auto library = std::make_unique<torch::Library>(torch::Library::IMPL, "aten",
                                                    c10::DispatchKey::CUDA, __FILE__, __LINE__);
    library->impl("mm", TORCH_FN(backend_mm));
    library->impl("mm.out", TORCH_FN(backend_mm_out));
    library->impl("addmm", TORCH_FN(backend_addmm));
    backend_registration = std::move(library);
}
} // namespace

PYBIND11_MODULE(_camblas_cuda_torch, module)
{
    module.def("install_torch_backend", &install_torch_backend);
    module.def("set_default_algorithm", [](int algorithm) { default_algorithm = algorithm; });
    module.def("matmul",
               [](const Tensor &a, const Tensor &b, const std::optional<Tensor> &out, double alpha,
                  double beta, int algorithm) { return matmul(a, b, out, alpha, beta, algorithm); });
    module.def("matmul_public", &matmul_public, py::arg("a"), py::arg("b"), py::kw_only(),
               py::arg("out") = py::none(), py::arg("alpha") = 1., py::arg("beta") = 0.,
               py::arg("algorithm") = -1,
               "Multiply two GPU matrices (FP32, FP64 or BF16) with transpose views and autograd.");
    module.def("affine", [](const Tensor &x, const Tensor &weight, const Tensor &bias, bool relu,
                            const std::optional<Tensor> &output, int algorithm) {
        return affine(x, weight, bias, relu, output, algorithm < 0 ? default_algorithm : algorithm);
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
            return mlp(x, w1, b1, w2, b2, algorithm < 0 ? default_algorithm : algorithm);
        },
        py::arg("x"), py::arg("w1"), py::arg("b1"), py::arg("w2"), py::arg("b2"),
        py::arg("algorithm") = -1);
    module.def(
        "attention",
        [](const Tensor &q, const Tensor &k, const Tensor &v, double scale, int algorithm) {
            c10::AutoGradMode inference(false);
            return attention_public(q, k, v, scale, algorithm);
        },
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("scale"), py::arg("algorithm") = -1);
    module.def("attention_public", &attention_public, py::arg("q"), py::arg("k"), py::arg("v"),
               py::kw_only(), py::arg("scale") = py::none(), py::arg("algorithm") = -1);
    module.def("linear_public", &linear_public, py::arg("input"), py::arg("weight"),
               py::arg("bias") = py::none(), py::kw_only(), py::arg("algorithm") = -1,
               "Apply a linear transform with [outputs, inputs] weights and autograd.");
    module.def("qkv_linear", &qkv_linear_public, py::arg("input"), py::arg("q_weight"),
               py::arg("k_weight"), py::arg("v_weight"), py::kw_only(), py::arg("algorithm") = -1,
               "Apply three bias-free linear projections for inference.");
    module.def("silu_multiply", &silu_multiply_public, py::arg("gate"), py::arg("up"),
               "Compute SiLU(gate)*up with storage rounding, for inference.");
    module.def("swiglu", &swiglu_public, py::arg("gate"), py::arg("up"), py::kw_only(),
               py::arg("routing") = py::none(), py::arg("limit") = 0.,
               "Compute SiLU(gate)*up in FP32 with one final storage rounding.");
    module.def("rms_norm", &rms_norm_public, py::arg("input"), py::arg("weight"),
               py::arg("epsilon") = 1e-6, py::kw_only(), py::arg("round_before_weight") = true,
               "Apply RMS normalisation in FP32.");
    module.def("add_rms_norm", &add_rms_norm_public, py::arg("x"), py::arg("residual"),
               py::arg("weight"), py::arg("epsilon") = 1e-6,
               "Return fresh residual sum and RMS-normalised output.");
    module.def("gated_mlp", &gated_mlp_public, py::arg("input"), py::arg("gate_weight"),
               py::arg("up_weight"), py::arg("down_weight"), py::kw_only(),
               py::arg("algorithm") = -1, "Apply a bias-free SiLU gated MLP for inference.");
    module.def("fp8_block_matmul", &fp8_block_matmul_public, py::arg("input"),
               py::arg("input_scale"), py::arg("weight"), py::arg("weight_scale"),
               "Multiply E4M3fn activations (1x128 FP32 scales) by E4M3fn weights (128x128 FP32 "
               "scales), returning BF16.");
    module.attr("quantized_tile_rows") = 16;
    py::class_<QuantizedGroups>(module, "QuantizedGroups",
                                "Capture GPU quantized weight storages and retain their lifetimes. "
                                "In-place value updates are visible; recreate the group after "
                                "storage relocation.")
        .def(py::init<const std::vector<Tensor> &, const std::vector<Tensor> &>(), py::arg("weights"),
             py::arg("scales"))
        .def("matmul", &QuantizedGroups::matmul, py::arg("input"), py::arg("input_scale"),
             py::arg("active"), py::arg("counts"), py::kw_only(), py::arg("activation_block") = 32,
             "Multiply [groups,rows,inner] FP8 input with selected captured weights. Invalid "
             "active indices and padding return zero; counts clip to [0,rows]. Inference only.");
    module.def("route_groups", &route_groups_public, py::arg("experts"), py::arg("active"),
               py::kw_only(), py::arg("first_expert") = 0, py::arg("rows"),
               "Return slots, reverse mapping and counts for expert/choice IDs. Excess rows are "
               "discarded and unassigned slots are -1; execution uses the active stream.");
    module.def("reduce_groups", &reduce_groups_public, py::arg("input"), py::arg("experts"),
               py::arg("reverse"),
               "Sum BF16 contributions into FP32 in expert/choice order. Invalid IDs/rows are "
               "ignored; requires inference and contiguous GPU tensors.");
    module.def("quantized_matmul", &quantized_matmul_public, py::arg("input"), py::arg("input_scale"),
               py::arg("weight"), py::arg("weight_scale"), py::kw_only(),
               py::arg("activation_block") = 32,
               "Multiply block-scaled FP8 input by FP8 or packed FP4 weights, returning BF16. "
               "Requires contiguous GPU operands and E8M0 scales.");
    module.def("fp8_decode_supported", &fp8_decode_supported_public, py::arg("device") = -1,
               "Return whether this build and device support the block-32 FP8 decode product.");
    module.def(
        "fp8_decode",
        [](const Tensor &x, const Tensor &x_scale, const Tensor &weight, const Tensor &weight_scale) {
            return fp8_block32_product(x, x_scale, weight, weight_scale);
        },
        py::arg("input"), py::arg("input_scale"), py::arg("weight"), py::arg("weight_scale"),
        "Multiply one block32 E4M3 token by E4M3 weights, using FP32 scales and ordered FP32 "
        "accumulation; positive scale strides are allowed.");
    module.def(
        "fp8_linear",
        [](const Tensor &x, const Tensor &weight, const Tensor &weight_scale) {
            return fp8_block32_product(x, std::nullopt, weight, weight_scale);
        },
        py::arg("input"), py::arg("weight"), py::arg("weight_scale"),
        "Quantise one finite BF16 token to block32 E4M3 with power-of-two FP32 scales and "
        "multiply E4M3 weights with ordered FP32 accumulation.");
    module.def("stats", &stats);
    module.def("stats_all", &stats_all);
    module.def("close", &close_all);
}
