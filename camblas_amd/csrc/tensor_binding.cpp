// ATen binding for libcamblas_hip.so, built as _camblas_cuda_torch*.so beside the core library: the
// module name and function surface are the ones the reference's Python layer imports
// (ref: src/cuda/torch_bindings.cpp:1194-1294 for the exported names, camblas/_native.py:40-66 for
// how it is found). Row-major tensors are handed to the column-major C ABI as the swapped product
// (ref: src/cuda/torch_bindings.cpp:146-199), and `install_torch_backend` re-routes aten::mm,
// aten::mm.out and aten::addmm for the GPU dispatch key (ref: src/cuda/torch_backend.cuh:7-88).
//
// This unit holds the contexts, the tensor checks, the GEMM-shaped entry points and the module
// definition; binding_dense.cpp, binding_fusion.cpp and binding_quantized.cpp hold the rest.
// PyTorch is used for device memory, the current stream and dispatch only; every product runs in
// the library's own kernels. One library context exists per (thread, device, stream); a global
// table lets `stats_all` and `close` reach the contexts of every thread.
#include "binding.hpp"

#include <torch/library.h>

#include <ATen/CUDAFunctions.h>
#include <ATen/Context.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>

#include <hip/hip_runtime_api.h>
#include <unistd.h>

#include <map>
#include <memory>
#include <mutex>
#include <unordered_map>

namespace py = pybind11;

namespace binding
{
namespace
{
constexpr const char *COUNTER_NAMES[8] = {"classical", "strassen",       "gram",      "affine",
                                          "lt",        "guard_fallback", "attention", "backward"};
const pid_t creator_process = getpid();
thread_local int default_algorithm = CAMBLAS_CUDA_AUTO;
} // namespace

void same_process()
{
    require(creator_process == getpid(), "GPU bindings cannot be reused after fork; use spawn");
}

void succeed(int status, camblas_cuda_context *context)
{
    if (status != 0)
        throw std::runtime_error(camblas_cuda_error(context));
}

int current_default_algorithm() { return default_algorithm; }

namespace
{
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

} // namespace

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

namespace
{
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

} // namespace

// ---------------------------------------------------------------------------- operands
void admit(const char *role, const Tensor &tensor, const at::Device &device, const Want &want)
{
    const std::string who(role);
    require(tensor.device() == device, who + " must live on the GPU of the call");
    bool typed = false;
    for (at::ScalarType accepted : want.dtypes)
        typed = typed || tensor.scalar_type() == accepted;
    require(typed, who + " has an unsupported dtype");
    require(want.rank < 0 ? tensor.dim() >= 1 : tensor.dim() == want.rank, who + " has the wrong rank");
    require(!want.dense || tensor.is_contiguous(), who + " must be contiguous");
    for (int64_t size : tensor.sizes())
        require(size <= INT_MAX, who + ": LP64 dimension overflow");
    require(!recording(tensor), who + " requires gradients; this operation supports inference only");
}

int64_t flattened_rows(const Tensor &tensor, int64_t limit, const char *what)
{
    int64_t rows = 1;
    for (int64_t index = 0; index + 1 < tensor.dim(); ++index) {
        const int64_t size = tensor.size(index);
        require(size == 0 || rows <= limit / size, what);
        rows *= size;
    }
    return rows;
}

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
    require(!recording(tensor), "Native fusion supports inference only");
}

namespace
{
// How the column-major C ABI sees a row-major [r, c] tensor: as the [c, r] matrix stored with unit
// stride along c ('N', leading dimension = row pitch), or, when the tensor is itself a transposed
// view (unit stride along r), as that matrix transposed ('T', leading dimension = column pitch).
// Any other striding is copied first (ref for the rule: src/cuda/torch_bindings.cpp:146-154).
struct AbiOperand {
    Tensor storage; // keeps a copy alive when one had to be made
    char flag;
    int leading;

    explicit AbiOperand(const Tensor &matrix)
    {
        const int64_t rows = matrix.size(0), columns = matrix.size(1);
        const bool row_pitched = matrix.stride(1) == 1 && matrix.stride(0) >= std::max<int64_t>(columns, 1);
        const bool column_pitched = matrix.stride(0) == 1 && matrix.stride(1) >= std::max<int64_t>(rows, 1);
        storage = row_pitched || column_pitched ? matrix : matrix.contiguous();
        flag = !row_pitched && column_pitched ? 'T' : 'N';
        leading = int(flag == 'T' ? storage.stride(1) : std::max<int64_t>(storage.stride(0), 1));
    }
    const void *data() const { return storage.const_data_ptr(); }
};
} // namespace

// ---------------------------------------------------------------------------- products
// out[m, n] = alpha * a[m, k] b[k, n] + beta * out, all row-major. Seen column-major the same
// memory is out^T = b^T a^T, so `b` travels as the ABI's first operand and `a` as its second
// (ref: src/cuda/torch_bindings.cpp:156-199).
Tensor matmul(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output, double alpha,
              double beta, int algorithm, bool update_version)
{
    check_tensor(a, a, true);
    check_tensor(b, a, true);
    require(a.dim() == 2 && b.dim() == 2 && b.size(0) == a.size(1), "matmul requires compatible rank-two operands");
    c10::DeviceGuard guard(a.device());
    const int rows = int(a.size(0)), inner = int(a.size(1)), columns = int(b.size(1));
    Tensor result;
    if (!output) {
        require(beta == 0, "beta requires an existing output tensor");
        result = at::empty({rows, columns}, a.options());
    } else {
        result = *output;
        check_tensor(result, a, true);
        require(!recording(result), "Autograd matmul does not support an out tensor requiring gradients");
        const bool fits = result.dim() == 2 && result.size(0) == rows && result.size(1) == columns;
        require(fits && result.is_contiguous(), "Output must have the product shape and contiguous row storage");
        require(!result.is_alias_of(a) && !result.is_alias_of(b), "GEMM output cannot alias an input");
    }
    const AbiOperand first(b), second(a);
    camblas_cuda_context *context = context_for(a.get_device(), algorithm);
    const int pitch = std::max(columns, 1);
    int status = 0;
    if (a.scalar_type() == at::kBFloat16)
        status = camblas_cuda_bgemm(context, first.flag, second.flag, columns, rows, inner, float(alpha),
                                    first.data(), first.leading, second.data(), second.leading, float(beta),
                                    result.mutable_data_ptr(), pitch);
    else if (a.scalar_type() == at::kDouble)
        status = camblas_cuda_dgemm(context, first.flag, second.flag, columns, rows, inner, alpha,
                                    static_cast<const double *>(first.data()), first.leading,
                                    static_cast<const double *>(second.data()), second.leading, beta,
                                    result.mutable_data_ptr<double>(), pitch);
    else
        status = camblas_cuda_sgemm(context, first.flag, second.flag, columns, rows, inner, float(alpha),
                                    static_cast<const float *>(first.data()), first.leading,
                                    static_cast<const float *>(second.data()), second.leading, float(beta),
                                    result.mutable_data_ptr<float>(), pitch);
    succeed(status, context);
    if (output && update_version && !result.is_inference())
        torch::autograd::impl::bump_version(result);
    return result;
}

namespace
{
// d(ab)/da = g b^T and d(ab)/db = a^T g, themselves products through matmul_public so that higher
// derivatives build a graph
struct ProductFunction : torch::autograd::Function<ProductFunction> {
    static Tensor forward(torch::autograd::AutogradContext *state, const Tensor &a, const Tensor &b,
                          int64_t algorithm)
    {
        state->saved_data["algorithm"] = algorithm;
        state->save_for_backward({a, b});
        return matmul(a, b, std::nullopt, 1, 0, int(algorithm));
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *state,
                                                   torch::autograd::variable_list incoming)
    {
        const auto operands = state->get_saved_variables();
        const int algorithm = int(state->saved_data["algorithm"].toInt());
        torch::autograd::variable_list gradients(3);
        if (state->needs_input_grad(0))
            gradients[0] = matmul_public(incoming[0], operands[1].t(), std::nullopt, 1, 0, algorithm);
        if (state->needs_input_grad(1))
            gradients[1] = matmul_public(operands[0].t(), incoming[0], std::nullopt, 1, 0, algorithm);
        return gradients;
    }
};
} // namespace

Tensor matmul_public(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output, double alpha,
                     double beta, int algorithm)
{
    same_process();
    algorithm = resolve(algorithm);
    if (!recording(a) && !recording(b))
        return matmul(a, b, output, alpha, beta, algorithm);
    require(alpha == 1 && beta == 0 && !output, "Autograd matmul requires alpha=1, beta=0 and no out");
    return ProductFunction::apply(a, b, int64_t(algorithm));
}

// y = x W^T (+ bias) for W [outputs, inputs]; the leading dimensions of x are flattened into rows
Tensor linear_public(const Tensor &x, const Tensor &weight, const std::optional<Tensor> &bias, int algorithm)
{
    check_tensor(x, x, true);
    check_tensor(weight, x, true);
    const bool chained = x.dim() >= 1 && weight.dim() == 2 && weight.size(1) == x.size(-1);
    require(chained, "linear requires matching input and [outputs, inputs] weight dimensions");
    const int64_t outputs = weight.size(0);
    if (bias) {
        check_tensor(*bias, x, true);
        require(bias->dim() == 1 && bias->size(0) == outputs, "linear bias must have the output width");
    }
    const int64_t rows = flattened_rows(x, INT_MAX, "LP64 flattened row overflow");
    Tensor product = matmul_public(x.reshape({rows, x.size(-1)}), weight.t(), std::nullopt, 1., 0., algorithm);
    if (bias)
        product = product.add(*bias);
    std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
    shape.back() = outputs;
    return product.reshape(shape);
}

namespace
{
// ---------------------------------------------------------------------------- ATen backend
// aten::mm / mm.out / addmm on the GPU dispatch key run here once installed. A call the library
// does not take goes to ATen's own GPU implementation through the at::cuda:: entry points, which
// bypass the dispatcher and so cannot come back here (ref for which calls are taken:
// src/cuda/torch_backend.cuh:7-71).
std::unique_ptr<torch::Library> backend_registration;
int backend_algorithm = CAMBLAS_CUDA_LT;

// an ordinary strided matrix view: no lazy conjugation or negation, 32-bit extents and strides
bool plain(const Tensor &tensor)
{
    if (tensor.layout() != at::kStrided || tensor.is_conj() || tensor.is_neg())
        return false;
    for (int64_t stride : tensor.strides())
        if (stride < 0 || stride > INT_MAX)
            return false;
    for (int64_t size : tensor.sizes())
        if (size > INT_MAX)
            return false;
    return true;
}

bool takes_product(const Tensor &a, const Tensor &b)
{
    if (!(a.is_cuda() && b.is_cuda() && plain(a) && plain(b) && a.dim() == 2 && b.dim() == 2))
        return false;
    if (a.device() != b.device() || a.scalar_type() != b.scalar_type() || a.size(1) != b.size(0))
        return false;
    // empty products stay with ATen (ref: torch_backend.cuh:20-22)
    if (a.numel() == 0 || b.numel() == 0)
        return false;
    switch (a.scalar_type()) {
    case at::kFloat: // a caller that allowed reduced-precision FP32 products keeps ATen's behaviour
        return !at::globalContext().allowTF32CuBLAS();
    case at::kDouble:
    case at::kBFloat16:
        return true;
    default:
        return false;
    }
}

// a bias that broadcasts against the [rows, columns] product: scalar-like, a row, a column or full
bool takes_bias(const Tensor &bias, int64_t rows, int64_t columns, const Tensor &like)
{
    if (!plain(bias) || bias.device() != like.device() || bias.scalar_type() != like.scalar_type() ||
        bias.dim() > 2)
        return false;
    const bool last_fits = bias.dim() == 0 || bias.size(-1) == 1 || bias.size(-1) == columns;
    const bool first_fits = bias.dim() < 2 || bias.size(0) == 1 || bias.size(0) == rows;
    return last_fits && first_fits;
}

bool takes_output(const Tensor &out, const Tensor &a, const Tensor &b)
{
    return plain(out) && out.device() == a.device() && out.scalar_type() == a.scalar_type() && out.dim() == 2 &&
           out.size(0) == a.size(0) && out.size(1) == b.size(1) && out.is_contiguous() && !out.is_alias_of(a) &&
           !out.is_alias_of(b);
}

Tensor backend_mm(const Tensor &a, const Tensor &b)
{
    return takes_product(a, b) ? matmul(a, b, std::nullopt, 1., 0., backend_algorithm, false) : at::cuda::mm(a, b);
}

Tensor &backend_mm_out(const Tensor &a, const Tensor &b, Tensor &out)
{
    if (!takes_product(a, b) || !takes_output(out, a, b))
        return at::cuda::mm_out(out, a, b);
    matmul(a, b, out, 1., 0., backend_algorithm, false); // the dispatcher bumps the version itself
    return out;
}

// A BF16 bias the product's epilogue can read where it lies: one row for every output row ([n] or
// [1, n]) or a full [rows, n] matrix, with unit stride along n. `pitch` is the row stride in
// elements, 0 for the repeated row.
struct Addend {
    const void *data = nullptr;
    int pitch = 0;
};

Addend epilogue_addend(const Tensor &bias, int64_t rows, int64_t columns)
{
    if (bias.scalar_type() != at::kBFloat16 || bias.dim() < 1 || bias.size(-1) != columns ||
        (columns > 1 && bias.stride(-1) != 1))
        return {};
    if (bias.dim() == 1 || bias.size(0) == 1)
        return {bias.const_data_ptr(), 0};
    if (rows > 1 && bias.stride(0) < columns)
        return {};
    return {bias.const_data_ptr(), rows > 1 ? int(bias.stride(0)) : 0};
}

// out = alpha * a b + beta * addend into a fresh tensor, the addend read by the product itself
Tensor bf16_product_adding(const Addend &addend, const Tensor &a, const Tensor &b, double alpha, double beta)
{
    const int rows = int(a.size(0)), inner = int(a.size(1)), columns = int(b.size(1));
    Tensor result = at::empty({rows, columns}, a.options());
    const AbiOperand first(b), second(a);
    camblas_cuda_context *context = context_for(a.get_device(), backend_algorithm);
    succeed(camblas_cuda_bgemm_add(context, first.flag, second.flag, columns, rows, inner, float(alpha), first.data(),
                                   first.leading, second.data(), second.leading, float(beta), addend.data,
                                   addend.pitch, result.mutable_data_ptr(), std::max(columns, 1)),
            context);
    return result;
}

Tensor backend_addmm(const Tensor &bias, const Tensor &a, const Tensor &b, const at::Scalar &beta,
                     const at::Scalar &alpha)
{
    const bool taken = takes_product(a, b) && takes_bias(bias, a.size(0), b.size(1), a) && !beta.isComplex() &&
                       !alpha.isComplex();
    if (!taken)
        return at::cuda::addmm(bias, a, b, beta, alpha);
    c10::DeviceGuard guard(a.device());
    const double keep = beta.toDouble();
    const std::vector<int64_t> shape = {a.size(0), b.size(1)};
    if (keep != 0 && a.numel() > 0 && b.numel() > 0) {
        const Addend addend = epilogue_addend(bias, shape[0], shape[1]);
        if (addend.data)
            return bf16_product_adding(addend, a, b, alpha.toDouble(), keep);
    }
    // beta == 0 never reads the bias (NaN-safe); otherwise the product accumulates onto a copy of it
    Tensor out = keep == 0 ? at::empty(shape, a.options()) : bias.expand(shape).clone(at::MemoryFormat::Contiguous);
    return matmul(a, b, out, alpha.toDouble(), keep, backend_algorithm, false);
}

void install_torch_backend(int algorithm)
{
    static std::mutex guard;
    std::lock_guard<std::mutex> lock(guard);
    if (backend_registration)
        return;
    TORCH_CHECK(algorithm >= CAMBLAS_CUDA_AUTO && algorithm <= CAMBLAS_CUDA_STRASSEN_FOUR, "Invalid CAMBLAS algorithm");
    backend_algorithm = algorithm;
    backend_registration =
        std::make_unique<torch::Library>(torch::Library::IMPL, "aten", c10::DispatchKey::CUDA, __FILE__, __LINE__);
    backend_registration->impl("mm", TORCH_FN(backend_mm));
    backend_registration->impl("mm.out", TORCH_FN(backend_mm_out));
    backend_registration->impl("addmm", TORCH_FN(backend_addmm));
}

void set_default_algorithm(int algorithm) { default_algorithm = algorithm; }
} // namespace
} // namespace binding

PYBIND11_MODULE(_camblas_cuda_torch, module)
{
    using namespace binding;
    module.def("install_torch_backend", &install_torch_backend);
    module.def("set_default_algorithm", &set_default_algorithm);
    module.def("matmul",
               [](const Tensor &a, const Tensor &b, const std::optional<Tensor> &out, double alpha,
                  double beta, int algorithm) { return matmul(a, b, out, alpha, beta, algorithm); });
    module.def("matmul_public", &matmul_public, py::arg("a"), py::arg("b"), py::kw_only(),
               py::arg("out") = py::none(), py::arg("alpha") = 1., py::arg("beta") = 0.,
               py::arg("algorithm") = -1,
               "Multiply two GPU matrices (FP32, FP64 or BF16) with transpose views and autograd.");
    module.def("linear_public", &linear_public, py::arg("input"), py::arg("weight"),
               py::arg("bias") = py::none(), py::kw_only(), py::arg("algorithm") = -1,
               "Apply a linear transform with [outputs, inputs] weights and autograd.");
    register_dense(module);
    register_fusion(module);
    register_quantized(module);
    module.def("stats", &stats);
    module.def("stats_all", &stats_all);
    module.def("close", &close_all);
}
