// Shared pieces of the ATen binding (_camblas_cuda_torch*.so): the per-thread library contexts,
// argument checking for tensors, and the entry points other translation units call.
//
// The module's function surface is the one the reference's Python layer imports
// (ref: src/cuda/torch_bindings.cpp:1194-1294); how tensors are checked is this binding's own: an
// operand is described by a `Want` (accepted dtypes, rank, density) and admitted against the device
// of the call, instead of condition chains per function.
#pragma once

#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/core/GradMode.h>

#include <climits>
#include <initializer_list>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "camblas_hip.h"

namespace binding
{
using at::Tensor;

// ---- failures: invalid arguments raise ValueError, library failures RuntimeError
inline void require(bool condition, const char *message)
{
    if (!condition)
        throw std::invalid_argument(message);
}
inline void require(bool condition, const std::string &message)
{
    if (!condition)
        throw std::invalid_argument(message);
}
void same_process();                                           // refuses use after fork
void succeed(int status, camblas_cuda_context *context);       // raises with the library's text

// ---- contexts: one per (thread, device, current stream); refused while that stream is capturing
camblas_cuda_context *context_for(int device, int algorithm);
int current_default_algorithm();                               // the calling thread's policy
inline int resolve(int algorithm) { return algorithm < 0 ? current_default_algorithm() : algorithm; }

// ---- operand descriptions
struct Want {
    std::initializer_list<at::ScalarType> dtypes; // any of these
    int rank = -1;                                // exact number of dimensions; -1: at least one
    bool dense = true;                            // contiguous storage
};

// Throws unless `tensor` lives on `device`, matches `want`, has 32-bit sizes, and (when autograd is
// recording) does not require gradients. `role` names the operand in the message.
void admit(const char *role, const Tensor &tensor, const at::Device &device, const Want &want);

// rows of a tensor viewed as [rows, last dimension]; throws when they exceed `limit`
int64_t flattened_rows(const Tensor &tensor, int64_t limit, const char *what);

inline bool recording(const Tensor &tensor)
{
    return c10::GradMode::is_enabled() && tensor.requires_grad();
}

// ---- the dense checks shared with the GEMM entry points (FP32 / FP64 / optionally BF16 on one GPU)
void check_tensor(const Tensor &tensor, const Tensor &like, bool allow_bf16);
void check_inference(const Tensor &tensor, const Tensor &like);
inline int storage_code(const Tensor &tensor) { return tensor.scalar_type() == at::kFloat ? 0 : 2; }

// ---- products other units build on
Tensor matmul(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output, double alpha,
              double beta, int algorithm, bool update_version = true);
Tensor matmul_public(const Tensor &a, const Tensor &b, const std::optional<Tensor> &output, double alpha,
                     double beta, int algorithm);
Tensor linear_public(const Tensor &x, const Tensor &weight, const std::optional<Tensor> &bias, int algorithm);

// ---- registration of each unit's functions on the module
void register_dense(pybind11::module_ &module);
void register_fusion(pybind11::module_ &module);
void register_quantized(pybind11::module_ &module);
} // namespace binding
