// What every extern "C" entry point of libcamblas_hip.so does before and after its own work:
// make the context's device current for the duration of the call, turn C++ exceptions into status
// codes, and check arguments from small tables instead of long boolean chains.
//
// The contract these helpers implement is the reference's (src/cuda/backend.cu:81-86 for the
// status convention, :913-951 for device activation and exception mapping): a failed call leaves
// "<operation> failed (status <code>)" in the context, returns -code (or -1), never throws, and
// leaves the caller's current device as it found it.
#pragma once

#include "common.hpp"

#include <cstdint>
#include <exception>
#include <initializer_list>
#include <new>

namespace camblas_hip
{
// One call through the C ABI. Constructed first thing in an entry point; `run` executes the body.
class Entry
{
  public:
    explicit Entry(camblas_cuda_context *context) : context_(context)
    {
        if (!context_)
            return;
        int current = -1;
        activation_ = hipGetDevice(&current);
        if (activation_ == hipSuccess && current != context_->device) {
            activation_ = hipSetDevice(context_->device);
            if (activation_ == hipSuccess)
                restore_to_ = current;
        }
    }
    Entry(const Entry &) = delete;
    Entry &operator=(const Entry &) = delete;
    ~Entry()
    {
        if (restore_to_ >= 0)
            (void)hipSetDevice(restore_to_);
    }

    camblas_cuda_context *context() const { return context_; }
    hipStream_t stream() const { return context_->stream; }

    // Records the failure text and returns the status to hand back to the caller.
    int refuse(const char *operation, int code = 1) const { return fail(context_, operation, code); }

    // Status of a launch: 0, or the recorded failure.
    int finish(hipError_t launched, const char *operation) const
    {
        return launched == hipSuccess ? 0 : fail(context_, operation, int(launched));
    }

    // Runs `body` (returning an int status) on the context's device; nothing escapes as an exception.
    template <typename Body> int run(Body body) const
    {
        if (!context_)
            return fail(nullptr, "missing context", 1);
        if (activation_ != hipSuccess)
            return fail(context_, "activate device", int(activation_));
        try {
            return body();
        } catch (const std::bad_alloc &) {
            return fail(context_, "host allocation", 2);
        } catch (const std::exception &error) {
            std::snprintf(context_->error, sizeof(context_->error), "host exception: %s", error.what());
        } catch (...) {
            return fail(context_, "unexpected host exception", 1);
        }
        return -1;
    }

  private:
    camblas_cuda_context *context_;
    hipError_t activation_ = hipSuccess;
    int restore_to_ = -1; // the caller's device when the call had to switch away from it
};

// ---- argument tables -----------------------------------------------------------------------

// low <= value <= high and value a multiple of `step`
struct Bound {
    long long value, low, high, step;
};

inline bool within(std::initializer_list<Bound> bounds)
{
    for (const Bound &bound : bounds)
        if (bound.value < bound.low || bound.value > bound.high || (bound.step > 1 && bound.value % bound.step))
            return false;
    return true;
}

// A buffer argument: where it points, the alignment its kernel needs, whether it may be absent.
struct Buffer {
    const void *address;
    size_t alignment;
    bool optional = false;
};

inline bool is_aligned(const void *address, size_t bytes)
{
    return reinterpret_cast<uintptr_t>(address) % bytes == 0;
}

inline bool usable(std::initializer_list<Buffer> buffers)
{
    for (const Buffer &buffer : buffers) {
        if (!buffer.address) {
            if (!buffer.optional)
                return false;
        } else if (!is_aligned(buffer.address, buffer.alignment)) {
            return false;
        }
    }
    return true;
}

// `written` starts at none of the given (non-null) addresses
inline bool apart(const void *written, std::initializer_list<const void *> others)
{
    if (!written)
        return true;
    for (const void *other : others)
        if (other == written)
            return false;
    return true;
}

// every pair of the given non-null addresses differs
inline bool all_apart(std::initializer_list<const void *> addresses)
{
    for (auto first = addresses.begin(); first != addresses.end(); ++first)
        for (auto second = first + 1; second != addresses.end(); ++second)
            if (*first && *first == *second)
                return false;
    return true;
}

// storage codes of the ABI: 0 FP32, 1 FP64, 2 BF16
inline bool storage_in(int dtype, std::initializer_list<int> accepted)
{
    for (int code : accepted)
        if (dtype == code)
            return true;
    return false;
}

inline size_t storage_bytes(int dtype) { return dtype == 0 ? 4 : dtype == 1 ? 8 : 2; }

inline bool is_flag(int value) { return value == 0 || value == 1; }

// 'N'/'n' -> 0, 'T'/'t' -> 1, anything else -> -1
inline int transposition(char flag)
{
    return flag == 'N' || flag == 'n' ? 0 : flag == 'T' || flag == 't' ? 1 : -1;
}
} // namespace camblas_hip
