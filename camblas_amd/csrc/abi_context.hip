// Context lifetime, status text, scratch arena, counters and planner introspection of
// libcamblas_hip.so (ref for the contract: include/camblas_cuda.h:12-42, :211-215 and
// src/cuda/backend.cu:57-86, :399-426, :954-1055, :1477-1493). No kernel lives here.
#include "entry.hpp"

#include <algorithm>
#include <cstring>
#include <new>

namespace camblas_hip
{
namespace
{
thread_local char creation_error[256] = ""; // failures that have no context to record them in

// growth beyond this size takes exactly what is asked for instead of doubling
constexpr size_t DOUBLING_LIMIT = size_t(256) << 20;

bool stream_is_capturing(hipStream_t stream)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone;
}
} // namespace

int fail(camblas_cuda_context *context, const char *operation, int code)
{
    char *text = context ? context->error : creation_error;
    std::snprintf(text, 256, "%s failed (status %d)", operation, code);
    return code > 0 ? -code : -1;
}

// The arena only grows, and never while the stream is being captured (a captured launch holds the
// old address). Small arenas double so that a run of slightly larger requests settles quickly;
// large ones (the multi-gigabyte Strassen workspaces) take the exact size. A superseded arena is
// freed at once when nothing captured can still refer to it, i.e. when this context has never
// launched under capture; otherwise it is parked until the context is destroyed.
hipError_t reserve_scratch(camblas_cuda_context *context, size_t bytes)
{
    if (bytes <= context->scratch_bytes) {
        // remember the first use under capture: from then on a replaced arena has to be kept
        if (bytes && !context->seen_capture && stream_is_capturing(context->stream))
            context->seen_capture = true;
        return hipSuccess;
    }
    if (stream_is_capturing(context->stream))
        return hipErrorStreamCaptureUnsupported;
    size_t wanted = bytes < DOUBLING_LIMIT ? std::max(bytes, 2 * context->scratch_bytes) : bytes;
    wanted = (wanted + 255) / 256 * 256;
    void *arena = nullptr;
    const hipError_t status = hipMalloc(&arena, wanted);
    if (status != hipSuccess) {
        (void)hipGetLastError(); // the failure is reported by our own status, not by the next launch
        return status;
    }
    if (context->scratch) {
        if (context->seen_capture || hipStreamSynchronize(context->stream) != hipSuccess) {
            context->retired.push_back(context->scratch);
            context->retired_bytes += context->scratch_bytes;
        } else
            (void)hipFree(context->scratch);
    }
    context->scratch = arena;
    context->scratch_bytes = wanted;
    return hipSuccess;
}

void *claim_scratch(camblas_cuda_context *context, size_t bytes)
{
    const size_t offset = (context->held_bytes + 255) / 256 * 256;
    if (context->held_bytes && offset + bytes > context->scratch_bytes)
        return nullptr;
    if (reserve_scratch(context, offset + bytes) != hipSuccess)
        return nullptr;
    return static_cast<char *>(context->scratch) + offset;
}

hipError_t reserve_arrivals(camblas_cuda_context *context)
{
    if (context->arrivals)
        return hipSuccess;
    if (stream_is_capturing(context->stream))
        return hipErrorStreamCaptureUnsupported;
    void *counters = nullptr;
    hipError_t status = hipMalloc(&counters, STREAM_ARRIVAL_SLOTS * sizeof(unsigned));
    if (status == hipSuccess)
        status = hipMemsetAsync(counters, 0, STREAM_ARRIVAL_SLOTS * sizeof(unsigned), context->stream);
    if (status != hipSuccess) {
        (void)hipGetLastError();
        if (counters)
            (void)hipFree(counters);
        return status;
    }
    context->arrivals = static_cast<unsigned *>(counters);
    return hipSuccess;
}

} // namespace camblas_hip

using namespace camblas_hip;

extern "C" int camblas_cuda_create(int device, void *stream, camblas_cuda_context **out)
{
    if (!out)
        return fail(nullptr, "missing context output", 1);
    *out = nullptr;
    // the new context's device has to be current for the queries below; put the caller's back after
    int callers = -1;
    hipError_t status = hipGetDevice(&callers);
    if (status == hipSuccess && callers != device)
        status = hipSetDevice(device);
    if (status != hipSuccess)
        return fail(nullptr, "activate device", int(status));
    struct Restore {
        int device, callers;
        ~Restore()
        {
            if (callers != device)
                (void)hipSetDevice(callers);
        }
    } restore{device, callers};

    hipDeviceProp_t properties;
    status = hipGetDeviceProperties(&properties, device);
    if (status != hipSuccess)
        return fail(nullptr, "device properties", int(status));
    if (std::strncmp(properties.gcnArchName, "gfx950", 6) != 0) {
        std::snprintf(creation_error, sizeof(creation_error),
                      "libcamblas_hip is built for gfx950 only; device %d is %s", device,
                      properties.gcnArchName);
        return -1;
    }
    // the allocation-free attention entry point's fixed array: find this device's copy now, so
    // that the entry point itself never has to ask the runtime
    void *resident = nullptr;
    status = gqa_resident_scratch(device, &resident);
    if (status != hipSuccess)
        return fail(nullptr, "resident scratch address", int(status));
    camblas_cuda_context *context = new (std::nothrow) camblas_cuda_context;
    if (!context)
        return fail(nullptr, "context allocation", 2);
    context->device = device;
    context->stream = static_cast<hipStream_t>(stream);
    context->compute_units = properties.multiProcessorCount;
    *out = context;
    return 0;
}

extern "C" int camblas_cuda_destroy(camblas_cuda_context *context)
{
    if (!context)
        return 0;
    Entry entry(context);
    return entry.run([&] {
        // pending work may still read the arenas: wait for the stream, then release everything
        const hipError_t drained = hipStreamSynchronize(context->stream);
        if (context->scratch)
            (void)hipFree(context->scratch);
        if (context->arrivals)
            (void)hipFree(context->arrivals);
        for (void *arena : context->retired)
            (void)hipFree(arena);
        delete context;
        return drained == hipSuccess ? 0
                                     : fail(nullptr, "stream completion during destruction", int(drained));
    });
}

extern "C" const char *camblas_cuda_error(const camblas_cuda_context *context)
{
    return context ? context->error : creation_error;
}

extern "C" int camblas_cuda_set_algorithm(camblas_cuda_context *context, int algorithm)
{
    if (!context || !within({{algorithm, CAMBLAS_CUDA_AUTO, CAMBLAS_CUDA_STRASSEN_FOUR, 1}}))
        return fail(context, "invalid algorithm", 1);
    context->algorithm = algorithm;
    return 0;
}

extern "C" int camblas_cuda_stats(const camblas_cuda_context *context, uint64_t *counts, int length)
{
    if (!context || !counts || (length != 6 && length != 8))
        return fail(nullptr, "invalid stats output", 1);
    std::transform(context->counts, context->counts + length, counts,
                   [](const std::atomic<uint64_t> &count) { return count.load(std::memory_order_relaxed); });
    return 0;
}

extern "C" int camblas_cuda_reset_stats(camblas_cuda_context *context)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    for (std::atomic<uint64_t> &count : context->counts)
        count.store(0, std::memory_order_relaxed);
    return 0;
}

// ---- planner introspection and the test override

extern "C" int camblas_hip_plan_describe(int dtype, int algorithm, char trans_a, char trans_b, int m,
                                         int n, int k, int lda, int ldb, int ldc, int aligned16,
                                         char *text, size_t text_bytes)
{
    const int ta = transposition(trans_a), tb = transposition(trans_b);
    if (!storage_in(dtype, {0, 2, 3}) || ta < 0 || tb < 0 || m < 1 || n < 1 || k < 1)
        return -1;
    const Plan plan =
        make_plan(dtype, algorithm, ta == 1, tb == 1, m, n, k, lda, ldb, ldc, aligned16 != 0, 256);
    describe_plan(plan, dtype, text, text_bytes);
    return plan.family * 1000 + plan.kernel;
}

extern "C" int camblas_hip_set_plan_override(camblas_cuda_context *context, int kernel, int split_k)
{
    if (!context)
        return fail(nullptr, "missing context", 1);
    context->override_kernel = kernel;
    context->override_split = split_k;
    return 0;
}

extern "C" int camblas_hip_kernel_count(int dtype)
{
    return dtype == 2 ? tn_variant_count() : dtype == 3 ? fp8_variant_count() : 1;
}
