/* Test-only fault injection for the allocation-failure routes of libcamblas_hip.so: preloaded into
 * a child process, it makes the next hipMalloc after arm() return hipErrorOutOfMemory once, without
 * touching the device. Every other call goes to the HIP runtime unchanged. (The counterpart of the
 * reference's tests/cuda_fail_alloc.c.) */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stddef.h>

static int pending;

void camblas_test_fail_next_allocation(void) { __atomic_store_n(&pending, 1, __ATOMIC_RELEASE); }

int camblas_test_allocation_pending(void) { return __atomic_load_n(&pending, __ATOMIC_ACQUIRE); }

/* same signature as the runtime's: hipError_t hipMalloc(void **, size_t); 2 is hipErrorOutOfMemory */
int hipMalloc(void **pointer, size_t bytes)
{
    static int (*runtime)(void **, size_t);
    if (__atomic_exchange_n(&pending, 0, __ATOMIC_ACQ_REL)) {
        if (pointer)
            *pointer = NULL;
        return 2;
    }
    if (!runtime)
        runtime = (int (*)(void **, size_t))dlsym(RTLD_NEXT, "hipMalloc");
    if (!runtime) {
        /* the runtime was loaded into a local scope (as a dependency of a dlopen'ed module): ask the
         * already-loaded library itself, without loading another copy */
        static const char *const names[] = {"libamdhip64.so.7", "libamdhip64.so", "libamdhip64.so.6"};
        for (unsigned i = 0; i < sizeof(names) / sizeof(names[0]) && !runtime; ++i) {
            void *handle = dlopen(names[i], RTLD_NOLOAD | RTLD_LAZY);
            if (handle)
                runtime = (int (*)(void **, size_t))dlsym(handle, "hipMalloc");
        }
    }
    return runtime ? runtime(pointer, bytes) : 999; /* hipErrorUnknown */
}
