/*
 * TEST INFRASTRUCTURE ONLY. Thin driver around the reference's own CPU library, compiled together
 * with the reference's C sources (where they lie, never copied) into oracle/_ref/. It exposes two
 * plain entry points so Python can call the reference without mirroring its context structs:
 *   ref_sgemm_scalar  - camblas_sgemm on the default context (scalar kernel, one thread;
 *                       src/planner.c:409-418, src/scalar.c:223-255)
 *   ref_sgemm_packed  - camblas_sgemm with planner_mode "shape-aware", the discovered topology
 *                       and a pthread-pool executor on `threads` allowed CPUs
 *                       (src/planner.c:553-591, src/packed.c:465-626, src/pthread_pool.c)
 */
#include "camblas.h"
#include "camblas_pthread.h"
#include "camblas_topology.h"

#include <stdlib.h>

int ref_sgemm_scalar(char ta, char tb, int m, int n, int k, float alpha, const float *a, int lda,
                     const float *b, int ldb, float beta, float *c, int ldc)
{
    return camblas_sgemm(&camblas_ctx_default, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

static camblas_topology_t topology;
static int topology_ready;
static camblas_pthread_pool_t *pool;
static int pool_threads;

int ref_threads_available(void)
{
    if (!topology_ready) {
        int status = camblas_topology_discover(&topology);
        if (CAMBLAS_TOPO_IS_FATAL(status))
            return -1;
        topology_ready = 1;
    }
    return topology.n_allowed_cpus;
}

int ref_sgemm_packed(int threads, char ta, char tb, int m, int n, int k, float alpha,
                     const float *a, int lda, const float *b, int ldb, float beta, float *c, int ldc)
{
    int available = ref_threads_available();
    if (available < 1)
        return -2;
    if (threads < 1 || threads > available)
        threads = available;
    if (!pool || pool_threads != threads) {
        if (pool)
            camblas_pthread_pool_destroy(pool);
        int *cpus = (int *)malloc(sizeof(int) * (size_t)threads), found = 0;
        for (int cpu = 0; cpu < topology.allowed_cpus.nbits && found < threads; ++cpu)
            if (topology.allowed_cpus.bits[cpu / 64] >> (cpu % 64) & 1)
                cpus[found++] = cpu;
        pool = camblas_pthread_pool_create(found, cpus);
        free(cpus);
        pool_threads = threads;
        if (!pool)
            return -3;
    }
    camblas_ctx_t context = {.num_threads = threads,
                             .reproducibility = CAMBLAS_REPRO_FAST,
                             .planner_mode = "shape-aware",
                             .topo = &topology,
                             .executor = camblas_pthread_pool_executor(pool)};
    return camblas_sgemm(&context, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}
