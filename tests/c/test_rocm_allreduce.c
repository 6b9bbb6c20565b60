/*
 * test_rocm_allreduce.c -- the reference's device tests, for the ROCm memory
 * component, in one process.
 *
 * Shape of reference test/test_mpi_cuda_allreduce.c (allreduce: device send
 * and receive buffers, INT32, SUM, count 32, sbuf[i] = rank + 1 + 12345 + i,
 * result copied back and memcmp'ed) and test/test_mpi_cuda_reduce.c (the same
 * for every root).  MPI and UCX are replaced by the loopback ranks of
 * libxccl_ucx_replay.so; the expected vector is the closed form the
 * reference's threaded test checks, test/test_mt.c:58.
 *
 * usage: test_rocm_allreduce <plugin dir> [team size] [count]
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "xccl_rocm_mem_component.h"
#include "xccl_rocm_ucx_replay.h"

#define CHECK(cmd)                                                         \
    do {                                                                   \
        int st_ = (int)(cmd);                                              \
        if (st_ != 0) {                                                    \
            fprintf(stderr, "%s:%d %s failed: %d\n", __FILE__, __LINE__, #cmd, st_); \
            return 2;                                                      \
        }                                                                  \
    } while (0)

static int run_case(xccl_replay_alg_t alg, int size, int count, int root, int radix, xccl_replay_reduce_mode_t mode)
{
    const size_t msg_size = (size_t)count * sizeof(int);
    int         *sbuf_host = (int *)malloc(msg_size), *rbuf_host = (int *)malloc(msg_size);
    int         *expected = (int *)malloc(msg_size);
    void       **sbuf_rocm = (void **)calloc((size_t)size, sizeof(void *));
    void       **rbuf_rocm = (void **)calloc((size_t)size, sizeof(void *));
    int          rank, i, status = 0;
    const int    rooted = alg == XCCL_REPLAY_REDUCE_KNOMIAL || alg == XCCL_REPLAY_REDUCE_LINEAR;

    for (rank = 0; rank < size; rank++) {
        CHECK(xccl_mem_component_alloc(&sbuf_rocm[rank], msg_size, UCS_MEMORY_TYPE_ROCM));
        CHECK(xccl_mem_component_alloc(&rbuf_rocm[rank], msg_size, UCS_MEMORY_TYPE_ROCM));
        for (i = 0; i < count; i++) {
            sbuf_host[i] = rank + 1 + 12345 + i;
        }
        CHECK(hipMemcpy(sbuf_rocm[rank], sbuf_host, msg_size, hipMemcpyHostToDevice));
        CHECK(hipMemset(rbuf_rocm[rank], 0, msg_size));
    }
    CHECK(hipDeviceSynchronize());
    for (i = 0; i < count; i++) {
        expected[i] = size * (size + 1) / 2 + size * (i + 12345);
    }

    xccl_replay_params_t coll = {
        .alg         = alg,
        .reduce_mode = mode,
        .team_size   = size,
        .radix       = radix,
        .root        = root,
        .count       = (size_t)count,
        .dtype       = XCCL_DT_INT32,
        .op          = XCCL_OP_SUM,
        .src         = sbuf_rocm,
        .dst         = rbuf_rocm,
    };
    CHECK(xccl_replay_run(&coll, NULL, 0));

    for (rank = 0; rank < size; rank++) {
        if (rooted && rank != root) {
            continue;
        }
        CHECK(hipMemcpy(rbuf_host, rbuf_rocm[rank], msg_size, hipMemcpyDeviceToHost));
        if (0 != memcmp(rbuf_host, expected, msg_size)) {
            fprintf(stderr, "RST CHECK FAILURE at rank %d (alg %d, size %d, root %d, radix %d)\n", rank, (int)alg, size,
                    root, radix);
            status = 1;
        }
    }
    for (rank = 0; rank < size; rank++) {
        CHECK(xccl_mem_component_free(sbuf_rocm[rank], UCS_MEMORY_TYPE_ROCM));
        CHECK(xccl_mem_component_free(rbuf_rocm[rank], UCS_MEMORY_TYPE_ROCM));
    }
    free(sbuf_host);
    free(rbuf_host);
    free(expected);
    free(sbuf_rocm);
    free(rbuf_rocm);
    return status;
}

int main(int argc, char **argv)
{
    const int size  = argc > 2 ? atoi(argv[2]) : 8;
    const int count = argc > 3 ? atoi(argv[3]) : 32;
    int       status = 0, root, alg, mode;
    ucs_memory_type_t mt;
    void             *probe;

    if (argc < 2) {
        fprintf(stderr, "usage: %s <plugin dir> [team size] [count]\n", argv[0]);
        return 2;
    }
    CHECK(hipSetDevice(0));
    CHECK(xccl_mem_component_init(argv[1]));
    if (xccl_mem_component_get(UCS_MEMORY_TYPE_ROCM) == NULL) {
        fprintf(stderr, "no ROCm memory component in %s\n", argv[1]);
        return 2;
    }
    CHECK(xccl_mem_component_alloc(&probe, 64, UCS_MEMORY_TYPE_ROCM));
    CHECK(xccl_mem_component_type(probe, &mt));
    if (mt != UCS_MEMORY_TYPE_ROCM) {
        fprintf(stderr, "device pointer not recognised as ROCm memory\n");
        return 1;
    }
    CHECK(xccl_mem_component_free(probe, UCS_MEMORY_TYPE_ROCM));

    for (mode = 0; mode < 2; mode++) {
        for (alg = XCCL_REPLAY_ALLREDUCE_KNOMIAL; alg <= XCCL_REPLAY_ALLREDUCE_SRA; alg++) {
            status |= run_case((xccl_replay_alg_t)alg, size, count, 0, 4, (xccl_replay_reduce_mode_t)mode);
        }
        for (alg = XCCL_REPLAY_REDUCE_KNOMIAL; alg <= XCCL_REPLAY_REDUCE_LINEAR; alg++) {
            for (root = 0; root < size; root++) { /* test_mpi_cuda_reduce.c: every root */
                status |= run_case((xccl_replay_alg_t)alg, size, count, root, 4, (xccl_replay_reduce_mode_t)mode);
            }
        }
    }
    xccl_mem_component_free_cache();
    xccl_mem_component_finalize();
    if (status == 0) {
        printf("Correctness check: PASSED (team size %d, count %d)\n", size, count);
    } else {
        printf("Correctness check: FAILED\n");
    }
    return status;
}
