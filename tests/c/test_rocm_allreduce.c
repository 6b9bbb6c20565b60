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
 * usage: test_rocm_allreduce <plugin dir> [team size] [count] [dtype op]
 *
 * Without dtype and op: INT32 SUM on the reference's inputs, as above.  With
 * them ("INT8" .. "UINT64", "FLOAT32", "FLOAT64"; "MAX" "MIN" "SUM" "PROD"
 * "LAND" "LOR" "LXOR" "BAND" "BOR" "BXOR"; or "ALL ALL" for every such pair):
 * the reference's "then every (dtype, op)" step -- seeded inputs, expected
 * vector folded on the host with the C operators of the reference's reduce.h.
 * Only operators whose result does not depend on the fold order are run
 * (integers: all ten; floating point: MAX, MIN, and SUM on small integers).
 */
#include <stdint.h>
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

/* ---- typed inputs and the host fold ------------------------------------- */
typedef struct {
    const char *name;
    xccl_dt_t   dt;
    size_t      size;
    int         is_float;
} dt_desc_t;

static const dt_desc_t dts[] = {
    {"INT8", XCCL_DT_INT8, 1, 0},     {"INT16", XCCL_DT_INT16, 2, 0},   {"INT32", XCCL_DT_INT32, 4, 0},
    {"INT64", XCCL_DT_INT64, 8, 0},   {"UINT8", XCCL_DT_UINT8, 1, 0},   {"UINT16", XCCL_DT_UINT16, 2, 0},
    {"UINT32", XCCL_DT_UINT32, 4, 0}, {"UINT64", XCCL_DT_UINT64, 8, 0}, {"FLOAT32", XCCL_DT_FLOAT32, 4, 1},
    {"FLOAT64", XCCL_DT_FLOAT64, 8, 1},
};

typedef struct {
    const char *name;
    xccl_op_t   op;
} op_desc_t;

static const op_desc_t ops[] = {
    {"MAX", XCCL_OP_MAX},   {"MIN", XCCL_OP_MIN},   {"SUM", XCCL_OP_SUM},   {"PROD", XCCL_OP_PROD},
    {"LAND", XCCL_OP_LAND}, {"LOR", XCCL_OP_LOR},   {"LXOR", XCCL_OP_LXOR}, {"BAND", XCCL_OP_BAND},
    {"BOR", XCCL_OP_BOR},   {"BXOR", XCCL_OP_BXOR},
};

static uint64_t mix(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

/* reduce.h:14-23, on one element of type T held in memory at a, b, out */
#define FOLD_INT(T)                                                                 \
    static void fold_##T(xccl_op_t op, const void *pa, const void *pb, void *po)    \
    {                                                                               \
        T a, b, r = 0;                                                              \
        memcpy(&a, pa, sizeof(T));                                                  \
        memcpy(&b, pb, sizeof(T));                                                  \
        switch (op) {                                                               \
        case XCCL_OP_MAX:  r = a > b ? a : b; break;                                \
        case XCCL_OP_MIN:  r = a < b ? a : b; break;                                \
        case XCCL_OP_SUM:  r = (T)((uint64_t)a + (uint64_t)b); break;               \
        case XCCL_OP_PROD: r = (T)((uint64_t)a * (uint64_t)b); break;               \
        case XCCL_OP_LAND: r = (T)(a && b); break;                                  \
        case XCCL_OP_LOR:  r = (T)(a || b); break;                                  \
        case XCCL_OP_LXOR: r = (T)((!a) != (!b)); break;                            \
        case XCCL_OP_BAND: r = (T)(a & b); break;                                   \
        case XCCL_OP_BOR:  r = (T)(a | b); break;                                   \
        case XCCL_OP_BXOR: r = (T)(a ^ b); break;                                   \
        default: break;                                                             \
        }                                                                           \
        memcpy(po, &r, sizeof(T));                                                  \
    }
#define FOLD_FP(T)                                                                  \
    static void fold_##T(xccl_op_t op, const void *pa, const void *pb, void *po)    \
    {                                                                               \
        T a, b, r = 0;                                                              \
        memcpy(&a, pa, sizeof(T));                                                  \
        memcpy(&b, pb, sizeof(T));                                                  \
        switch (op) {                                                               \
        case XCCL_OP_MAX: r = a > b ? a : b; break;                                 \
        case XCCL_OP_MIN: r = a < b ? a : b; break;                                 \
        case XCCL_OP_SUM: r = a + b; break;                                         \
        default: break;                                                             \
        }                                                                           \
        memcpy(po, &r, sizeof(T));                                                  \
    }
FOLD_INT(int8_t) FOLD_INT(int16_t) FOLD_INT(int32_t) FOLD_INT(int64_t)
FOLD_INT(uint8_t) FOLD_INT(uint16_t) FOLD_INT(uint32_t) FOLD_INT(uint64_t)
FOLD_FP(float) FOLD_FP(double)

typedef void (*fold_fn_t)(xccl_op_t, const void *, const void *, void *);

static fold_fn_t fold_of(xccl_dt_t dt)
{
    switch (dt) {
    case XCCL_DT_INT8:    return fold_int8_t;
    case XCCL_DT_INT16:   return fold_int16_t;
    case XCCL_DT_INT32:   return fold_int32_t;
    case XCCL_DT_INT64:   return fold_int64_t;
    case XCCL_DT_UINT8:   return fold_uint8_t;
    case XCCL_DT_UINT16:  return fold_uint16_t;
    case XCCL_DT_UINT32:  return fold_uint32_t;
    case XCCL_DT_UINT64:  return fold_uint64_t;
    case XCCL_DT_FLOAT32: return fold_float;
    default:              return fold_double;
    }
}

/* Element i of rank `rank`: full-range bits for integers (half of them zero
 * for the logical operators), integers of magnitude < 2^20 for floating
 * point (sums of up to 2^3 ranks of them stay exact). */
static void make_element(const dt_desc_t *d, xccl_op_t op, int rank, int i, void *out)
{
    const uint64_t x = mix(((uint64_t)rank << 32) + (uint64_t)i);
    const int logical = op == XCCL_OP_LAND || op == XCCL_OP_LOR || op == XCCL_OP_LXOR;

    if (d->is_float) {
        const double v = (double)((int64_t)(x >> 43) - (1 << 20));
        if (d->size == 4) {
            const float f = (float)v;
            memcpy(out, &f, 4);
        } else {
            memcpy(out, &v, 8);
        }
    } else {
        const uint64_t v = (logical && (x >> 63)) ? 0 : x;
        memcpy(out, &v, d->size); /* little endian: the low bytes */
    }
}

static int run_case(xccl_replay_alg_t alg, int size, int count, int root, int radix, xccl_replay_reduce_mode_t mode,
                    const dt_desc_t *d, xccl_op_t op)
{
    const size_t msg_size = (size_t)count * (d ? d->size : sizeof(int));
    char        *sbuf_host = (char *)malloc(msg_size), *rbuf_host = (char *)malloc(msg_size);
    char        *expected = (char *)malloc(msg_size);
    void       **sbuf_rocm = (void **)calloc((size_t)size, sizeof(void *));
    void       **rbuf_rocm = (void **)calloc((size_t)size, sizeof(void *));
    int          rank, i, status = 0;
    const int    rooted = alg == XCCL_REPLAY_REDUCE_KNOMIAL || alg == XCCL_REPLAY_REDUCE_LINEAR;

    for (rank = 0; rank < size; rank++) {
        CHECK(xccl_mem_component_alloc(&sbuf_rocm[rank], msg_size, UCS_MEMORY_TYPE_ROCM));
        CHECK(xccl_mem_component_alloc(&rbuf_rocm[rank], msg_size, UCS_MEMORY_TYPE_ROCM));
        for (i = 0; i < count; i++) {
            if (d == NULL) {
                ((int *)sbuf_host)[i] = rank + 1 + 12345 + i;
            } else {
                make_element(d, op, rank, i, sbuf_host + (size_t)i * d->size);
                if (rank == 0) {
                    memcpy(expected + (size_t)i * d->size, sbuf_host + (size_t)i * d->size, d->size);
                } else {
                    fold_of(d->dt)(op, expected + (size_t)i * d->size, sbuf_host + (size_t)i * d->size,
                                   expected + (size_t)i * d->size);
                }
            }
        }
        CHECK(hipMemcpy(sbuf_rocm[rank], sbuf_host, msg_size, hipMemcpyHostToDevice));
        CHECK(hipMemset(rbuf_rocm[rank], 0, msg_size));
    }
    CHECK(hipDeviceSynchronize());
    if (d == NULL) {
        for (i = 0; i < count; i++) {
            ((int *)expected)[i] = size * (size + 1) / 2 + size * (i + 12345);
        }
    }

    xccl_replay_params_t coll = {
        .alg         = alg,
        .reduce_mode = mode,
        .team_size   = size,
        .radix       = radix,
        .root        = root,
        .count       = (size_t)count,
        .dtype       = d ? d->dt : XCCL_DT_INT32,
        .op          = d ? op : XCCL_OP_SUM,
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
            fprintf(stderr, "RST CHECK FAILURE at rank %d (alg %d, size %d, root %d, radix %d, %s %d)\n", rank, (int)alg,
                    size, root, radix, d ? d->name : "INT32", (int)coll.op);
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

/* every algorithm, both reduction modes, every root for the rooted ones */
static int run_all_algorithms(int size, int count, const dt_desc_t *d, xccl_op_t op)
{
    int status = 0, root, alg, mode;

    for (mode = 0; mode < 2; mode++) {
        for (alg = XCCL_REPLAY_ALLREDUCE_KNOMIAL; alg <= XCCL_REPLAY_ALLREDUCE_SRA; alg++) {
            status |= run_case((xccl_replay_alg_t)alg, size, count, 0, 4, (xccl_replay_reduce_mode_t)mode, d, op);
        }
        for (alg = XCCL_REPLAY_REDUCE_KNOMIAL; alg <= XCCL_REPLAY_REDUCE_LINEAR; alg++) {
            for (root = 0; root < size; root++) { /* test_mpi_cuda_reduce.c: every root */
                if (d != NULL && root != 0 && root != size - 1) {
                    continue; /* the typed sweep checks the first and the last root */
                }
                status |= run_case((xccl_replay_alg_t)alg, size, count, root, 4, (xccl_replay_reduce_mode_t)mode, d, op);
            }
        }
    }
    return status;
}

int main(int argc, char **argv)
{
    const int   size  = argc > 2 ? atoi(argv[2]) : 8;
    const int   count = argc > 3 ? atoi(argv[3]) : 32;
    const char *dname = argc > 5 ? argv[4] : NULL, *oname = argc > 5 ? argv[5] : NULL;
    int         status = 0, cases = 0;
    size_t      di, oi;
    ucs_memory_type_t mt;
    void             *probe;

    if (argc < 2 || argc == 5 || size < 1 || size > 8 * (dname != NULL) + 1024 * (dname == NULL)) {
        fprintf(stderr, "usage: %s <plugin dir> [team size] [count] [dtype op]   (team size <= 8 with dtype op)\n",
                argv[0]);
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

    if (dname == NULL) {
        status = run_all_algorithms(size, count, NULL, XCCL_OP_SUM);
        cases  = 1;
    } else {
        for (di = 0; di < sizeof(dts) / sizeof(dts[0]); di++) {
            if (strcmp(dname, "ALL") != 0 && strcmp(dname, dts[di].name) != 0) {
                continue;
            }
            for (oi = 0; oi < sizeof(ops) / sizeof(ops[0]); oi++) {
                if (strcmp(oname, "ALL") != 0 && strcmp(oname, ops[oi].name) != 0) {
                    continue;
                }
                if (dts[di].is_float && ops[oi].op != XCCL_OP_MAX && ops[oi].op != XCCL_OP_MIN &&
                    ops[oi].op != XCCL_OP_SUM) {
                    continue; /* PROD depends on the fold order; logical and bitwise are not defined */
                }
                status |= run_all_algorithms(size, count, &dts[di], ops[oi].op);
                cases++;
            }
        }
        if (cases == 0) {
            fprintf(stderr, "no (dtype, op) pair matches %s %s\n", dname, oname);
            return 2;
        }
    }
    xccl_mem_component_free_cache();
    xccl_mem_component_finalize();
    if (status == 0) {
        printf("Correctness check: PASSED (team size %d, count %d, %d dtype/op case%s)\n", size, count, cases,
               cases == 1 ? "" : "s");
    } else {
        printf("Correctness check: FAILED\n");
    }
    return status;
}
