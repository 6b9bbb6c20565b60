/*
 * xccl_oracle.c -- CPU restatement of XCCL's host reduction path.
 *
 * TEST INFRASTRUCTURE, NOT PRODUCT: see xccl_oracle.h.
 *
 * Follows, in this order:
 *   operators            reference src/utils/reduce.h:14-23
 *   typed loop           reference src/utils/reduce.h:25-30
 *   dtype/op selection   reference src/utils/reduce.h:32-92, 113-140
 *   multi-source fold    reference src/utils/mem_component.c:122-148
 * Built with -O3 -fwrapv (the reference builds -O3, configure.ac:81; -fwrapv
 * turns the signed overflow the reference relies on into defined wrapping).
 *
 * Parity pins (tests/test_oracle_*.py): the INT32 SUM known answer of the
 * reference's own tests (test/test_mt.c:58), brute force against Python
 * integers on edge values for every integer dtype/op, numpy float16/32/64 for
 * the floating-point operators, the MIN/MAX truth table on +-0 and NaN, and
 * the chained-reduce invariant for the multi-source fold.  The reference
 * itself cannot be built here (needs UCX headers the image lacks), so there
 * is no oracle/_ref; INT8, UINT* and FLOAT16 have no reference implementation
 * at all and are pinned by C semantics only.
 */
#include "xccl_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* datatype and operator numbers, src/api/xccl.h:371-407 */
enum { DT_I8 = 0, DT_I16 = 1, DT_I32 = 2, DT_I64 = 3, DT_U8 = 5, DT_U16 = 6,
       DT_U32 = 7, DT_U64 = 8, DT_F16 = 10, DT_F32 = 11, DT_F64 = 12 };
enum { OP_MAX = 0, OP_MIN = 1, OP_SUM = 2, OP_PROD = 3, OP_LAND = 7, OP_LOR = 8,
       OP_LXOR = 9, OP_BAND = 10, OP_BOR = 11, OP_BXOR = 12 };

/* ---- operators: reduce.h:14-23, x = first macro argument ------------------ */
#define F_MAX(x, y)  ((x) > (y) ? (x) : (y))
#define F_MIN(x, y)  ((x) < (y) ? (x) : (y))
#define F_SUM(x, y)  ((x) + (y))
#define F_PROD(x, y) ((x) * (y))
#define F_LAND(x, y) ((x) && (y))
#define F_LOR(x, y)  ((x) || (y))
#define F_LXOR(x, y) ((!(x)) != (!(y)))
#define F_BAND(x, y) ((x) & (y))
#define F_BOR(x, y)  ((x) | (y))
#define F_BXOR(x, y) ((x) ^ (y))

/* one typed loop per (type, operator): reduce.h:25-30 */
#define LOOP(T, tag, F)                                                        \
    static void loop_##tag##_##F(const void *a_, const void *b_, void *d_,     \
                                 size_t n)                                     \
    {                                                                          \
        const T *a = (const T *)a_;                                            \
        const T *b = (const T *)b_;                                            \
        T       *d = (T *)d_;                                                  \
        for (size_t i = 0; i < n; i++) {                                       \
            d[i] = F(a[i], b[i]);                                              \
        }                                                                      \
    }

#define INT_LOOPS(T, tag)                                                      \
    LOOP(T, tag, F_MAX) LOOP(T, tag, F_MIN) LOOP(T, tag, F_SUM)                \
    LOOP(T, tag, F_PROD) LOOP(T, tag, F_LAND) LOOP(T, tag, F_LOR)              \
    LOOP(T, tag, F_LXOR) LOOP(T, tag, F_BAND) LOOP(T, tag, F_BOR)              \
    LOOP(T, tag, F_BXOR)

#define FP_LOOPS(T, tag)                                                       \
    LOOP(T, tag, F_MAX) LOOP(T, tag, F_MIN) LOOP(T, tag, F_SUM)                \
    LOOP(T, tag, F_PROD)

INT_LOOPS(int8_t, i8)
INT_LOOPS(int16_t, i16)
INT_LOOPS(int32_t, i32)
INT_LOOPS(int64_t, i64)
INT_LOOPS(uint8_t, u8)
INT_LOOPS(uint16_t, u16)
INT_LOOPS(uint32_t, u32)
INT_LOOPS(uint64_t, u64)
FP_LOOPS(float, f32)
FP_LOOPS(double, f64)

/* ---- binary16 ------------------------------------------------------------ */
float oracle_half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp  = (h >> 10) & 0x1fu;
    uint32_t       man  = h & 0x3ffu;
    uint32_t       bits;
    float          f;

    if (exp == 0x1f) {
        bits = sign | 0x7f800000u | (man << 13); /* inf / NaN, payload kept */
    } else if (exp != 0) {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        bits = sign;
    } else { /* subnormal: man * 2^-24, normal in binary32 */
        int e = -1;
        do {
            man <<= 1;
            e++;
        } while ((man & 0x400u) == 0);
        bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3ffu) << 13);
    }
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oracle_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ax   = x & 0x7fffffffu;

    if (ax >= 0x7f800000u) { /* inf / NaN (quieted, top payload bits kept) */
        if (ax == 0x7f800000u) {
            return sign | 0x7c00u;
        }
        return sign | 0x7e00u | (uint16_t)((ax >> 13) & 0x3ffu);
    }
    if (ax >= 0x477ff000u) { /* rounds to >= 2^16: overflow to inf */
        return sign | 0x7c00u;
    }
    if (ax >= 0x38800000u) { /* normal range of binary16 */
        uint32_t m   = ax - 0x38000000u; /* rebias 127 -> 15 */
        uint32_t rnd = m & 0x1fffu;
        m >>= 13;
        if (rnd > 0x1000u || (rnd == 0x1000u && (m & 1u))) {
            m++; /* carry into the exponent is the right answer */
        }
        return sign | (uint16_t)m;
    }
    if (ax < 0x33000000u) { /* < 2^-25: rounds to zero (2^-25 ties to even 0) */
        return sign;
    }
    { /* subnormal result: value = man24 * 2^(e-150), want units of 2^-24 */
        const uint32_t e     = ax >> 23;
        const uint32_t man24 = (ax & 0x7fffffu) | 0x800000u;
        const uint32_t shift = 126u - e; /* 14 .. 24 */
        uint32_t       m     = man24 >> shift;
        const uint32_t rem   = man24 & ((1u << shift) - 1u);
        const uint32_t half  = 1u << (shift - 1);
        if (rem > half || (rem == half && (m & 1u))) {
            m++;
        }
        return sign | (uint16_t)m;
    }
}

/* binary16 operators: compute in binary32 and round once.  For + and * of
 * two binary16 values the binary32 result is exact or rounds innocuously
 * (24 >= 2*11+2 significand bits), so this equals a native half operation.
 * MAX/MIN compare the values and hand back the chosen operand's bits. */
#define HALF_ARITH(name, expr)                                                 \
    static void loop_f16_##name(const void *a_, const void *b_, void *d_,      \
                                size_t n)                                      \
    {                                                                          \
        const uint16_t *a = (const uint16_t *)a_;                              \
        const uint16_t *b = (const uint16_t *)b_;                              \
        uint16_t       *d = (uint16_t *)d_;                                    \
        for (size_t i = 0; i < n; i++) {                                       \
            const float x = oracle_half_to_float(a[i]);                        \
            const float y = oracle_half_to_float(b[i]);                        \
            d[i] = (expr);                                                     \
        }                                                                      \
    }
HALF_ARITH(F_MAX, (x > y ? a[i] : b[i]))
HALF_ARITH(F_MIN, (x < y ? a[i] : b[i]))
HALF_ARITH(F_SUM, oracle_float_to_half(x + y))
HALF_ARITH(F_PROD, oracle_float_to_half(x * y))

/* ---- selection: reduce.h:32-92, 113-140 ---------------------------------- */
typedef void (*loop_fn)(const void *, const void *, void *, size_t);

#define INT_ROW(tag)                                                           \
    { loop_##tag##_F_MAX, loop_##tag##_F_MIN, loop_##tag##_F_SUM,              \
      loop_##tag##_F_PROD, loop_##tag##_F_LAND, loop_##tag##_F_LOR,            \
      loop_##tag##_F_LXOR, loop_##tag##_F_BAND, loop_##tag##_F_BOR,            \
      loop_##tag##_F_BXOR }
#define FP_ROW(tag)                                                            \
    { loop_##tag##_F_MAX, loop_##tag##_F_MIN, loop_##tag##_F_SUM,              \
      loop_##tag##_F_PROD, 0, 0, 0, 0, 0, 0 }

/* column order of the rows above */
static int op_column(int op)
{
    switch (op) {
    case OP_MAX:  return 0;
    case OP_MIN:  return 1;
    case OP_SUM:  return 2;
    case OP_PROD: return 3;
    case OP_LAND: return 4;
    case OP_LOR:  return 5;
    case OP_LXOR: return 6;
    case OP_BAND: return 7;
    case OP_BOR:  return 8;
    case OP_BXOR: return 9;
    default:      return -1;
    }
}

static const loop_fn *dtype_row(int dtype, int *is_fp, size_t *esize)
{
    static const loop_fn i8[10] = INT_ROW(i8), i16[10] = INT_ROW(i16),
                         i32[10] = INT_ROW(i32), i64[10] = INT_ROW(i64),
                         u8[10] = INT_ROW(u8), u16[10] = INT_ROW(u16),
                         u32[10] = INT_ROW(u32), u64[10] = INT_ROW(u64),
                         f16[10] = FP_ROW(f16), f32[10] = FP_ROW(f32),
                         f64[10] = FP_ROW(f64);
    *is_fp = 0;
    switch (dtype) {
    case DT_I8:  *esize = 1; return i8;
    case DT_I16: *esize = 2; return i16;
    case DT_I32: *esize = 4; return i32;
    case DT_I64: *esize = 8; return i64;
    case DT_U8:  *esize = 1; return u8;
    case DT_U16: *esize = 2; return u16;
    case DT_U32: *esize = 4; return u32;
    case DT_U64: *esize = 8; return u64;
    case DT_F16: *esize = 2; *is_fp = 1; return f16;
    case DT_F32: *esize = 4; *is_fp = 1; return f32;
    case DT_F64: *esize = 8; *is_fp = 1; return f64;
    default:     return 0;
    }
}

int oracle_dtype_in_reference(int dtype)
{
    return dtype == DT_I16 || dtype == DT_I32 || dtype == DT_I64 ||
           dtype == DT_F32 || dtype == DT_F64;
}

int oracle_dt_reduce(const void *sbuf1, const void *sbuf2, void *target,
                     size_t count, int dtype, int op)
{
    int            is_fp;
    size_t         esize;
    const loop_fn *row = dtype_row(dtype, &is_fp, &esize);
    const int      col = op_column(op);

    if (row == 0) {
        return -1; /* reduce.h:135-137 */
    }
    if (col < 0 || row[col] == 0) {
        return is_fp ? -1 : 0; /* reduce.h:87-90 vs the default-less :36-67 */
    }
    row[col](sbuf1, sbuf2, target, count);
    return 0;
}

int oracle_reduce_multi(const void *sbuf1, const void *sbuf2, void *rbuf,
                        size_t count, size_t size, size_t stride, int dtype,
                        int op)
{
    if (size == 0) {
        return 0; /* mem_component.c:129-131 */
    }
    (void)oracle_dt_reduce(sbuf1, sbuf2, rbuf, size, dtype, op);
    for (size_t j = 1; j < count; j++) {
        (void)oracle_dt_reduce((const char *)sbuf2 + stride * j, rbuf, rbuf,
                               size, dtype, op); /* mem_component.c:135-138 */
    }
    return 0;
}

/* ---- threaded form -------------------------------------------------------- */
typedef struct {
    const char *s1, *s2;
    char       *dst;
    size_t      count, size, stride;
    int         dtype, op;
} mt_job;

static void *mt_run(void *p)
{
    mt_job *j = (mt_job *)p;
    oracle_reduce_multi(j->s1, j->s2, j->dst, j->count, j->size, j->stride,
                        j->dtype, j->op);
    return 0;
}

int oracle_reduce_multi_mt(const void *sbuf1, const void *sbuf2, void *rbuf,
                           size_t count, size_t size, size_t stride, int dtype,
                           int op, int nthreads)
{
    int     is_fp;
    size_t  esize = 0;
    if (nthreads < 1) {
        nthreads = 1;
    }
    if (dtype_row(dtype, &is_fp, &esize) == 0 || nthreads == 1 || size < 4096) {
        return oracle_reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride,
                                   dtype, op);
    }
    pthread_t *tid  = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
    mt_job    *jobs = (mt_job *)malloc(sizeof(mt_job) * (size_t)nthreads);
    size_t     per  = (size + (size_t)nthreads - 1) / (size_t)nthreads;
    per             = (per + 63) & ~(size_t)63;
    int started     = 0;
    for (int t = 0; t < nthreads; t++) {
        size_t lo = per * (size_t)t;
        if (lo >= size) {
            break;
        }
        size_t hi = lo + per < size ? lo + per : size;
        jobs[t]   = (mt_job){ (const char *)sbuf1 + lo * esize,
                              (const char *)sbuf2 + lo * esize,
                              (char *)rbuf + lo * esize,
                              count, hi - lo, stride, dtype, op };
        pthread_create(&tid[t], 0, mt_run, &jobs[t]);
        started++;
    }
    for (int t = 0; t < started; t++) {
        pthread_join(tid[t], 0);
    }
    free(tid);
    free(jobs);
    return 0;
}

/* ---- synthetic inputs ------------------------------------------------------ */
uint64_t oracle_splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

typedef struct {
    char    *dst;
    size_t   lo, hi;
    int      dtype, sparse;
    uint64_t base;
} fill_job;

static void *fill_run(void *p)
{
    fill_job *j = (fill_job *)p;
    for (size_t i = j->lo; i < j->hi; i++) {
        const uint64_t x    = oracle_splitmix64(j->base + i);
        const uint64_t y    = oracle_splitmix64(x);
        const uint64_t keep = (j->sparse && (y >> 63)) ? 0 : ~0ull;
        switch (j->dtype) {
        case DT_I8: case DT_U8:
            ((uint8_t *)j->dst)[i] = (uint8_t)(x & keep);
            break;
        case DT_I16: case DT_U16:
            ((uint16_t *)j->dst)[i] = (uint16_t)(x & keep);
            break;
        case DT_I32: case DT_U32:
            ((uint32_t *)j->dst)[i] = (uint32_t)(x & keep);
            break;
        case DT_I64: case DT_U64:
            ((uint64_t *)j->dst)[i] = x & keep;
            break;
        case DT_F16:
            ((uint16_t *)j->dst)[i] =
                oracle_float_to_half((float)(x >> 53) * 0x1p-11f - 0.5f);
            break;
        case DT_F32:
            ((float *)j->dst)[i] = (float)(x >> 40) * 0x1p-23f - 1.0f;
            break;
        case DT_F64: {
            const double u1 = ((double)(x >> 11) + 1.0) * 0x1p-53;
            const double u2 = (double)(y >> 11) * 0x1p-53;
            ((double *)j->dst)[i] =
                sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
            break;
        }
        default:
            break;
        }
    }
    return 0;
}

int oracle_fill(void *dst, size_t count, int dtype, uint64_t seed, uint64_t vec,
                int sparse, int nthreads)
{
    int    is_fp;
    size_t esize;
    if (dtype_row(dtype, &is_fp, &esize) == 0) {
        return -1;
    }
    if (nthreads < 1 || count < 65536) {
        nthreads = 1;
    }
    const uint64_t base = seed * 0x9E3779B97F4A7C15ull + (vec << 40);
    pthread_t     *tid  = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
    fill_job      *jobs = (fill_job *)malloc(sizeof(fill_job) * (size_t)nthreads);
    const size_t   per  = (count + (size_t)nthreads - 1) / (size_t)nthreads;
    int            started = 0;
    for (int t = 0; t < nthreads; t++) {
        const size_t lo = per * (size_t)t;
        if (lo >= count) {
            break;
        }
        jobs[t] = (fill_job){ (char *)dst, lo, lo + per < count ? lo + per : count,
                              dtype, sparse, base };
        if (nthreads == 1) {
            fill_run(&jobs[t]);
        } else {
            pthread_create(&tid[t], 0, fill_run, &jobs[t]);
            started++;
        }
    }
    for (int t = 0; t < started; t++) {
        pthread_join(tid[t], 0);
    }
    free(tid);
    free(jobs);
    return 0;
}
