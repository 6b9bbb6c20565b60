/*
 * xccl_oracle.h -- CPU restatement of XCCL's host reduction path.
 *
 * TEST INFRASTRUCTURE, NOT PRODUCT.  Nothing under xccl_amd/ or include/
 * links, loads or calls this; it is the checker for the GPU path (tests,
 * the smoke check) and the CPU leg that the benchmark times next to the GPU.
 *
 * Datatype / operator / status numbers are those of include/xccl_rocm_types.h
 * (reference src/api/xccl.h:371-407), passed as plain ints.
 */
#ifndef XCCL_ORACLE_H_
#define XCCL_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 1 if reference src/utils/reduce.h:113-140 itself implements this dtype
 * (INT16, INT32, INT64, FLOAT32, FLOAT64), 0 for the dtypes this oracle adds
 * by instantiating the same operator macros (INT8, UINT8..UINT64, FLOAT16). */
int oracle_dtype_in_reference(int dtype);

/* reduce.h:113-140.  target[i] = OP(sbuf1[i], sbuf2[i]), i ascending.
 * Returns 0, or -1 for an unsupported dtype or a floating-point dtype with a
 * logical/bitwise operator.  For an integer dtype, an operator outside the
 * ten implemented ones leaves target untouched and returns 0, as the
 * reference's default-less switch does (reduce.h:36-67). */
int oracle_dt_reduce(const void *sbuf1, const void *sbuf2, void *target,
                     size_t count, int dtype, int op);

/* Host branch of xccl_mem_component_reduce_multi, mem_component.c:122-148:
 * size == 0 -> nothing; rbuf = OP(sbuf1, sbuf2{0}); then for j = 1..count-1
 * rbuf = OP(sbuf2{j}, rbuf) -- the new source is the FIRST operand.  One full
 * pass over rbuf per source; the inner status is dropped; always returns 0
 * (XCCL_OK). */
int oracle_reduce_multi(const void *sbuf1, const void *sbuf2, void *rbuf,
                        size_t count, size_t size, size_t stride, int dtype,
                        int op);

/* The same fold applied to `nthreads` disjoint contiguous element ranges,
 * one per thread; bit-identical to oracle_reduce_multi. */
int oracle_reduce_multi_mt(const void *sbuf1, const void *sbuf2, void *rbuf,
                           size_t count, size_t size, size_t stride, int dtype,
                           int op, int nthreads);

/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept. */
float    oracle_half_to_float(uint16_t h);
uint16_t oracle_float_to_half(float f);

/* Synthetic inputs: element i of vector `vec` of stream `seed` is a pure
 * function of (seed, vec, i):
 *   x = splitmix64(seed*0x9E3779B97F4A7C15 + (vec<<40) + i), y = splitmix64(x)
 *   FLOAT32 (x>>40)*2^-23 - 1; FLOAT16 (x>>53)*2^-11 - 0.5;
 *   FLOAT64 Box-Muller normal(0,1) from x, y; integers: low bits of x, zeroed
 *   when `sparse` and bit 63 of y is set.
 * Fills dst[0..count) using `nthreads` threads.  Returns 0 / -1 (dtype). */
int oracle_fill(void *dst, size_t count, int dtype, uint64_t seed, uint64_t vec,
                int sparse, int nthreads);

uint64_t oracle_splitmix64(uint64_t z);

#ifdef __cplusplus
}
#endif
#endif
