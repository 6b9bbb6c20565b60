/* Stand-in for UCX v1.10's <ucs/memory/memory_type.h> (the UCX version the
 * XCCL tree's CI pins): enumerators and their order as published there.
 * Test infrastructure. */
#ifndef XCCL_TEST_STUB_UCS_MEMORY_TYPE_H_
#define XCCL_TEST_STUB_UCS_MEMORY_TYPE_H_
#include <ucs/sys/compiler_def.h>
typedef enum ucs_memory_type {
    UCS_MEMORY_TYPE_HOST,
    UCS_MEMORY_TYPE_CUDA,
    UCS_MEMORY_TYPE_CUDA_MANAGED,
    UCS_MEMORY_TYPE_ROCM,
    UCS_MEMORY_TYPE_ROCM_MANAGED,
    UCS_MEMORY_TYPE_LAST,
    UCS_MEMORY_TYPE_UNKNOWN = UCS_MEMORY_TYPE_LAST
} ucs_memory_type_t;
extern const char *ucs_memory_type_names[];
#endif
