/* Stand-in for UCX's <ucs/sys/compiler_def.h>: only what the XCCL files
 * under test use.  Test infrastructure, never part of the product. */
#ifndef XCCL_TEST_STUB_UCS_COMPILER_DEF_H_
#define XCCL_TEST_STUB_UCS_COMPILER_DEF_H_
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
#define BEGIN_C_DECLS extern "C" {
#define END_C_DECLS }
#else
#define BEGIN_C_DECLS
#define END_C_DECLS
#endif
#define UCS_BIT(i) (1ul << (i))
#define UCS_MASK(i) (UCS_BIT(i) - 1)
#define UCS_S_PACKED __attribute__((packed))
#define UCS_F_ALWAYS_INLINE inline __attribute__((always_inline))
#define ucs_likely(x) __builtin_expect(!!(x), 1)
#define ucs_unlikely(x) __builtin_expect(!!(x), 0)
#define ucs_container_of(_ptr, _type, _member) ((_type *)((char *)(_ptr)-offsetof(_type, _member)))
#define ucs_derived_of(_ptr, _type) ((_type *)(_ptr))
#define ucs_offsetof(_type, _member) offsetof(_type, _member)
#define ucs_static_array_size(_a) (sizeof(_a) / sizeof((_a)[0]))
#endif
