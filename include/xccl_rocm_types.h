/*
 * xccl_rocm_types.h -- the XCCL types that cross the mem-component boundary.
 *
 * A build inside the XCCL tree defines XCCL_MC_ROCM_IN_TREE and gets these
 * types from XCCL's and UCX's own headers.  A standalone build (this
 * repository: no UCX installed) gets value-identical definitions from here.
 * Every numeric value below is part of the binary contract with libxccl and
 * its team libraries and must not change:
 *
 *   xccl_op_t      reference src/api/xccl.h:371-389
 *   xccl_dt_t      reference src/api/xccl.h:391-407
 *   xccl_dt_size   reference src/api/xccl.h:478-502
 *   xccl_stream_t  reference src/api/xccl.h:439-446
 *   xccl_status_t  reference src/api/xccl_status.h:10-30
 *   ucs_memory_type_t  UCX v1.10 ucs/memory/memory_type.h (the UCX version
 *                      the reference's CI pins, .github/workflows/main.yml:9)
 */
#ifndef XCCL_ROCM_TYPES_H_
#define XCCL_ROCM_TYPES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef XCCL_MC_ROCM_IN_TREE
#include <api/xccl.h>
#include <ucs/memory/memory_type.h>
#else

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    XCCL_OK                    = 0,
    XCCL_INPROGRESS            = 1,
    XCCL_ERR_NO_MESSAGE        = -1,
    XCCL_ERR_NO_RESOURCE       = -2,
    XCCL_ERR_NO_MEMORY         = -4,
    XCCL_ERR_INVALID_PARAM     = -5,
    XCCL_ERR_UNREACHABLE       = -6,
    XCCL_ERR_NOT_IMPLEMENTED   = -8,
    XCCL_ERR_MESSAGE_TRUNCATED = -9,
    XCCL_ERR_NO_PROGRESS       = -10,
    XCCL_ERR_BUFFER_TOO_SMALL  = -11,
    XCCL_ERR_NO_ELEM           = -12,
    XCCL_ERR_UNSUPPORTED       = -22,
    XCCL_ERR_LAST              = -100
} xccl_status_t;

typedef enum {
    XCCL_OP_MAX             = 0,
    XCCL_OP_MIN             = 1,
    XCCL_OP_SUM             = 2,
    XCCL_OP_PROD            = 3,
    XCCL_OP_AND             = 4,
    XCCL_OP_OR              = 5,
    XCCL_OP_XOR             = 6,
    XCCL_OP_LAND            = 7,
    XCCL_OP_LOR             = 8,
    XCCL_OP_LXOR            = 9,
    XCCL_OP_BAND            = 10,
    XCCL_OP_BOR             = 11,
    XCCL_OP_BXOR            = 12,
    XCCL_OP_MAXLOC          = 13,
    XCCL_OP_MINLOC          = 14,
    XCCL_OP_LAST_PREDEFINED = 15,
    XCCL_OP_UNSUPPORTED     = 16
} xccl_op_t;

typedef enum {
    XCCL_DT_INT8            = 0,
    XCCL_DT_INT16           = 1,
    XCCL_DT_INT32           = 2,
    XCCL_DT_INT64           = 3,
    XCCL_DT_INT128          = 4,
    XCCL_DT_UINT8           = 5,
    XCCL_DT_UINT16          = 6,
    XCCL_DT_UINT32          = 7,
    XCCL_DT_UINT64          = 8,
    XCCL_DT_UINT128         = 9,
    XCCL_DT_FLOAT16         = 10,
    XCCL_DT_FLOAT32         = 11,
    XCCL_DT_FLOAT64         = 12,
    XCCL_DT_LAST_PREDEFINED = 13,
    XCCL_DT_UNSUPPORTED     = 14
} xccl_dt_t;

/* Bytes per element; 0 for anything that is not a predefined datatype. */
static inline size_t xccl_dt_size(xccl_dt_t dt)
{
    static const unsigned char bytes[XCCL_DT_LAST_PREDEFINED] = {
        1, 2, 4, 8, 16, /* INT8..INT128   */
        1, 2, 4, 8, 16, /* UINT8..UINT128 */
        2, 4, 8         /* FLOAT16/32/64  */
    };
    return ((unsigned)dt < (unsigned)XCCL_DT_LAST_PREDEFINED) ? bytes[dt] : 0;
}

/*
 * Stream handle as XCCL passes it around: `stream` points AT the caller's
 * runtime stream handle (the reference dereferences it as
 * *(cudaStream_t*)stream->stream, src/utils/cuda/cuda_mem_component.c:155).
 * XCCL_STREAM_TYPE_ROCM is the value this component adds; `stream` then
 * points at a hipStream_t.
 */
typedef enum {
    XCCL_STREAM_TYPE_CUDA = 0,
    XCCL_STREAM_TYPE_ROCM = 1,
    XCCL_STREAM_TYPE_LAST
} xccl_stream_type_t;

typedef struct xccl_stream {
    xccl_stream_type_t type;
    void              *stream;
} xccl_stream_t;

typedef enum ucs_memory_type {
    UCS_MEMORY_TYPE_HOST         = 0,
    UCS_MEMORY_TYPE_CUDA         = 1,
    UCS_MEMORY_TYPE_CUDA_MANAGED = 2,
    UCS_MEMORY_TYPE_ROCM         = 3,
    UCS_MEMORY_TYPE_ROCM_MANAGED = 4,
    UCS_MEMORY_TYPE_LAST         = 5
} ucs_memory_type_t;

#ifdef __cplusplus
}
#endif

#endif /* XCCL_MC_ROCM_IN_TREE */
#endif /* XCCL_ROCM_TYPES_H_ */
