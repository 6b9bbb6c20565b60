/* Stand-in for UCX's <ucs/type/status.h>: the codes and pointer-status
 * helpers the XCCL UCX team library uses.  Test infrastructure. */
#ifndef XCCL_TEST_STUB_UCS_STATUS_H_
#define XCCL_TEST_STUB_UCS_STATUS_H_
#include <stdint.h>
typedef enum {
    UCS_OK             = 0,
    UCS_INPROGRESS     = 1,
    UCS_ERR_NO_MESSAGE = -1,
    UCS_ERR_LAST       = -100
} ucs_status_t;
typedef void *ucs_status_ptr_t;
#define UCS_PTR_IS_ERR(_ptr) (((uintptr_t)(_ptr)) >= ((uintptr_t)UCS_ERR_LAST))
#define UCS_PTR_IS_PTR(_ptr) (((uintptr_t)(_ptr)-1) < ((uintptr_t)UCS_ERR_LAST - 1))
#define UCS_PTR_STATUS(_ptr) ((ucs_status_t)(intptr_t)(_ptr))
const char *ucs_status_string(ucs_status_t status);
#endif
