/* Stand-in for UCX's <ucp/api/ucp.h>: declarations of the tag-matching calls
 * the XCCL UCX team library makes, so that a compiler can check its sources
 * where UCX is not installed.  Nothing is implemented.  Test infrastructure,
 * never part of the product. */
#ifndef XCCL_TEST_STUB_UCP_H_
#define XCCL_TEST_STUB_UCP_H_
#include <stddef.h>
#include <stdint.h>
#include <ucs/memory/memory_type.h>
#include <ucs/type/status.h>

typedef struct ucp_context *ucp_context_h;
typedef struct ucp_worker  *ucp_worker_h;
typedef struct ucp_ep      *ucp_ep_h;
typedef struct ucp_address  ucp_address_t;
typedef uint64_t            ucp_tag_t;
typedef uint64_t            ucp_datatype_t;

typedef struct ucp_tag_recv_info {
    ucp_tag_t sender_tag;
    size_t    length;
} ucp_tag_recv_info_t;

typedef void (*ucp_send_nbx_callback_t)(void *request, ucs_status_t status, void *user_data);
typedef void (*ucp_tag_recv_nbx_callback_t)(void *request, ucs_status_t status,
                                            const ucp_tag_recv_info_t *tag_info, void *user_data);

enum {
    UCP_OP_ATTR_FIELD_CALLBACK    = UCS_BIT(1),
    UCP_OP_ATTR_FIELD_USER_DATA   = UCS_BIT(2),
    UCP_OP_ATTR_FIELD_DATATYPE    = UCS_BIT(3),
    UCP_OP_ATTR_FIELD_MEMORY_TYPE = UCS_BIT(5)
};

typedef struct {
    uint32_t       op_attr_mask;
    uint32_t       flags;
    void          *request;
    union {
        ucp_send_nbx_callback_t     send;
        ucp_tag_recv_nbx_callback_t recv;
    } cb;
    ucp_datatype_t    datatype;
    void             *user_data;
    void             *reply_buffer;
    ucs_memory_type_t memory_type;
} ucp_request_param_t;

enum { UCP_EP_PARAM_FIELD_REMOTE_ADDRESS = UCS_BIT(0) };
enum { UCP_EP_CLOSE_MODE_FORCE = 0, UCP_EP_CLOSE_MODE_FLUSH = 1 };

typedef struct ucp_ep_params {
    uint64_t             field_mask;
    const ucp_address_t *address;
} ucp_ep_params_t;

#define ucp_dt_make_contig(_elem_size) (((ucp_datatype_t)(_elem_size) << 3) | 0)

ucs_status_ptr_t ucp_tag_send_nbx(ucp_ep_h ep, const void *buffer, size_t count, ucp_tag_t tag,
                                  const ucp_request_param_t *param);
ucs_status_ptr_t ucp_tag_recv_nbx(ucp_worker_h worker, void *buffer, size_t count, ucp_tag_t tag,
                                  ucp_tag_t tag_mask, const ucp_request_param_t *param);
void             ucp_request_cancel(ucp_worker_h worker, void *request);
void             ucp_request_free(void *request);
ucs_status_t     ucp_request_check_status(void *request);
unsigned         ucp_worker_progress(ucp_worker_h worker);
ucs_status_t     ucp_ep_create(ucp_worker_h worker, const ucp_ep_params_t *params, ucp_ep_h *ep_p);
ucs_status_ptr_t ucp_ep_close_nb(ucp_ep_h ep, unsigned mode);
#endif
