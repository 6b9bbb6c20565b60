/* Stand-in for UCX's <ucs/datastruct/list.h>.  Test infrastructure. */
#ifndef XCCL_TEST_STUB_UCS_LIST_H_
#define XCCL_TEST_STUB_UCS_LIST_H_
typedef struct ucs_list_link {
    struct ucs_list_link *prev;
    struct ucs_list_link *next;
} ucs_list_link_t;
#endif
