/* Stand-in for UCX's <ucs/config/parser.h>: the types the XCCL headers
 * mention, no parser.  Test infrastructure. */
#ifndef XCCL_TEST_STUB_UCS_CONFIG_PARSER_H_
#define XCCL_TEST_STUB_UCS_CONFIG_PARSER_H_
#include <ucs/config/types.h>
#include <ucs/datastruct/list.h>
typedef struct ucs_config_field {
    const char *name;
    const char *dfl_value;
    const char *doc;
    size_t      offset;
    struct {
        int         kind;
        const void *arg;
    } parser;
} ucs_config_field_t;
#define UCS_CONFIG_TYPE_BOOL {1, NULL}
#define UCS_CONFIG_TYPE_UINT {2, NULL}
#define UCS_CONFIG_TYPE_STRING_ARRAY {3, NULL}
#define UCS_CONFIG_TYPE_ENUM(_names) {4, (_names)}
#define UCS_CONFIG_TYPE_TABLE(_table) {5, (_table)}
typedef struct ucs_config_global_list_entry {
    const char         *name;
    const char         *prefix;
    ucs_config_field_t *table;
    size_t              size;
    ucs_list_link_t     list;
} ucs_config_global_list_entry_t;
#endif
