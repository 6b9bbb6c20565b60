/* Stand-in for UCX's <ucs/debug/log_def.h>: messages at or above the
 * component's level go to stderr.  Test infrastructure. */
#ifndef XCCL_TEST_STUB_UCS_LOG_DEF_H_
#define XCCL_TEST_STUB_UCS_LOG_DEF_H_
#include <stdio.h>
#include <ucs/config/types.h>
#define ucs_log_component(_level, _comp, _fmt, ...)                                 \
    do {                                                                           \
        if ((int)(_level) <= (int)(_comp)->log_level) {                            \
            fprintf(stderr, "[xccl %d] " _fmt "\n", (int)(_level), ##__VA_ARGS__); \
        }                                                                          \
    } while (0)
#endif
