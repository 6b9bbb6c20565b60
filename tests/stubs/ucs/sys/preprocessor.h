/* Stand-in for UCX's <ucs/sys/preprocessor.h>.  Test infrastructure. */
#ifndef XCCL_TEST_STUB_UCS_PREPROCESSOR_H_
#define XCCL_TEST_STUB_UCS_PREPROCESSOR_H_
#define UCS_PP_QUOTE(x) #x
#define UCS_PP_MAKE_STRING(x) UCS_PP_QUOTE(x)
#endif
