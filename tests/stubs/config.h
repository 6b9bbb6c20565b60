/* Stand-in for the config.h that the XCCL tree's configure step generates.
 * Test infrastructure: lets a compiler check the patched XCCL sources where
 * autotools have not run.  Nothing in the product includes it. */
#ifndef XCCL_TEST_STUB_CONFIG_H_
#define XCCL_TEST_STUB_CONFIG_H_
#ifndef _GNU_SOURCE
#define _GNU_SOURCE 1
#endif
#define XCCL_TEST_STUB_HEADERS 1
#endif
