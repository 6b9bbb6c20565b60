// reduce_w32.hip -- 32-bit integer instantiations of the reduction kernel.
// SUM, PROD, the logical and the bitwise operators give the same bits for
// int32_t and uint32_t, so they are built once, on the unsigned type;
// MAX and MIN are built for both.
// Bitwise operators are served by the 8-bit unit for every width.
#include "reduce_kernel.hpp"

namespace xccl_rocm {

const KernelEntry *lookup_w32(int kop, bool is_signed)
{
    typedef uint32_t U;
    typedef int32_t  S;
    static const KernelEntry common[K_COUNT] = {
        make_entry<U, OpMax>(),  make_entry<U, OpMin>(),  make_entry<U, OpSum>(),
        make_entry<U, OpProd>(), make_entry<U, OpLand>(), make_entry<U, OpLor>(),
        make_entry<U, OpLxor>(),
    };
    static const KernelEntry smax = make_entry<S, OpMax>();
    static const KernelEntry smin = make_entry<S, OpMin>();
    if (kop < 0 || kop >= K_BAND) {
        return nullptr;
    }
    if (is_signed && kop == K_MAX) {
        return &smax;
    }
    if (is_signed && kop == K_MIN) {
        return &smin;
    }
    return &common[kop];
}

} // namespace xccl_rocm
