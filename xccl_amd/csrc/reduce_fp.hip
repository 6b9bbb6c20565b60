// reduce_fp.hip -- floating-point instantiations of the reduction kernel:
// IEEE binary16 / binary32 / binary64, operators MAX, MIN, SUM, PROD
// (reference src/utils/reduce.h:70-92; binary16 is not in the reference and
// follows the same macros with one round-to-nearest-even per operation,
// which is what a native half add/mul is).
// MAX/MIN stay compare+select (`a > b ? a : b`): the hardware max/min
// instructions order +0/-0 and propagate NaN differently from the ternary.
#include "reduce_kernel.hpp"

namespace xccl_rocm {

template <typename T>
static const KernelEntry *fp_table(int kop)
{
    static const KernelEntry t[4] = {
        make_entry<T, OpMax>(), make_entry<T, OpMin>(),
        make_entry<T, OpSum>(), make_entry<T, OpProd>(),
    };
    return &t[kop];
}

const KernelEntry *lookup_fp(int kop, int bytes)
{
    if (kop < K_MAX || kop > K_PROD) {
        return nullptr;
    }
    switch (bytes) {
    case 2:
        return fp_table<_Float16>(kop);
    case 4:
        return fp_table<float>(kop);
    case 8:
        return fp_table<double>(kop);
    default:
        return nullptr;
    }
}

} // namespace xccl_rocm

// The completion word of a launch too large to count its own workgroups, as
// a second packet behind it on the component's own dispatch queue: one lane
// stores the sequence number once everything queued before has completed
// (the packet carries the barrier bit).  Lives in this unit because the own
// queues load their kernels from the five embedded code objects.
extern "C" __global__ void xccl_rocm_tail_flag_kernel(uint32_t *flag, uint32_t seq)
{
    __hip_atomic_store(flag, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
