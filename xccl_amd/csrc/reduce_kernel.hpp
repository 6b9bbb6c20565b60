// reduce_kernel.hpp -- the one gfx950 kernel template behind reduce and
// reduce_multi, and the per-(type, op) table entries built from it.
//
// What it computes (reference src/utils/mem_component.c:133-139 for the fold,
// src/utils/reduce.h:14-23 for the operators):
//     acc = OP(sbuf1[i], sbuf2{0}[i]);  acc = OP(sbuf2{j}[i], acc), j = 1..n-1
//     rbuf[i] = acc
// The reference's CUDA kernel (xccl_cuda_reduce_multi.cu:17-40) keeps acc in
// global memory and reads 2/4/8 bytes per lane; here every lane moves 16 bytes
// per source with one global_load_dwordx4, all sources of a tile are in flight
// before the first fold, and acc never leaves registers.
//
// Shape, from measurement on MI355X (fp32 SUM, 8 x 256 MiB): one-wave
// workgroups, one tile per workgroup (a grid as large as the tile count; the
// grid-stride loop only runs when that exceeds the grid cap) beat 256-lane
// persistent workgroups by ~25%; streaming cache policy (non-temporal loads,
// system-scope write-through stores) beats default-policy accesses by ~17%;
// holding the workgroups resident per compute unit to about ten (the launch
// asks for LDS it never touches) adds 4-12%: the memory side is saturated
// long before the wave slots are, and fewer waves in flight keep the
// addresses being served close together.
//
// Layout of one call, in elements of T:
//     [0, head)                 peeled so that the vector body starts on a
//                               16-byte boundary of the buffer chosen by the
//                               host (fewer than 16/sizeof(T) elements)
//     [head, head + nvec*VE)    nvec 16-byte vectors, VE = 16/sizeof(T)
//     [.., .. + tail)           fewer than VE elements
// Head and tail are folded element-wise by the first lanes of the last block.
// Vector accesses are emitted as dwordx4 whatever the address is (the device
// runs in unaligned access mode), so a source whose alignment differs from
// the peeled one costs extra cache-line touches, never correctness.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xccl_rocm {

constexpr int kBlock = 64; // one wavefront per workgroup

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_u __attribute__((aligned(1)));

constexpr uint32_t kDoneShards = 64; // second-level arrival counters of a completion word
constexpr uint32_t kDoneStride = 32; // uint32 words between counters: one per 128-byte line

struct ReduceArgs {
    const char *s1;     // sbuf1, at the first byte of the vector body (head elements lie before it)
    const char *s2;     // sbuf2 (vector 0), likewise
    char       *dst;    // rbuf / target, likewise
    size_t      stride; // bytes between vectors of sbuf2
    size_t      head;   // elements before the vector body
    size_t      nvec;   // 16-byte vectors in the body
    size_t      tail;   // elements after the vector body
    uint32_t    n2;     // vectors in sbuf2 (>= 1)
    // Completion word (small launches only; all NULL/0 otherwise): when the last workgroup
    // is through, done_seq is stored to *done_flag, a host-mapped word the caller polls.
    uint32_t    done_seq;
    uint32_t   *done_count; // device words (1 + kDoneShards, kDoneStride apart), zero between launches
    uint32_t   *done_flag;
};

// ---- operators: reduce.h:14-23, first macro argument = a ------------------
// Integer kernels run on unsigned types wherever the result bits do not
// depend on signedness (SUM, PROD, logical, bitwise), which also makes
// wrap-around defined; MIN/MAX are instantiated for both signednesses.
struct OpMax  { template <class T> static __device__ __forceinline__ T f(T a, T b) { return a > b ? a : b; } };
struct OpMin  { template <class T> static __device__ __forceinline__ T f(T a, T b) { return a < b ? a : b; } };
struct OpSum  { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a + b); } };
struct OpProd { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a * b); } };
struct OpLand { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a && b); } };
struct OpLor  { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a || b); } };
struct OpLxor { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)((!a) != (!b)); } };
struct OpBand { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a & b); } };
struct OpBor  { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a | b); } };
struct OpBxor { template <class T> static __device__ __forceinline__ T f(T a, T b) { return (T)(a ^ b); } };

// uint16 * uint16 promotes to (signed) int and can overflow it; multiply in
// 32-bit unsigned and truncate, which is what the promoted product's low bits
// are.
template <> __device__ __forceinline__ uint16_t OpProd::f<uint16_t>(uint16_t a, uint16_t b)
{
    return (uint16_t)((uint32_t)a * (uint32_t)b);
}

template <typename T> struct Vec {
    static constexpr int n = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};

template <typename T, class Op>
__device__ __forceinline__ u32x4 vfold(u32x4 a, u32x4 b)
{
    typedef typename Vec<T>::type V;
    V x = __builtin_bit_cast(V, a);
    V y = __builtin_bit_cast(V, b);
    V r;
#pragma unroll
    for (int k = 0; k < Vec<T>::n; ++k) {
        r[k] = Op::template f<T>(x[k], y[k]);
    }
    return __builtin_bit_cast(u32x4, r);
}

// Bitwise operators do not care where element boundaries are.
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpBand>(u32x4 a, u32x4 b) { return a & b; }
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpBor>(u32x4 a, u32x4 b)  { return a | b; }
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpBxor>(u32x4 a, u32x4 b) { return a ^ b; }

// Cache policy of the vector accesses.
//   POL_PLAIN   default loads and stores.
//   POL_STREAM  sources are read once: non-temporal loads.  The result is
//               about to be read by another agent (the NIC sending it, the
//               next round's kernel): stores carry system scope (sc0 sc1),
//               i.e. write through instead of lingering dirty in L2.
enum { POL_PLAIN = 0, POL_STREAM = 1 };

// Vector accesses are addressed as (uniform 64-bit base) + (32-bit lane
// offset): the base lives in scalar registers, one VGPR serves every access of
// a tile, and a wave gets from its first instruction to its first load in a
// few cycles -- with one tile per wave, the prologue is part of every tile.
template <int POL>
__device__ __forceinline__ u32x4 vload(const char *base, uint32_t off)
{
    if (POL == POL_STREAM) {
        return __builtin_nontemporal_load((const u32x4_u *)(base + off));
    }
    return *(const u32x4_u *)(base + off);
}

template <int POL>
__device__ __forceinline__ void vstore(char *base, uint32_t off, u32x4 v)
{
    if (POL == POL_STREAM) {
        // No builtin emits a 16-byte store with these scope bits, hence asm --
        // and asm the compiler's hazard recogniser cannot see into, so the
        // statement has to be hazard-free by construction:
        //  * it takes its address as a 64-bit VGPR pair, never a scalar base:
        //    a VMEM instruction that reads an SGPR within 5 wait states of a
        //    VALU write to it (v_readlane restoring a spilled SGPR does that)
        //    sees the old value, i.e. a wild address;
        //  * it ends in s_nop: gfx9 reads the data registers of a store wider
        //    than 8 bytes one cycle after issue, and a VALU write to them in
        //    the next slot corrupts the stored value.
        // A store has no result register, so the compiler's s_waitcnt
        // bookkeeping stays valid; the clobber keeps it ordered after the loads.
        char *p = base + off;
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
    } else {
        *(u32x4_u *)(base + off) = v;
    }
}

template <typename T>
__device__ __forceinline__ T eload(const char *p)
{
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

// One element, all sources, in fold order.  `rel`: byte offset of the element
// from the start of the vector body (negative in the head).
template <typename T, class Op>
__device__ __forceinline__ void fold_element(const ReduceArgs &a, ptrdiff_t rel)
{
    T acc = Op::template f<T>(eload<T>(a.s1 + rel), eload<T>(a.s2 + rel));
    for (uint32_t j = 1; j < a.n2; ++j) {
        acc = Op::template f<T>(eload<T>(a.s2 + (size_t)j * a.stride + rel), acc);
    }
    __builtin_memcpy(a.dst + rel, &acc, sizeof(T));
}

// One tile = UNROLL x kBlock vectors; lane t of the block owns vectors
// v0 + u*kBlock + t.  NSRC > 0: exactly NSRC sources, all NSRC*UNROLL loads
// issued before the first fold.  NSRC == 0: any number of sources, loaded four
// at a time.  GUARD: the tile may run past nvec.
template <typename T, class Op, int NSRC, int UNROLL, int POL, bool GUARD>
__device__ __forceinline__ void fold_tile(const ReduceArgs &a, size_t v0)
{
    const size_t tile_off = v0 * 16; // uniform: same for every lane of the workgroup
    const char  *p1       = a.s1 + tile_off;
    const char  *p2       = a.s2 + tile_off;
    char        *pd       = a.dst + tile_off;
    uint32_t     off[UNROLL];
    bool         live[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        off[u]  = (uint32_t)(u * kBlock + (int)threadIdx.x) * 16u;
        live[u] = !GUARD || v0 + (size_t)u * kBlock + threadIdx.x < a.nvec;
    }

    if constexpr (NSRC > 0) {
        constexpr int N = NSRC;
        u32x4         r[UNROLL][N];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (live[u]) {
                r[u][0] = vload<POL>(p1, off[u]);
#pragma unroll
                for (int j = 1; j < N; ++j) {
                    r[u][j] = vload<POL>(p2 + (size_t)(j - 1) * a.stride, off[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (live[u]) {
                u32x4 acc = vfold<T, Op>(r[u][0], r[u][1]);
#pragma unroll
                for (int j = 2; j < N; ++j) {
                    acc = vfold<T, Op>(r[u][j], acc);
                }
                vstore<POL>(pd, off[u], acc);
            }
        }
    } else {
        u32x4 acc[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (live[u]) {
                u32x4 x = vload<POL>(p1, off[u]);
                u32x4 y = vload<POL>(p2, off[u]);
                acc[u]  = vfold<T, Op>(x, y);
            }
        }
        uint32_t j = 1;
        for (; j + 4 <= a.n2; j += 4) {
            const char *p = p2 + (size_t)j * a.stride;
            u32x4       r[UNROLL][4];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (live[u]) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        r[u][k] = vload<POL>(p + (size_t)k * a.stride, off[u]);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (live[u]) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        acc[u] = vfold<T, Op>(r[u][k], acc[u]);
                    }
                }
            }
        }
        for (; j < a.n2; ++j) {
            const char *p = p2 + (size_t)j * a.stride;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (live[u]) {
                    acc[u] = vfold<T, Op>(vload<POL>(p, off[u]), acc[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (live[u]) {
                vstore<POL>(pd, off[u], acc[u]);
            }
        }
    }
}

// Tells the host that the launch is complete without going through the queue's
// completion signal (which costs ~4 us more than the kernel's own store on this
// part).  Every workgroup -- one wave -- waits until its own result stores have
// completed, then counts itself in; the last one to arrive publishes the
// sequence number and re-arms the counter.
//   Streaming policy: the vector stores are system-scope write-through, so
//   "completed" already means "in memory"; a wave only needs its vmcnt to
//   drain (a workgroup-scope release) before it counts itself in.  Stores made
//   with default policy (`wrote_plain`: the element-wise head/tail, or every
//   store under POL_PLAIN) sit dirty in this XCD's L2 and need the wave's own
//   system-scope release, which writes that L2 back.
// One contended atomic per workgroup: for small grids only.
template <int POL>
__device__ __forceinline__ void publish_completion(const ReduceArgs &a, bool wrote_plain)
{
    if (POL != POL_STREAM || wrote_plain) {
        __threadfence_system();
    } else {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    }
    if (threadIdx.x == 0) {
        // Arrival counting in two levels, so that no single word takes more than
        // grid/kDoneShards increments: workgroup b counts into shard b % shards, the
        // wave that fills a shard counts into word 0, the wave that fills word 0 is
        // the last.  atomicInc wraps to zero at its bound, so every word is back at
        // zero by itself when the launch is over.  Words are kDoneStride apart
        // (one per 128-byte line): [0] top, [1 + s] shard s.
        const uint32_t grid   = gridDim.x;
        const uint32_t shards = grid < kDoneShards ? grid : kDoneShards;
        bool           last   = true;
        if (grid > kDoneShards) {
            const uint32_t sh    = blockIdx.x % kDoneShards;
            const uint32_t total = grid / kDoneShards + (sh < grid % kDoneShards ? 1u : 0u);
            last = atomicInc(a.done_count + (1 + sh) * kDoneStride, total - 1) == total - 1;
        }
        if (last && grid > 1) {
            last = atomicInc(a.done_count, shards - 1) == shards - 1;
        }
        if (last) {
            __hip_atomic_store(a.done_flag, a.done_seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

template <typename T, class Op, int NSRC, int UNROLL, int POL>
__global__ void __launch_bounds__(kBlock) reduce_multi_kernel(const ReduceArgs a)
{
    constexpr size_t tile = (size_t)kBlock * UNROLL;
    const size_t     step = (size_t)gridDim.x * tile;
    size_t           v0   = (size_t)blockIdx.x * tile;

    // Fetch the completion-word pointer together with the other arguments: left
    // alone, its scalar load sinks below the stores and the wave waits for it
    // there instead of retiring.
    uint32_t *const done_flag = a.done_flag;
    asm volatile("" : : "s"(done_flag));

    // Head and tail first: they use ordinary loads and stores, whose completion
    // the compiler tracks.  The tiles end in asm stores it cannot see; anything
    // it had to order after them (a loop back-edge, say) would make it wait for
    // every outstanding store, and the wave would sit on its slot for a
    // write-through round trip instead of retiring.
    const bool edges = blockIdx.x == gridDim.x - 1 && a.head + a.tail != 0;
    if (edges) {
        const size_t t = threadIdx.x;
        if (t < a.head) {
            fold_element<T, Op>(a, -(ptrdiff_t)((a.head - t) * sizeof(T)));
        } else if (t - a.head < a.tail) {
            fold_element<T, Op>(a, (ptrdiff_t)(a.nvec * 16 + (t - a.head) * sizeof(T)));
        }
    }
    if (step >= a.nvec) {
        // the usual launch: at most one tile per workgroup, straight-line code
        if (v0 < a.nvec) {
            if (v0 + tile <= a.nvec) {
                fold_tile<T, Op, NSRC, UNROLL, POL, false>(a, v0);
            } else {
                fold_tile<T, Op, NSRC, UNROLL, POL, true>(a, v0);
            }
        }
    } else {
        // more tiles than the grid cap allows workgroups: loop
        for (; v0 < a.nvec; v0 += step) {
            if (v0 + tile <= a.nvec) {
                fold_tile<T, Op, NSRC, UNROLL, POL, false>(a, v0);
            } else {
                fold_tile<T, Op, NSRC, UNROLL, POL, true>(a, v0);
            }
        }
    }
    if (done_flag != nullptr) {
        publish_completion<POL>(a, edges);
    }
}

// ---- table of instantiations ---------------------------------------------
// Source-count variants: exact counts for the radices the k-nomial and
// scatter-reduce steps use (2, 3, 4, 8, 16 sources), and the any-count kernel.
enum { NV_ANY = 0, NV_2, NV_3, NV_4, NV_8, NV_16, NV_COUNT };

constexpr int nsrc_of(int nv) { return nv == NV_2 ? 2 : nv == NV_3 ? 3 : nv == NV_4 ? 4 : nv == NV_8 ? 8 : nv == NV_16 ? 16 : 0; }
// vectors per lane per tile: two -- with the resident-workgroup cap, two tiles
// per wave measured best for 2, 4, 8 and 16 sources alike -- except 16 sources
// of 8-bit elements, where 32 vectors in flight plus the unpacked bytes do not
// fit the register file and the compiler would spill to scratch memory
constexpr int unroll_of(int nv, int esize) { return (nv == NV_16 && esize == 1) ? 1 : 2; }

struct KernelEntry {
    const void *fn[2][NV_COUNT]; // [cache policy][variant]
    int         elem_size;       // sizeof(T) the kernel folds in
};

template <typename T, class Op, int POL, int NV>
constexpr const void *kernel_ptr()
{
    return (const void *)&reduce_multi_kernel<T, Op, nsrc_of(NV), unroll_of(NV, (int)sizeof(T)), POL>;
}

template <typename T, class Op>
KernelEntry make_entry()
{
    KernelEntry e;
    e.fn[0][NV_ANY] = kernel_ptr<T, Op, POL_PLAIN, NV_ANY>();
    e.fn[0][NV_2]   = kernel_ptr<T, Op, POL_PLAIN, NV_2>();
    e.fn[0][NV_3]   = kernel_ptr<T, Op, POL_PLAIN, NV_3>();
    e.fn[0][NV_4]   = kernel_ptr<T, Op, POL_PLAIN, NV_4>();
    e.fn[0][NV_8]   = kernel_ptr<T, Op, POL_PLAIN, NV_8>();
    e.fn[0][NV_16]  = kernel_ptr<T, Op, POL_PLAIN, NV_16>();
    e.fn[1][NV_ANY] = kernel_ptr<T, Op, POL_STREAM, NV_ANY>();
    e.fn[1][NV_2]   = kernel_ptr<T, Op, POL_STREAM, NV_2>();
    e.fn[1][NV_3]   = kernel_ptr<T, Op, POL_STREAM, NV_3>();
    e.fn[1][NV_4]   = kernel_ptr<T, Op, POL_STREAM, NV_4>();
    e.fn[1][NV_8]   = kernel_ptr<T, Op, POL_STREAM, NV_8>();
    e.fn[1][NV_16]  = kernel_ptr<T, Op, POL_STREAM, NV_16>();
    e.elem_size     = (int)sizeof(T);
    return e;
}

// Operator slots of a per-type table.
enum { K_MAX = 0, K_MIN, K_SUM, K_PROD, K_LAND, K_LOR, K_LXOR, K_BAND, K_BOR, K_BXOR, K_COUNT };

// One translation unit per element width keeps the build parallel.  Each
// returns NULL for a slot it does not implement.
const KernelEntry *lookup_w8(int kop, bool is_signed);
const KernelEntry *lookup_w16(int kop, bool is_signed);
const KernelEntry *lookup_w32(int kop, bool is_signed);
const KernelEntry *lookup_w64(int kop, bool is_signed);
const KernelEntry *lookup_fp(int kop, int bytes); // bytes = 2, 4, 8; K_MAX..K_PROD

} // namespace xccl_rocm
