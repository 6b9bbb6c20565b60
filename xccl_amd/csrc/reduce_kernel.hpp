// reduce_kernel.hpp -- the one gfx950 kernel template behind reduce and
// reduce_multi, and the per-(type, op) table entries built from it.
//
// What it computes (reference src/utils/mem_component.c:133-139 for the fold,
// src/utils/reduce.h:14-23 for the operators):
//     acc = OP(sbuf1[i], sbuf2{0}[i]);  acc = OP(sbuf2{j}[i], acc), j = 1..n-1
//     rbuf[i] = acc
// The reference's CUDA kernel (xccl_cuda_reduce_multi.cu:17-40) keeps acc in
// global memory and reads 2/4/8 bytes per lane; here every lane moves 16 bytes
// per source with one buffer_load_dwordx4 and acc never leaves registers.
//
// Shape, from measurement on MI355X.  A workgroup is one wavefront and owns
// one tile: 64 x 16 bytes = 1 KiB of every source.  The wave walks the
// sources in fold order with two loads in flight (ping-pong registers):
// while source j is folded into the accumulator, sources j+1 and j+2 are on
// their way.  One kernel serves any number of sources.  The obvious
// alternative -- issue the loads of all sources at the same offset at once,
// then fold -- makes every wave send a burst of same-offset requests to
// vectors that lie a power of two apart, which land on the same memory
// channels at the same moment: on the headline shape (8 x 256 MiB, fp32 SUM)
// that is 6.4 TB/s against 6.8-7.0 TB/s for the source-by-source walk, and
// 5.5 against 6.6 TB/s with 1 GiB vectors.  Persistent workgroups that loop
// over tiles, larger tiles and multi-wave workgroups all measured slower.
// Sources are read once: non-temporal loads.  The result is about to be read
// by another agent (the NIC sending it, the next round's kernel): stores carry
// system scope (sc0 sc1), i.e. write through instead of lingering dirty in L2.
// The launch asks for LDS it never touches to hold the resident workgroups
// per compute unit to 16-32 (by source count): the memory side saturates
// before the wave slots do.
//   Launches of a few thousand tiles at most are a different regime: the
// memory side is idle and the call is bound by the chain of load latencies.
// They run the second form of the kernel (Burst = true), which does issue
// the loads of up to nine sources at once.
//
// Layout of one call, in elements of T:
//     [0, head)                 peeled so that the vector body starts on a
//                               16-byte boundary of the buffer chosen by the
//                               host (fewer than 16/sizeof(T) elements)
//     [head, head + nvec*VE)    nvec 16-byte vectors, VE = 16/sizeof(T)
//     [.., .. + tail)           fewer than VE elements
// Head and tail are folded one element per lane by the last block, through
// buffer accesses of sizeof(T) bytes with the same cache-policy bits.
// Vector accesses are emitted as dwordx4 whatever the address is (the device
// runs in unaligned access mode, for buffer instructions too), so a source
// whose alignment differs from the peeled one costs extra cache-line touches,
// never correctness.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xccl_rocm {

constexpr int kBlock = 64; // one wavefront per workgroup

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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
    uint32_t    grid;   // workgroups of the launch (the kernel reads no implicit launch arguments)
    // Completion word (small launches only; all NULL/0 otherwise): when the last workgroup
    // is through, done_seq is stored to *done_flag, a host-mapped word the caller polls.
    uint32_t    done_seq;
    uint32_t   *done_count; // device words (1 + kDoneShards, kDoneStride apart), zero between launches
    uint32_t    done_slots; // != 0: no counting, workgroup b stores done_seq to done_flag[b] (grid <= done_slots)
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

// 8- and 16-bit elements, four or two to a register: the logical operators and
// the 8-bit SUM as whole-register arithmetic.  Element by element the compiler
// unpacks and repacks every byte (about 40 VALU instructions per 16-byte vector
// and source for LAND), which made these the slowest rows of the integer sweep.
//   nz(x): 1 in every element of x that is non-zero, else 0 -- adding 0x7f..
//   to the low bits carries into an element's top bit iff they are non-zero.
__device__ __forceinline__ u32x4 nz8(u32x4 x)
{
    return ((((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) >> 7) & 0x01010101u;
}
__device__ __forceinline__ u32x4 nz16(u32x4 x)
{
    return ((((x & 0x7fff7fffu) + 0x7fff7fffu) | x) >> 15) & 0x00010001u;
}
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpLand>(u32x4 a, u32x4 b) { return nz8(a) & nz8(b); }
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpLor>(u32x4 a, u32x4 b)  { return nz8(a | b); }
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpLxor>(u32x4 a, u32x4 b) { return nz8(a) ^ nz8(b); }
template <> __device__ __forceinline__ u32x4 vfold<uint16_t, OpLand>(u32x4 a, u32x4 b) { return nz16(a) & nz16(b); }
template <> __device__ __forceinline__ u32x4 vfold<uint16_t, OpLor>(u32x4 a, u32x4 b)  { return nz16(a | b); }
template <> __device__ __forceinline__ u32x4 vfold<uint16_t, OpLxor>(u32x4 a, u32x4 b) { return nz16(a) ^ nz16(b); }
// byte-wise wrapping add: add the low 7 bits of every byte (no carry can leave
// a byte), then put the top bits back with an exclusive or
template <> __device__ __forceinline__ u32x4 vfold<uint8_t, OpSum>(u32x4 a, u32x4 b)
{
    return ((a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu)) ^ ((a ^ b) & 0x80808080u);
}

// Vector accesses go through buffer instructions: the descriptor (scalar
// registers) holds the tile's base address and its length in bytes, the lane
// supplies a 32-bit offset.  The hardware drops stores and returns zero for
// loads beyond the length, so the ragged last tile needs no branch, and the
// cache-policy bits are ordinary operands the compiler tracks (no inline asm).
//   loads:  nt            (aux bit 1)
//   stores: sc0 sc1       (aux bits 0 and 4)
constexpr int kAuxLoad  = 0x02;
constexpr int kAuxStore = 0x11;
// DST_SEL_X/Y/Z/W = X/Y/Z/W, 32-bit data format: the raw-buffer descriptor word gfx9 expects
constexpr int kRsrcFlags = 0x00027000;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const char *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)bytes, kRsrcFlags);
}

__device__ __forceinline__ u32x4 vload(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, kAuxLoad);
}

__device__ __forceinline__ void vstore(__amdgpu_buffer_rsrc_t r, uint32_t off, u32x4 v)
{
    __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)off, 0, kAuxStore);
}

// Single elements (head and tail) go through the same kind of access: a buffer
// load or store of sizeof(T) bytes with the same cache-policy bits, the lane's
// element picked by its offset, lanes past the descriptor's length clipped by
// the hardware.
template <int Bytes> struct ElemAccess;
template <> struct ElemAccess<1> {
    typedef uint8_t U;
    static __device__ __forceinline__ U ld(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b8(r, (int)off, 0, kAuxLoad); }
    static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, uint32_t off, U v) { __builtin_amdgcn_raw_buffer_store_b8(v, r, (int)off, 0, kAuxStore); }
};
template <> struct ElemAccess<2> {
    typedef uint16_t U;
    static __device__ __forceinline__ U ld(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, kAuxLoad); }
    static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, uint32_t off, U v) { __builtin_amdgcn_raw_buffer_store_b16(v, r, (int)off, 0, kAuxStore); }
};
template <> struct ElemAccess<4> {
    typedef uint32_t U;
    static __device__ __forceinline__ U ld(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, kAuxLoad); }
    static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, uint32_t off, U v) { __builtin_amdgcn_raw_buffer_store_b32(v, r, (int)off, 0, kAuxStore); }
};
template <> struct ElemAccess<8> {
    typedef uint32_t U __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ U ld(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, kAuxLoad); }
    static __device__ __forceinline__ void st(__amdgpu_buffer_rsrc_t r, uint32_t off, U v) { __builtin_amdgcn_raw_buffer_store_b64(v, r, (int)off, 0, kAuxStore); }
};

template <typename T>
__device__ __forceinline__ T eload(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    const typename ElemAccess<sizeof(T)>::U u = ElemAccess<sizeof(T)>::ld(r, off);
    T v;
    __builtin_memcpy(&v, &u, sizeof(T));
    return v;
}

template <typename T>
__device__ __forceinline__ void estore(__amdgpu_buffer_rsrc_t r, uint32_t off, T v)
{
    typename ElemAccess<sizeof(T)>::U u;
    __builtin_memcpy(&u, &v, sizeof(T));
    ElemAccess<sizeof(T)>::st(r, off, u);
}

constexpr int kBurst = 8; // loads a latency-bound path keeps in flight per lane

// `count` (< 16) consecutive elements that start `rel` bytes from the vector
// body (negative: the head), all sources, in fold order: lane t folds element
// t; lanes from `count` on read zeros and their store is dropped.  The vectors
// of sbuf2 are requested kBurst at a time; slots past the last vector get a
// zero-length descriptor and a select keeps them out of the fold.
template <typename T, class Op>
__device__ __forceinline__ void fold_elements(const ReduceArgs &a, ptrdiff_t rel, uint32_t count)
{
    const uint32_t bytes = count * (uint32_t)sizeof(T);
    const uint32_t off   = threadIdx.x * (uint32_t)sizeof(T);
    const uint32_t n2    = a.n2;
    const char    *p     = a.s2 + rel;

    T acc = eload<T>(tile_rsrc(a.s1 + rel, bytes), off);
    T l[kBurst];
#pragma unroll
    for (int d = 0; d < kBurst; ++d) {
        l[d] = eload<T>(tile_rsrc(p + (size_t)d * a.stride, (uint32_t)d < n2 ? bytes : 0), off);
    }
    acc = Op::template f<T>(acc, l[0]);
#pragma unroll
    for (int d = 1; d < kBurst; ++d) {
        const T f = Op::template f<T>(l[d], acc);
        acc = (uint32_t)d < n2 ? f : acc;
    }
    for (uint32_t j = kBurst; j < n2; j += kBurst) {
        p += (size_t)kBurst * a.stride;
#pragma unroll
        for (int d = 0; d < kBurst; ++d) {
            l[d] = eload<T>(tile_rsrc(p + (size_t)d * a.stride, j + (uint32_t)d < n2 ? bytes : 0), off);
        }
#pragma unroll
        for (int d = 0; d < kBurst; ++d) {
            const T f = Op::template f<T>(l[d], acc);
            acc = j + (uint32_t)d < n2 ? f : acc;
        }
    }
    estore<T>(tile_rsrc(a.dst + rel, bytes), off, acc);
}

// One tile: kBlock vectors, lane t owns vector v0 + t.  Sources are walked in
// fold order, two loads in flight.  The scheduling barriers pin the issue
// order: left alone, the compiler hoists and clusters the loads and the walk
// turns back into a burst.
template <typename T, class Op>
__device__ __forceinline__ void fold_tile(const ReduceArgs &a, size_t v0)
{
    const size_t   left  = a.nvec - v0;
    const uint32_t bytes = (uint32_t)(left < (size_t)kBlock ? left : (size_t)kBlock) * 16u; // the descriptor clips the ragged tile
    const size_t   toff  = v0 * 16; // uniform: same for every lane of the workgroup
    const uint32_t off   = threadIdx.x * 16u;
    const uint32_t n2    = a.n2;
    const char    *p     = a.s2 + toff; // vector j of sbuf2 as the walk advances

    // A load past the last source gets a descriptor of length zero: the
    // hardware returns zeros without touching memory, and the walk needs no
    // branch around a load (a branch there makes the compiler wait for every
    // load in flight where the paths join).
    u32x4 acc = vload(tile_rsrc(a.s1 + toff, bytes), off);
    u32x4 l0  = vload(tile_rsrc(p, bytes), off);
    p += a.stride;
    u32x4 l1 = vload(tile_rsrc(p, n2 > 1 ? bytes : 0), off);
    __builtin_amdgcn_sched_barrier(0);
    acc = vfold<T, Op>(acc, l0); // OP(sbuf1, sbuf2{0})
    __builtin_amdgcn_sched_barrier(0);
    // here: l1 holds vector j of sbuf2 (in flight), p points at it, l0 is free
    for (uint32_t j = 1; j < n2; j += 2) {
        p += a.stride;
        l0 = vload(tile_rsrc(p, j + 1 < n2 ? bytes : 0), off);
        __builtin_amdgcn_sched_barrier(0);
        acc = vfold<T, Op>(l1, acc); // OP(sbuf2{j}, acc)
        __builtin_amdgcn_sched_barrier(0);
        if (j + 1 >= n2) {
            break;
        }
        p += a.stride;
        l1 = vload(tile_rsrc(p, j + 2 < n2 ? bytes : 0), off);
        __builtin_amdgcn_sched_barrier(0);
        acc = vfold<T, Op>(l0, acc);
        __builtin_amdgcn_sched_barrier(0);
    }
    vstore(tile_rsrc(a.dst + toff, bytes), off, acc);
}

// The same tile for launches so small that the memory side is idle and only
// latency counts: the first kBurst vectors of sbuf2 are requested together with
// sbuf1 and folded as they arrive, in fold order; a longer sbuf2 goes on in
// bursts of kBurst.  Selects, not branches, skip the slots past the last
// vector (their loads have zero-length descriptors and fetch nothing).

template <typename T, class Op>
__device__ __forceinline__ void fold_tile_burst(const ReduceArgs &a, size_t v0)
{
    const size_t   left  = a.nvec - v0;
    const uint32_t bytes = (uint32_t)(left < (size_t)kBlock ? left : (size_t)kBlock) * 16u;
    const size_t   toff  = v0 * 16;
    const uint32_t off   = threadIdx.x * 16u;
    const uint32_t n2    = a.n2;
    const char    *p     = a.s2 + toff;

    u32x4 acc = vload(tile_rsrc(a.s1 + toff, bytes), off);
    u32x4 l[kBurst];
#pragma unroll
    for (int d = 0; d < kBurst; ++d) {
        l[d] = vload(tile_rsrc(p + (size_t)d * a.stride, (uint32_t)d < n2 ? bytes : 0), off);
    }
    acc = vfold<T, Op>(acc, l[0]); // OP(sbuf1, sbuf2{0})
#pragma unroll
    for (int d = 1; d < kBurst; ++d) {
        const u32x4 f = vfold<T, Op>(l[d], acc); // OP(sbuf2{d}, acc)
        acc = (uint32_t)d < n2 ? f : acc;
    }
    for (uint32_t j = kBurst; j < n2; j += kBurst) {
        p += (size_t)kBurst * a.stride;
#pragma unroll
        for (int d = 0; d < kBurst; ++d) {
            l[d] = vload(tile_rsrc(p + (size_t)d * a.stride, j + (uint32_t)d < n2 ? bytes : 0), off);
        }
#pragma unroll
        for (int d = 0; d < kBurst; ++d) {
            const u32x4 f = vfold<T, Op>(l[d], acc);
            acc = j + (uint32_t)d < n2 ? f : acc;
        }
    }
    vstore(tile_rsrc(a.dst + toff, bytes), off, acc);
}

// Tells the host that the launch is complete without going through the queue's
// completion signal (which costs ~4 us more than the kernel's own store on this
// part).  Every workgroup -- one wave -- waits until its own result stores have
// completed, then counts itself in; the last one to arrive publishes the
// sequence number and re-arms the counter.
//   Every result store of the kernel, vectors and single elements alike, is a
//   system-scope write-through store, so "completed" already means "in
//   memory": the wave waits for its outstanding memory operations
//   (s_waitcnt vmcnt(0)) before it counts itself in.  Neither a workgroup-scope
//   fence nor the relaxed arrival atomic would make it wait.
// One contended atomic per workgroup: for small grids only.
__device__ __forceinline__ void publish_completion(const ReduceArgs &a)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (a.done_slots != 0) {
        // A handful of workgroups: each reports on a word of its own and the host
        // looks at all of them, which spares the launch the round trip of an
        // arrival atomic and the arrivals their turn on one counter.
        if (threadIdx.x == 0) {
            __hip_atomic_store(a.done_flag + blockIdx.x, a.done_seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        return;
    }
    if (threadIdx.x == 0) {
        // Arrival counting in two levels, so that no single word takes more than
        // grid/kDoneShards increments: workgroup b counts into shard b % shards, the
        // wave that fills a shard counts into word 0, the wave that fills word 0 is
        // the last.  atomicInc wraps to zero at its bound, so every word is back at
        // zero by itself when the launch is over.  Words are kDoneStride apart
        // (one per 128-byte line): [0] top, [1 + s] shard s.
        const uint32_t grid   = a.grid;
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
            // (a relaxed store here, without the cache write-back a release brings, measured 0.13 us
            // faster at the median and 4 us slower at the 99th percentile of a blocking call)
            __hip_atomic_store(a.done_flag, a.done_seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

// Burst = false: the source-by-source walk; true: fold_tile_burst, for small launches.
template <typename T, class Op, bool Burst>
__global__ void __launch_bounds__(kBlock) reduce_multi_kernel(const ReduceArgs a)
{
    // Head and tail: one element per lane, by the last workgroup.
    if (blockIdx.x == a.grid - 1) {
        if (a.head != 0) {
            fold_elements<T, Op>(a, -(ptrdiff_t)(a.head * sizeof(T)), (uint32_t)a.head);
        }
        if (a.tail != 0) {
            fold_elements<T, Op>(a, (ptrdiff_t)(a.nvec * 16), (uint32_t)a.tail);
        }
    }
    // One tile per workgroup in the usual launch; the loop only runs on when
    // there are more tiles than the grid cap allows workgroups.
    const size_t step = (size_t)a.grid * kBlock;
    for (size_t v0 = (size_t)blockIdx.x * kBlock; v0 < a.nvec; v0 += step) {
        if (Burst) {
            fold_tile_burst<T, Op>(a, v0);
        } else {
            fold_tile<T, Op>(a, v0);
        }
    }
    if (a.done_flag != nullptr) {
        publish_completion(a);
    }
}

// ---- table of instantiations ---------------------------------------------
struct KernelEntry {
    const void *fn;        // reduce_multi_kernel<T, Op, false>
    const void *fn_burst;  // reduce_multi_kernel<T, Op, true>
    int         elem_size; // sizeof(T) the kernels fold in
};

template <typename T, class Op>
KernelEntry make_entry()
{
    KernelEntry e;
    e.fn        = (const void *)&reduce_multi_kernel<T, Op, false>;
    e.fn_burst  = (const void *)&reduce_multi_kernel<T, Op, true>;
    e.elem_size = (int)sizeof(T);
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
