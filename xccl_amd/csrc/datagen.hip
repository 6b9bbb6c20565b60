// datagen.hip -- libxccl_rocm_benchkit.so: fills device buffers with the
// synthetic workload of the benchmarks, on the GPU.  Not part of the memory
// component; bench and tests use it so that multi-GiB inputs need not cross
// PCIe.
//
// Every element is a pure function of (seed, vector index, element index):
//     x = splitmix64(seed * 0x9E3779B97F4A7C15 + (vec << 40) + i)
//     FLOAT32  (x >> 40) * 2^-23 - 1          uniform [-1, 1), exact
//     FLOAT16  (x >> 53) * 2^-11 - 0.5        uniform [-0.5, 0.5), exact
//     FLOAT64  Box-Muller normal(0, 1) from x and y = splitmix64(x)
//     integers the low 8*sizeof(T) bits of x (full range); with `sparse`
//              set, the element is zeroed when bit 63 of y is set (the
//              inputs of the logical operators: half zeros)
// The CPU generator of the test oracle follows the same recipe; the two agree
// bit for bit except FLOAT64, where log/cos come from different math
// libraries.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "xccl_rocm_types.h"

namespace {

__host__ __device__ inline uint64_t splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

template <typename T> struct Gen;

template <> struct Gen<float> {
    static __device__ float make(uint64_t x, uint64_t, int) { return (float)(x >> 40) * 0x1p-23f - 1.0f; }
};
template <> struct Gen<_Float16> {
    static __device__ _Float16 make(uint64_t x, uint64_t, int) { return (_Float16)((float)(x >> 53) * 0x1p-11f - 0.5f); }
};
template <> struct Gen<double> {
    static __device__ double make(uint64_t x, uint64_t y, int)
    {
        const double u1 = ((double)(x >> 11) + 1.0) * 0x1p-53; // (0, 1]
        const double u2 = (double)(y >> 11) * 0x1p-53;         // [0, 1)
        return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
    }
};
template <typename T> struct Gen {
    static __device__ T make(uint64_t x, uint64_t y, int sparse) { return (sparse && (y >> 63)) ? (T)0 : (T)x; }
};

template <typename T>
__global__ void __launch_bounds__(256) fill_kernel(T *dst, size_t count, uint64_t base, int sparse)
{
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += step) {
        const uint64_t x = splitmix64(base + i);
        dst[i]           = Gen<T>::make(x, splitmix64(x), sparse);
    }
}

template <typename T>
hipError_t fill(void *dst, size_t count, uint64_t base, int sparse, hipStream_t s)
{
    size_t blocks = (count + 255) / 256;
    if (blocks > 65536) {
        blocks = 65536;
    }
    hipLaunchKernelGGL(fill_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, (T *)dst, count, base, sparse);
    return hipGetLastError();
}

// A plain 16-byte-per-lane copy: the known-traffic kernel that hardware
// counter readings are calibrated against (reads n bytes, writes n bytes).
__global__ void __launch_bounds__(256) copy_kernel(const uint4 *src, uint4 *dst, size_t nvec)
{
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += step) {
        dst[i] = src[i];
    }
}

// Reads what a reduction of `nsrc` vectors reads, in the same pattern (one
// wave per 1 KiB tile, the sources one after the other, non-temporal buffer
// loads, two in flight), and writes nothing: the read-only ceiling that the
// reduction's read-mostly mix is compared with.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(64) read_kernel(const char *src, size_t stride, uint32_t nsrc, size_t nvec,
                                                  uint32_t *sink)
{
    const size_t v0 = (size_t)blockIdx.x * 64;
    if (v0 >= nvec) {
        return;
    }
    const size_t   left  = nvec - v0;
    const uint32_t bytes = (uint32_t)(left < 64 ? left : 64) * 16u;
    const uint32_t off   = threadIdx.x * 16u;
    const char    *p     = src + v0 * 16;
    u32x4          acc   = {0, 0, 0, 0};
    u32x4          l0    = __builtin_amdgcn_raw_buffer_load_b128(
        __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, (int)bytes, 0x00027000), (int)off, 0, 2);
    for (uint32_t j = 1; j <= nsrc; ++j) {
        p += stride;
        u32x4 l1 = __builtin_amdgcn_raw_buffer_load_b128(
            __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, j < nsrc ? (int)bytes : 0, 0x00027000), (int)off, 0, 2);
        __builtin_amdgcn_sched_barrier(0);
        acc ^= l0;
        l0 = l1;
        __builtin_amdgcn_sched_barrier(0);
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5eed1234u && sink != nullptr) {
        *sink = acc.x; // practically never; keeps the loads alive
    }
}

} // namespace

// Reads `nsrc` vectors of `bytes` each (a multiple of 16), `stride` bytes apart, with read_kernel on
// `hip_stream`; `lds_bytes` of unused LDS per workgroup bound the resident waves like the reduction's launch.
extern "C" xccl_status_t xccl_rocm_bench_read(const void *src, size_t stride, unsigned nsrc, size_t bytes,
                                              unsigned lds_bytes, void *sink, void *hip_stream)
{
    if (bytes % 16 != 0 || nsrc == 0) {
        return XCCL_ERR_INVALID_PARAM;
    }
    const size_t nvec = bytes / 16;
    const size_t grid = (nvec + 63) / 64;
    if (grid == 0 || grid > 0x7fffffffu) {
        return XCCL_ERR_INVALID_PARAM;
    }
    hipLaunchKernelGGL(read_kernel, dim3((unsigned)grid), dim3(64), lds_bytes, (hipStream_t)hip_stream,
                       (const char *)src, stride, nsrc, nvec, (uint32_t *)sink);
    return hipGetLastError() == hipSuccess ? XCCL_OK : XCCL_ERR_NO_MESSAGE;
}

// Copies `bytes` (a multiple of 16) from src to dst with copy_kernel on `hip_stream`.
extern "C" xccl_status_t xccl_rocm_bench_copy(void *dst, const void *src, size_t bytes, void *hip_stream)
{
    if (bytes % 16 != 0) {
        return XCCL_ERR_INVALID_PARAM;
    }
    const size_t nvec   = bytes / 16;
    size_t       blocks = (nvec + 255) / 256;
    if (blocks > (1u << 20)) {
        blocks = 1u << 20;
    }
    if (blocks == 0) {
        return XCCL_OK;
    }
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)hip_stream, (const uint4 *)src,
                       (uint4 *)dst, nvec);
    return hipGetLastError() == hipSuccess ? XCCL_OK : XCCL_ERR_NO_MESSAGE;
}

// Fills dst[0 .. count) with vector `vec` of the stream identified by `seed`.
// Enqueues on `hip_stream` (hipStream_t as void*) and returns.
extern "C" xccl_status_t xccl_rocm_datagen_fill(void *dst, size_t count, xccl_dt_t dtype, uint64_t seed, uint64_t vec,
                                                int sparse, void *hip_stream)
{
    const uint64_t base = seed * 0x9E3779B97F4A7C15ull + (vec << 40);
    hipStream_t    s    = (hipStream_t)hip_stream;
    hipError_t     e;
    if (count == 0) {
        return XCCL_OK;
    }
    switch (dtype) {
    case XCCL_DT_INT8:
    case XCCL_DT_UINT8:   e = fill<uint8_t>(dst, count, base, sparse, s); break;
    case XCCL_DT_INT16:
    case XCCL_DT_UINT16:  e = fill<uint16_t>(dst, count, base, sparse, s); break;
    case XCCL_DT_INT32:
    case XCCL_DT_UINT32:  e = fill<uint32_t>(dst, count, base, sparse, s); break;
    case XCCL_DT_INT64:
    case XCCL_DT_UINT64:  e = fill<uint64_t>(dst, count, base, sparse, s); break;
    case XCCL_DT_FLOAT16: e = fill<_Float16>(dst, count, base, sparse, s); break;
    case XCCL_DT_FLOAT32: e = fill<float>(dst, count, base, sparse, s); break;
    case XCCL_DT_FLOAT64: e = fill<double>(dst, count, base, sparse, s); break;
    default:              return XCCL_ERR_UNSUPPORTED;
    }
    return e == hipSuccess ? XCCL_OK : XCCL_ERR_NO_MESSAGE;
}
