// Yardsticks for bench.py, not part of the C ABI of libbsa_hip.so: a plain streaming copy with the
// access pattern the block kernels use for data that is touched once (16 bytes per lane, non-temporal
// loads and stores, four loads in flight per lane), the same stream as a read alone and as a write alone,
// and a launch that does nothing.  bench.py times them on the softmax's byte count in the same run and the
// same way as the kernels, so that every "fraction of the HBM peak" in its output can be read against
// what plain streams reach on that box in that minute (reads and writes together are slower than the
// two apart, and a launch costs time before its first byte moves).
#include <hip/hip_runtime.h>
#include <stddef.h>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int K>
__global__ __launch_bounds__(256) void stream_copy_nt(const u32x4 *__restrict__ in, u32x4 *__restrict__ out, size_t n)
{
    const size_t base = (size_t)blockIdx.x * (256 * K) + threadIdx.x;
    u32x4 v[K];
#pragma unroll
    for (int k = 0; k < K; ++k)
        if (base + (size_t)k * 256 < n) v[k] = __builtin_nontemporal_load(in + base + (size_t)k * 256);
#pragma unroll
    for (int k = 0; k < K; ++k)
        if (base + (size_t)k * 256 < n) __builtin_nontemporal_store(v[k], out + base + (size_t)k * 256);
}

// copies `bytes` (a multiple of 16) from src to dst on `stream`; returns the hipError_t of the launch
extern "C" int bsa_bench_copy_nt(const void *src, void *dst, size_t bytes, void *stream)
{
    if (!src || !dst || bytes == 0 || bytes % 16) return (int)hipErrorInvalidValue;
    constexpr int K = 4;
    const size_t n = bytes / 16;
    const unsigned grid = (unsigned)((n + 256 * K - 1) / (256 * K));
    stream_copy_nt<K><<<grid, 256, 0, (hipStream_t)stream>>>((const u32x4 *)src, (u32x4 *)dst, n);
    return (int)hipGetLastError();
}

template <int K>
__global__ __launch_bounds__(256) void stream_read_nt(const u32x4 *__restrict__ in, unsigned *__restrict__ sink, size_t n)
{
    const size_t base = (size_t)blockIdx.x * (256 * K) + threadIdx.x;
    unsigned acc = 0;
#pragma unroll
    for (int k = 0; k < K; ++k)
        if (base + (size_t)k * 256 < n) {
            const u32x4 v = __builtin_nontemporal_load(in + base + (size_t)k * 256);
            acc += v.x ^ v.y ^ v.z ^ v.w;
        }
    if (acc == 0x9E3779B9u) *sink = acc;       // keeps the loads alive; practically never taken
}

template <int K>
__global__ __launch_bounds__(256) void stream_write_nt(u32x4 *__restrict__ out, size_t n)
{
    const size_t base = (size_t)blockIdx.x * (256 * K) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < K; ++k)
        if (base + (size_t)k * 256 < n) {
            const u32x4 v = {(unsigned)base, (unsigned)k, 0u, 1u};
            __builtin_nontemporal_store(v, out + base + (size_t)k * 256);
        }
}

__global__ void empty_launch(unsigned *sink)
{
    if (sink && threadIdx.x == 0xFFFFu) *sink = 0;
}

// reads `bytes` (a multiple of 16) from src; `sink` is 4 bytes of device memory that are practically never written
extern "C" int bsa_bench_read_nt(const void *src, void *sink, size_t bytes, void *stream)
{
    if (!src || !sink || bytes == 0 || bytes % 16) return (int)hipErrorInvalidValue;
    constexpr int K = 4;
    const size_t n = bytes / 16;
    const unsigned grid = (unsigned)((n + 256 * K - 1) / (256 * K));
    stream_read_nt<K><<<grid, 256, 0, (hipStream_t)stream>>>((const u32x4 *)src, (unsigned *)sink, n);
    return (int)hipGetLastError();
}

extern "C" int bsa_bench_write_nt(void *dst, size_t bytes, void *stream)
{
    if (!dst || bytes == 0 || bytes % 16) return (int)hipErrorInvalidValue;
    constexpr int K = 4;
    const size_t n = bytes / 16;
    const unsigned grid = (unsigned)((n + 256 * K - 1) / (256 * K));
    stream_write_nt<K><<<grid, 256, 0, (hipStream_t)stream>>>((u32x4 *)dst, n);
    return (int)hipGetLastError();
}

// a launch of `workgroups` x 256 threads that does nothing
extern "C" int bsa_bench_empty(unsigned workgroups, void *stream)
{
    if (workgroups == 0) return (int)hipErrorInvalidValue;
    empty_launch<<<workgroups, 256, 0, (hipStream_t)stream>>>(nullptr);
    return (int)hipGetLastError();
}
