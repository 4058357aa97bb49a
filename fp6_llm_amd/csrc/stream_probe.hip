// Measurement aid, not part of the engine: a kernel that only streams a buffer from HBM into registers with the same
// 128-bit non-temporal loads and the same launch geometry as the small-batch GEMM (one workgroup of 16 wavefronts per
// 48 KiB, 3 loads per lane).  Its duration is the floor for any kernel that must read those bytes once: the benchmark
// prints it beside the GEMM's time.  Built into its own library (libfp6mi_probe.so), which only the benchmark loads.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace {
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(1024) void stream_read(const v4u *__restrict__ src, uint32_t *__restrict__ sink, uint32_t chunks_per_wg)
{
    const v4u *p = src + (size_t)blockIdx.x * chunks_per_wg * 3072 + threadIdx.x;
    uint32_t   acc = 0;
    for (uint32_t c = 0; c < chunks_per_wg; c++, p += 3072) {
        v4u a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1024), d = __builtin_nontemporal_load(p + 2048);
        acc ^= a[0] ^ a[1] ^ a[2] ^ a[3] ^ b[0] ^ b[1] ^ b[2] ^ b[3] ^ d[0] ^ d[1] ^ d[2] ^ d[3];
    }
    if (acc == 0x9e3779b9u) sink[0] = acc; // keeps the loads alive; practically never true
}

// A producer / consumer pair for the question "where should the kernel that reads another kernel's output run?".
// pair_write: workgroup b fills region b (256 threads x `per` 16-byte pieces).  pair_read: workgroup b reads region
// (b + shift) mod grid.  Workgroup ids congruent mod 8 run on one XCD, so shift = 0 or 8 reads through the L2 the data was
// written through and any other shift reads from another XCD.
typedef float v4f __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void pair_write(v4f *__restrict__ buf, uint32_t per)
{
    v4f *p = buf + (size_t)blockIdx.x * 256 * per + threadIdx.x;
    for (uint32_t i = 0; i < per; i++) p[(size_t)i * 256] = (v4f){ 1.f, 2.f, 3.f, (float)i };
}
__global__ __launch_bounds__(256) void pair_read(const v4f *__restrict__ buf, uint32_t *__restrict__ sink, uint32_t per, uint32_t shift)
{
    const v4f *p = buf + (size_t)((blockIdx.x + shift) % gridDim.x) * 256 * per + threadIdx.x;
    v4f        acc = { 0.f, 0.f, 0.f, 0.f };
    for (uint32_t i = 0; i < per; i++) acc += p[(size_t)i * 256];
    if (acc[0] + acc[1] + acc[2] + acc[3] == -1.f) sink[0] = 1u; // never true: the sums are positive
}
} // namespace

// One write kernel followed by one read kernel over `wgs` regions of 4096 * per bytes each, on `stream`.
extern "C" int fp6mi_probe_write_then_read(void *stream, void *buf, unsigned wgs, unsigned per, unsigned shift, void *sink)
{
    if (!buf || !sink || wgs == 0 || per == 0) return -3;
    hipLaunchKernelGGL(pair_write, dim3(wgs), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<v4f *>(buf), per);
    hipLaunchKernelGGL(pair_read, dim3(wgs), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const v4f *>(buf),
                       static_cast<uint32_t *>(sink), per, shift);
    return (int)hipGetLastError();
}

// Reads the first `bytes` (rounded down to a multiple of 48 KiB times the chunks per workgroup) of `src` on `stream`.
// Workgroups stay near one per 48 KiB up to 2048 of them, then each takes several chunks.
extern "C" int fp6mi_probe_stream_read(void *stream, const void *src, size_t bytes, void *sink)
{
    if (!src || !sink) return -3;
    if ((reinterpret_cast<uintptr_t>(src) & 15u) != 0) return -6;
    size_t chunks = bytes / 49152;
    if (chunks == 0) return -2;
    uint32_t per_wg = (uint32_t)((chunks + 2047) / 2048);
    uint32_t wgs = (uint32_t)(chunks / per_wg);
    hipLaunchKernelGGL(stream_read, dim3(wgs), dim3(1024), 0, static_cast<hipStream_t>(stream), static_cast<const v4u *>(src),
                       static_cast<uint32_t *>(sink), per_wg);
    return (int)hipGetLastError();
}
