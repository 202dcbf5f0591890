// A plain device-to-device copy, one 16-byte load and store per thread.  Hardware counters read on it (rocprofv3 --pmc
// FETCH_SIZE / WRITE_SIZE over `bench.py --calibrate`) calibrate the same counters read on the rasterizer's kernels:
// the counters' units differ between GPU generations, a copy of known size does not.  Built into its own small library
// (libhtgs_copy.so, bound by htgs_amd/diagnostics/__init__.py); the rasterizer library does not contain it.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {
__global__ void __launch_bounds__(256) copy_bytes_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}
}  // namespace

// n_bytes: a multiple of 16.  0 = ok, 2 = bad argument, 3 = the launch failed.
extern "C" int htgs_diag_copy_bytes(void *dst, const void *src, size_t n_bytes, void *stream)
{
    if (!dst || !src || (n_bytes & 15)) return 2;
    const size_t n = n_bytes / 16;
    if (n == 0) return 0;
    if ((n + 255) / 256 > 0x7fffffffull) return 2;
    hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const uint4 *)src, (uint4 *)dst, n);
    return hipGetLastError() == hipSuccess ? 0 : 3;
}
