// Copy probe: a plain streaming copy kernel of known size.  HBM counters of a profile
// (bytes fetched / written per dispatch) are scaled by what they read for this kernel.
#include <hip/hip_runtime.h>
#include "internal.hpp"

using namespace sddmm;

namespace {

__global__ __launch_bounds__(256)
void sddmm_copy_probe_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst, int64_t n16)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

}  // namespace

extern "C" int sddmm_copy_probe(const void *d_src, void *d_dst, int64_t n_bytes, void *stream)
{
    if (!d_src || !d_dst || n_bytes < 16 || n_bytes % 16 || (((uintptr_t)d_src | (uintptr_t)d_dst) & 15u))
        return fail(SDDMM_ERR_ARG, "sddmm_copy_probe: pointers and size must be non-null multiples of 16 bytes");
    const int64_t n16 = n_bytes / 16;
    const unsigned grid = (unsigned)std::min<int64_t>((n16 + 255) / 256, 256 * 32);
    hipLaunchKernelGGL(sddmm_copy_probe_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                       (const float4 *)d_src, (float4 *)d_dst, n16);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SDDMM_ERR_HIP, "sddmm_copy_probe: %s", hipGetErrorString(e));
    return SDDMM_OK;
}
