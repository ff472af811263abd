// Zero fill by a kernel.  The library clears flags, split-K accumulators and empty-sum outputs with this instead of
// hipMemsetAsync so that every call can be recorded into a HIP graph by the caller (memset nodes of captured
// graphs have given wrong results on replay on this platform).
#include "amr_common.h"

namespace amr {

__global__ __launch_bounds__(256) void zero_u32_kernel(uint32_t* __restrict__ p, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) p[i] = 0u;
}

hipError_t launch_zero_u32(void* p, size_t n_dwords, hipStream_t stream) {
    if (n_dwords == 0) return hipSuccess;
    size_t blocks = (n_dwords + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(zero_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(p), n_dwords);
    return hipGetLastError();
}

// In-place conversion of uint32 sums to float32 (the forward pass with float output when K was split over workgroups:
// the partial sums meet as integers first).
__global__ __launch_bounds__(256) void u32_to_f32_kernel(uint32_t* __restrict__ p, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) p[i] = __float_as_uint((float)p[i]);
}

hipError_t launch_u32_to_f32(void* p, size_t n_dwords, hipStream_t stream) {
    if (n_dwords == 0) return hipSuccess;
    size_t blocks = (n_dwords + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(u32_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(p), n_dwords);
    return hipGetLastError();
}

}  // namespace amr
