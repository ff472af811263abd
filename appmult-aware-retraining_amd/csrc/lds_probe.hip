// LDS probes: calibrate the denominators of the LDS rooflines on the device at hand (gather rate; rate of LDS-direct
// chunk loads from the L2).
// Every wave issues rounds of 8 independent ds_read_u16 and waits for them; with `waves_per_cu` waves
// resident on each CU the LDS pipe is the only limiter, so gathers / time is the sustained
// conflict-free (pattern 0) or 2-way-conflicted uniform-row (pattern 1) gather rate.
#include "amr_common.h"

namespace amr {

__global__ __launch_bounds__(1024) void lds_probe_kernel(int pattern, int iters, uint32_t* __restrict__ sink) {
    __shared__ uint32_t lds[8192];
    for (int i = threadIdx.x; i < 8192; i += blockDim.x) lds[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    uint32_t addr[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        uint32_t h = (uint32_t)(lane * 4 + s) + 0x9e3779b9u;   // murmur3 finaliser: a real per-lane hash
        h ^= h >> 16; h *= 0x85ebca6bu; h ^= h >> 13; h *= 0xc2b2ae35u; h ^= h >> 16;
        // pattern 0: lane*2 (64 consecutive u16, conflict-free); pattern 1: random u16 inside a 256-byte row
        addr[s] = (pattern == 0 ? (uint32_t)(lane * 2) : ((h >> 10) % 128u) * 2u) + s * 1024;
    }
    uint32_t acc = 0;
    for (int it = 0; it < iters; ++it) {
        uint32_t r0, r1, r2, r3, r4, r5, r6, r7;
        asm volatile(
            "ds_read_u16 %0, %8\n ds_read_u16 %1, %9\n ds_read_u16 %2, %10\n ds_read_u16 %3, %11\n"
            "ds_read_u16 %4, %8 offset:4096\n ds_read_u16 %5, %9 offset:4096\n ds_read_u16 %6, %10 offset:4096\n"
            "ds_read_u16 %7, %11 offset:4096\n s_waitcnt lgkmcnt(0)\n"
            : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(r5), "=&v"(r6), "=&v"(r7)
            : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3])
            : "memory");
        acc += r0 + r1 + r2 + r3 + r4 + r5 + r6 + r7;
    }
    if (acc == 0x12345678u) sink[0] = acc;  // keeps the reads alive; practically never taken
}

// Pattern 2: the rate at which a CU takes 32 KB chunks from the L2 into LDS with LDS-direct loads
// (global_load_lds_dwordx4), the road the expanded-table kernels' chunks travel.  One 1024-thread workgroup per CU,
// three chunk buffers, two chunks requested ahead (the expanded-table kernels' own depth), every workgroup walks the same
// `n_chunks` chunks of `src` over and over (`iters` chunks in all), so that all but the first reader of a chunk are
// served by the L2.  No arithmetic, no LDS reads, no barrier: what is left is the delivery itself.
__global__ __launch_bounds__(1024) void lds_direct_probe_kernel(const uint32_t* __restrict__ src, int n_chunks, int iters) {
    __shared__ __align__(16) unsigned char smem[3 * 32768];
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int wave = uniform(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const u32x4* s4 = reinterpret_cast<const u32x4*>(src);
    auto request = [&](int i) {
        const u32x4* c = s4 + (size_t)(i % n_chunks) * 2048;
        unsigned char* dst = smem + (i % 3) * 32768;
#pragma unroll
        for (int h = 0; h < 2; ++h)
            __builtin_amdgcn_global_load_lds((gptr_t)(c + (wave + 16 * h) * 64 + lane), (lptr_t)(dst + (wave + 16 * h) * 1024), 16, 0, 0);
    };
    request(0);
    request(1);
    for (int i = 0; i < iters; ++i) {
        request(i + 2);
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");     // chunk i has landed; two chunks stay in flight
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

hipError_t run_lds_direct_probe(int n_chunks, int iters, int n_cu, float* ms_out, double* bytes_out, hipStream_t stream) {
    // (288 chunks = 9 MB: the expanded table of a 576 x 64 layer, more than an XCD's 4 MB L2 holds; 32 chunks stay in it)
    uint32_t* src = nullptr;
    hipError_t e = hipMalloc(&src, (size_t)n_chunks * 32768);
    if (e != hipSuccess) return e;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    hipLaunchKernelGGL(lds_direct_probe_kernel, dim3(n_cu), dim3(1024), 0, stream, src, n_chunks, 2 * n_chunks);  // warm-up
    (void)hipEventRecord(e0, stream);
    hipLaunchKernelGGL(lds_direct_probe_kernel, dim3(n_cu), dim3(1024), 0, stream, src, n_chunks, iters);
    (void)hipEventRecord(e1, stream);
    e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipGetLastError();
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(src);
    if (ms_out) *ms_out = ms;
    if (bytes_out) *bytes_out = (double)n_cu * (double)(iters + 2) * 32768.0;
    return e;
}

hipError_t run_lds_probe(int pattern, int waves_per_cu, int iters, int n_cu, float* ms_out, double* gathers_out,
                         hipStream_t stream) {
    if (waves_per_cu < 1) waves_per_cu = 1;
    if (waves_per_cu > 16) waves_per_cu = 16;
    uint32_t* sink = nullptr;
    hipError_t e = hipMalloc(&sink, 4);
    if (e != hipSuccess) return e;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    hipLaunchKernelGGL(lds_probe_kernel, dim3(n_cu), dim3(64 * waves_per_cu), 0, stream, pattern, 16, sink);  // warm-up
    (void)hipEventRecord(e0, stream);
    hipLaunchKernelGGL(lds_probe_kernel, dim3(n_cu), dim3(64 * waves_per_cu), 0, stream, pattern, iters, sink);
    (void)hipEventRecord(e1, stream);
    e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipGetLastError();
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (ms_out) *ms_out = ms;
    if (gathers_out) *gathers_out = (double)n_cu * waves_per_cu * (double)iters * 8.0 * 64.0;
    return e;
}

}  // namespace amr
