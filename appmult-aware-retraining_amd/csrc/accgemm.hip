// Accurate fp32 GEMM C = A.B (row-major) for gfx950; exported for API parity only.
// Replaces AccGemmForwardKernelFP32 (self_ops/src/approx_gemm_forward.cu:348-492), which no layer of
// the reference uses.  64x64 output tile per 256-thread workgroup, 16-deep K slices staged through
// LDS, 4x4 register tile per thread, fp32 FMA accumulation in ascending k.
#include "amr_common.h"

namespace amr {

__global__ __launch_bounds__(256) void accgemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                          float* __restrict__ C, int M, int K, int N) {
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float As[BK][BM + 1];
    __shared__ float Bs[BK][BN + 1];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    int tile_n, tile_m;
    folded_tile_xy((N + BN - 1) / BN, &tile_n, &tile_m);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
        for (int i = threadIdx.x; i < BM * BK; i += 256) {
            const int r = i / BK, c = i % BK;
            As[c][r] = (m0 + r < M && k0 + c < K) ? A[(size_t)(m0 + r) * K + k0 + c] : 0.f;
        }
        for (int i = threadIdx.x; i < BK * BN; i += 256) {
            const int r = i / BN, c = i % BN;
            Bs[r][c] = (k0 + r < K && n0 + c < N) ? B[(size_t)(k0 + r) * N + n0 + c] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + ty + 16 * i, n = n0 + tx + 16 * j;
            if (m < M && n < N) C[(size_t)m * N + n] = acc[i][j];
        }
}

hipError_t launch_accgemm(const float* A, const float* B, float* C, int M, int K, int N, hipStream_t stream) {
    dim3 grid((unsigned)((N + 63) / 64) * (unsigned)((M + 63) / 64));   // column tiles x row tiles, folded into x
    hipLaunchKernelGGL(accgemm_f32_kernel, grid, dim3(256), 0, stream, A, B, C, M, K, N);
    return hipGetLastError();
}

}  // namespace amr
