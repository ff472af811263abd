// Dequantisation of the LUT convolution result, gfx950: one pass from the GEMM's row layout to the NCHW activation.
//
//   out[b,n,pos] = (s_a*s_w) * ( c[m,n] + ((z_w*xs[m] + z_a*wr[n,pos]) + (z_a*z_w)*tp[pos]) ) + bias[n],   m = b*L + pos
//
// c [M,N] is the LUT-GEMM result as float, xs [M] the box sums of the input codes, wr [N,L] the response of the weight
// codes to an all-ones image, tp [L] the number of taps inside the image times the input channels: the three
// zero-point terms of the reference's ApproxConv2d.forward (micronet+/app_layers.py:175-183) in factorised form.
// The operations and their order are those of the torch expression this replaces (every product and sum rounded on
// its own, no fused multiply-add), so the values are bit-identical to it.  The backward kernel is the transpose back
// with the scale: g_c[m,n] = (s_a*s_w) * g[b,n,pos].
// Both go through 32 x 32 LDS tiles so that reads run along n (rows of c) and writes along pos (NCHW), or the reverse; a
// workgroup takes four such tiles along m and issues the 16 loads of a thread before the first is used.
#include "amr_common.h"

namespace amr {

__global__ __launch_bounds__(256) void dequant_rows_to_nchw_kernel(
    const float* __restrict__ c, const float* __restrict__ xs, const float* __restrict__ wr, const float* __restrict__ tp,
    const float* __restrict__ za_p, const float* __restrict__ zw_p, const float* __restrict__ sa_p, const float* __restrict__ sw_p,
    const float* __restrict__ bias, float* __restrict__ out, int M, int N, int L, const uint32_t* __restrict__ gate) {
    __shared__ float tile[4][32][33];
    if (gate != nullptr && *gate == 0u) return;       // queued behind a kernel that usually has done this work already
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int m0 = blockIdx.x * 128, n0 = blockIdx.y * 32;
    const float za = *za_p, zw = *zw_p;
    const float s = __fmul_rn(*sa_p, *sw_p), zz = __fmul_rn(za, zw);
    {
        float v[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = min(m0 + 32 * t + ty + 8 * r, M - 1), n = min(n0 + tx, N - 1);
                v[t][r] = c[(size_t)m * N + n];
            }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) tile[t][ty + 8 * r][tx] = v[t][r];
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int m = m0 + 32 * t + tx;
        if (m >= M) break;
        const int b = m / L, pos = m - b * L;
        const float x_term = __fmul_rn(zw, xs[m]);
        const float t_term = __fmul_rn(zz, tp[pos]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n0 + ty + 8 * r;
            if (n < N) {
                const float terms = __fadd_rn(__fadd_rn(x_term, __fmul_rn(za, wr[(size_t)n * L + pos])), t_term);
                float v = __fmul_rn(s, __fadd_rn(tile[t][tx][ty + 8 * r], terms));
                if (bias != nullptr) v = __fadd_rn(v, bias[n]);
                out[((size_t)b * N + n) * L + pos] = v;
            }
        }
    }
}

__global__ __launch_bounds__(256) void dequant_grad_nchw_to_rows_kernel(const float* __restrict__ g, const float* __restrict__ sa_p,
                                                                        const float* __restrict__ sw_p, float* __restrict__ gc,
                                                                        int M, int N, int L) {
    __shared__ float tile[4][32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int m0 = blockIdx.x * 128, n0 = blockIdx.y * 32;
    const float s = __fmul_rn(*sa_p, *sw_p);
    {
        float v[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int m = min(m0 + 32 * t + tx, M - 1);
            const int b = m / L, pos = m - b * L;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = min(n0 + ty + 8 * r, N - 1);
                v[t][r] = g[((size_t)b * N + n) * L + pos];
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) tile[t][tx][ty + 8 * r] = __fmul_rn(s, v[t][r]);
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + 32 * t + ty + 8 * r, n = n0 + tx;
            if (m < M && n < N) gc[(size_t)m * N + n] = tile[t][ty + 8 * r][tx];
        }
}

hipError_t launch_dequant(const float* c, const float* xs, const float* wr, const float* tp, const float* za, const float* zw,
                          const float* sa, const float* sw, const float* bias, float* out, int M, int N, int L, hipStream_t stream) {
    hipLaunchKernelGGL(dequant_rows_to_nchw_kernel, dim3((M + 127) / 128, (N + 31) / 32), dim3(256), 0, stream, c, xs, wr, tp, za, zw, sa,
                       sw, bias, out, M, N, L, (const uint32_t*)nullptr);
    return hipGetLastError();
}

// The same pass queued behind a kernel that normally produced `out` itself: it runs only when *gate != 0.
hipError_t launch_dequant_gated(const float* c, const float* xs, const float* wr, const float* tp, const float* za, const float* zw,
                                const float* sa, const float* sw, const float* bias, float* out, int M, int N, int L,
                                const uint32_t* gate, hipStream_t stream) {
    hipLaunchKernelGGL(dequant_rows_to_nchw_kernel, dim3((M + 127) / 128, (N + 31) / 32), dim3(256), 0, stream, c, xs, wr, tp, za, zw, sa,
                       sw, bias, out, M, N, L, gate);
    return hipGetLastError();
}

hipError_t launch_dequant_grad(const float* g, const float* sa, const float* sw, float* gc, int M, int N, int L, hipStream_t stream) {
    hipLaunchKernelGGL(dequant_grad_nchw_to_rows_kernel, dim3((M + 127) / 128, (N + 31) / 32), dim3(256), 0, stream, g, sa, sw, gc, M, N, L);
    return hipGetLastError();
}

}  // namespace amr
