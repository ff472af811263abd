// im2col of operand codes for the LUT convolution, gfx950.
//
// Replaces, for the LUT path, the pad + unfold + transpose + reshape + cast sequence of the reference's
// approx_conv2d_op (self_ops/ops_py/approx_ops.py:556-563 and :161-164): float32 code tensor
// x [B,C,H,W] (integer valued) -> uint8 A [B*oh*ow, C*kh*kw] in one pass.  Row m = (b, oy, ox), column
// k = c*kh*kw + i*kw + j, padding positions hold code 0 (as F.pad(value=0) does there).
//
// A workgroup transposes a tile of 64 consecutive rows x up to 512 columns through LDS: for one column
// the 64 lanes read 64 neighbouring pixels (coalesced), the finished tile is written out as contiguous
// row segments with 32-bit stores.
#include "amr_common.h"

namespace amr {

constexpr int kIm2colKC = 512;

__global__ __launch_bounds__(256) void im2col_u8_f32_kernel(const float* __restrict__ x, uint8_t* __restrict__ A, int C,
                                                            int H, int W, int kh, int kw, int stride, int pad, int dil, int oh,
                                                            int ow, int M, int K) {
    __shared__ __align__(4) uint8_t tile[64][kIm2colKC + 4];
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int m0 = blockIdx.x * 64;
    const int kc0 = blockIdx.y * kIm2colKC;
    const int kc = min(kIm2colKC, K - kc0);
    const int m = m0 + lane;
    const bool valid = m < M;
    const int mm = valid ? m : M - 1;
    const int b = mm / (oh * ow);
    const int r = mm - b * (oh * ow);
    const int oy = r / ow, ox = r - oy * ow;
    const int y0 = oy * stride - pad, x0 = ox * stride - pad;
    const float* xb = x + (size_t)b * C * H * W;
    const int khw = kh * kw;
    // Each wave takes every 4th column; kU columns per trip so that kU independent loads are in flight.
    // Out-of-image taps read a clamped (valid) address and are zeroed by a select: no divergent branch.
    constexpr int kU = 8;
    for (int kb = wave; kb < kc; kb += 4 * kU) {
        float v[kU];
        bool in[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int k = min(kc0 + kb + 4 * u, K - 1);   // wave-uniform: the divisions below are scalar
            const int c = k / khw;
            const int t = k - c * khw;
            const int i = t / kw, j = t - i * kw;
            const int yy = y0 + i * dil, xx = x0 + j * dil;
            in[u] = valid && yy >= 0 && yy < H && xx >= 0 && xx < W;
            const int yc = min(max(yy, 0), H - 1), xc = min(max(xx, 0), W - 1);
            v[u] = xb[((size_t)c * H + yc) * W + xc];
        }
#pragma unroll
        for (int u = 0; u < kU; ++u)
            if (kb + 4 * u < kc) tile[lane][kb + 4 * u] = in[u] ? (uint8_t)(int)v[u] : (uint8_t)0;
    }
    __syncthreads();
    const int rows = min(64, M - m0);
    if (((K | kc0) & 3) == 0 && (((uintptr_t)A) & 3) == 0) {
        const int dw = kc >> 2;              // kc is a multiple of 4 here
        for (int idx = threadIdx.x; idx < rows * dw; idx += 256) {
            const int rr = idx / dw, q = idx - rr * dw;
            *reinterpret_cast<uint32_t*>(A + (size_t)(m0 + rr) * K + kc0 + 4 * q) = *reinterpret_cast<const uint32_t*>(&tile[rr][4 * q]);
        }
    } else {
        for (int idx = threadIdx.x; idx < rows * kc; idx += 256) {
            const int rr = idx / kc, q = idx - rr * kc;
            A[(size_t)(m0 + rr) * K + kc0 + q] = tile[rr][q];
        }
    }
}

hipError_t launch_im2col_u8_f32(const float* x, uint8_t* A, int B, int C, int H, int W, int kh, int kw, int stride, int pad,
                                int dil, int oh, int ow, hipStream_t stream) {
    const long M = (long)B * oh * ow;
    const int K = C * kh * kw;
    dim3 grid((unsigned)((M + 63) / 64), (K + kIm2colKC - 1) / kIm2colKC);
    hipLaunchKernelGGL(im2col_u8_f32_kernel, grid, dim3(256), 0, stream, x, A, C, H, W, kh, kw, stride, pad, dil, oh, ow, (int)M, K);
    return hipGetLastError();
}

}  // namespace amr
