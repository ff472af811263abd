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

// ------------------------------------------------------------------------------------------ col2im
// Adjoint of the window extraction for the input gradient of the LUT convolution: cols [B][C*kh*kw][oh*ow] (the
// image-major layout gradA writes) -> x [B,C,H,W], x[b,c,y,x] = sum over the taps (i,j) whose window position
// (oy,ox) = ((y + pad - i*dil)/stride, (x + pad - j*dil)/stride) exists.  What the reference gets from autograd
// through F.unfold (self_ops/ops_py/approx_ops.py:558); a gather, so no atomics and a fixed summation order.
// One thread per input pixel; consecutive threads read consecutive window positions of the same tap row.
__global__ __launch_bounds__(256) void col2im_f32_kernel(const float* __restrict__ cols, float* __restrict__ x, int C, int H, int W,
                                                         int kh, int kw, int stride, int pad, int dil, int oh, int ow, size_t total) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int xx = (int)(idx % W);
    size_t r = idx / W;
    const int yy = (int)(r % H);
    r /= H;
    const int c = (int)(r % C);
    const size_t b = r / C;
    const size_t L = (size_t)oh * ow;
    const float* base = cols + (b * C + c) * (size_t)(kh * kw) * L;
    float acc = 0.f;
    for (int i = 0; i < kh; ++i) {
        const int ty = yy + pad - i * dil;
        if (ty < 0 || ty % stride != 0) continue;
        const int oy = ty / stride;
        if (oy >= oh) continue;
        for (int j = 0; j < kw; ++j) {
            const int tx = xx + pad - j * dil;
            if (tx < 0 || tx % stride != 0) continue;
            const int ox = tx / stride;
            if (ox >= ow) continue;
            acc += base[(size_t)(i * kw + j) * L + (size_t)oy * ow + ox];
        }
    }
    x[idx] = acc;
}

hipError_t launch_col2im_f32(const float* cols, float* x, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil,
                             int oh, int ow, hipStream_t stream) {
    const size_t total = (size_t)B * C * H * W;
    hipLaunchKernelGGL(col2im_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, cols, x, C, H, W, kh, kw,
                       stride, pad, dil, oh, ow, total);
    return hipGetLastError();
}

}  // namespace amr
