// im2col of operand codes for the LUT convolution, gfx950.
//
// Replaces, for the LUT path, the pad + unfold + transpose + reshape + cast sequence of the reference's
// approx_conv2d_op (self_ops/ops_py/approx_ops.py:556-563 and :161-164): float32 code tensor
// x [B,C,H,W] (integer valued) -> uint8 A [B*oh*ow, C*kh*kw] in one pass.  Row m = (b, oy, ox), column
// k = c*kh*kw + i*kw + j, padding positions hold code 0 (as F.pad(value=0) does there).
//
// A workgroup transposes a tile of 64 consecutive rows x up to 256 columns through LDS (256: the input pixels a tile
// reads nine times stay in the L1; 512 columns measured 15 % slower): for one column
// the 64 lanes read 64 neighbouring pixels (coalesced), four columns are packed into a dword, and the
// finished tile is written out as contiguous row segments with 32-bit stores.
#include "amr_common.h"

namespace amr {

constexpr int kIm2colKC = 256;

__global__ __launch_bounds__(256) void im2col_u8_f32_kernel(const float* __restrict__ x, uint8_t* __restrict__ A, int C,
                                                            int H, int W, int kh, int kw, int stride, int pad, int dil, int oh,
                                                            int ow, int M, int K) {
    __shared__ uint32_t tile[64][kIm2colKC / 4 + 1];     // 64 rows x 256 codes, one dword = four columns (+1: no bank conflicts)
    __shared__ int2 taps[kIm2colKC];                      // per column of the chunk: offset inside the image, (dy << 16 | dx)
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int m0 = blockIdx.x * 64;
    const int kc0 = blockIdx.y * kIm2colKC;
    const int kc = min(kIm2colKC, K - kc0);
    // the column -> (channel, tap) decomposition is done once per workgroup, not once per load
    const int n_taps = kh * kw;
    const bool few_taps = n_taps <= 32;
    for (int kk = threadIdx.x; kk < kIm2colKC; kk += 256) {
        const int k = min(kc0 + kk, K - 1);
        const int c = k / n_taps;
        const int t = k - c * n_taps;
        const int i = t / kw, j = t - i * kw;
        taps[kk] = make_int2((c * H + i * dil) * W + j * dil, few_taps ? t : (((i * dil) << 16) | (j * dil)));
    }
    const int m = m0 + lane;
    const bool valid = m < M;
    const int mm = valid ? m : M - 1;
    const int b = mm / (oh * ow);
    const int r = mm - b * (oh * ow);
    const int oy = r / ow, ox = r - oy * ow;
    const int y0 = oy * stride - pad, x0 = ox * stride - pad;
    const float* xb = x + (size_t)b * C * H * W + y0 * W + x0;      // window origin (may lie outside the image)
    // which taps of this row's window lie inside the image does not depend on the channel: one bit per tap, once per
    // row (windows of more than 32 taps test the coordinates of every element instead)
    uint32_t inside = 0;
    if (few_taps) {
        for (int t = 0; t < n_taps; ++t) {
            const int i = t / kw, j = t - i * kw;
            const int yy = y0 + i * dil, xx = x0 + j * dil;
            inside |= (uint32_t)(valid && yy >= 0 && yy < H && xx >= 0 && xx < W) << t;
        }
    }
    const int safe = -(y0 * W + x0);                                // the image's first pixel
    __syncthreads();
    // A wave takes every 4th group of four columns, four groups (16 loads in flight) per trip.  Taps outside the
    // image read the image's first pixel instead and are zeroed by a select: no divergent branch.  v_cvt_pk_u8_f32
    // converts and places a code in its byte of the dword in one instruction.
    const int quads = (kc + 3) >> 2;
    for (int q0 = wave; q0 < quads; q0 += 16) {
        float v[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int2 tp = taps[min(4 * (q0 + 4 * u) + e, kIm2colKC - 1)];      // wave-uniform address: one broadcast read
                bool in;
                if (few_taps) {
                    in = (inside >> tp.y) & 1u;
                } else {
                    const int yy = y0 + (tp.y >> 16), xx = x0 + (tp.y & 0xffff);
                    in = valid && yy >= 0 && yy < H && xx >= 0 && xx < W;
                }
                const float val = xb[in ? tp.x : safe];
                v[u][e] = in ? val : 0.f;
            }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int q = q0 + 4 * u;
            if (q < quads) {
                uint32_t w = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) w = __builtin_amdgcn_cvt_pk_u8_f32(v[u][e], e, w);
                tile[lane][q] = w;
            }
        }
    }
    __syncthreads();
    const int rows = min(64, M - m0);
    if (((K | kc0) & 3) == 0 && (((uintptr_t)A) & 3) == 0) {
        // kc is a multiple of 4 here: a wave writes the dwords of a row, 256 contiguous bytes per store
        for (int rr = wave; rr < rows; rr += 4)
            for (int q = lane; q < (kc >> 2); q += 64)
                *reinterpret_cast<uint32_t*>(A + (size_t)(m0 + rr) * K + kc0 + 4 * q) = tile[rr][q];
    } else {
        for (int rr = wave; rr < rows; rr += 4)
            for (int q = lane; q < kc; q += 64)
                A[(size_t)(m0 + rr) * K + kc0 + q] = (uint8_t)(tile[rr][q >> 2] >> (8 * (q & 3)));
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

// The same gather for the usual window sizes, without branches: every thread issues the loads of all its taps at once
// (addresses of taps that do not exist are clamped to the first entry and their values dropped), so that the kernel
// runs at the speed of its reads, 9 x the size of the result for a 3x3 window, instead of one dependent load after the
// other.  Same summation order as the generic kernel.
template <int KH, int KW, int STRIDE>
__global__ __launch_bounds__(256) void col2im_f32_taps_kernel(const float* __restrict__ cols, float* __restrict__ x, int C, int H, int W,
                                                              int pad, int dil, int oh, int ow, size_t total) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int xx = (int)(idx % W);
    size_t r = idx / W;
    const int yy = (int)(r % H);
    r /= H;                                   // = b * C + c
    const size_t L = (size_t)oh * ow;
    const float* base = cols + r * (size_t)(KH * KW) * L;
    float v[KH * KW];
    bool ok[KH * KW];
#pragma unroll
    for (int i = 0; i < KH; ++i) {
        const int ty = yy + pad - i * dil;
        const int oy = ty / STRIDE;
        const bool oky = ty >= 0 && (STRIDE == 1 || ty % STRIDE == 0) && oy < oh;
#pragma unroll
        for (int j = 0; j < KW; ++j) {
            const int tx = xx + pad - j * dil;
            const int ox = tx / STRIDE;
            const int tap = i * KW + j;
            ok[tap] = oky && tx >= 0 && (STRIDE == 1 || tx % STRIDE == 0) && ox < ow;
            v[tap] = base[ok[tap] ? (size_t)tap * L + (size_t)oy * ow + ox : 0];
        }
    }
    float acc = 0.f;
#pragma unroll
    for (int tap = 0; tap < KH * KW; ++tap) acc += ok[tap] ? v[tap] : 0.f;
    x[idx] = acc;
}

hipError_t launch_col2im_f32(const float* cols, float* x, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil,
                             int oh, int ow, hipStream_t stream) {
    const size_t total = (size_t)B * C * H * W;
    const dim3 grid((unsigned)((total + 255) / 256));
    if (total == 0) return hipSuccess;
    if (kh == 3 && kw == 3 && stride == 1)
        hipLaunchKernelGGL((col2im_f32_taps_kernel<3, 3, 1>), grid, dim3(256), 0, stream, cols, x, C, H, W, pad, dil, oh, ow, total);
    else if (kh == 3 && kw == 3 && stride == 2)
        hipLaunchKernelGGL((col2im_f32_taps_kernel<3, 3, 2>), grid, dim3(256), 0, stream, cols, x, C, H, W, pad, dil, oh, ow, total);
    else if (kh == 1 && kw == 1 && stride == 1)
        hipLaunchKernelGGL((col2im_f32_taps_kernel<1, 1, 1>), grid, dim3(256), 0, stream, cols, x, C, H, W, pad, dil, oh, ow, total);
    else if (kh == 1 && kw == 1 && stride == 2)
        hipLaunchKernelGGL((col2im_f32_taps_kernel<1, 1, 2>), grid, dim3(256), 0, stream, cols, x, C, H, W, pad, dil, oh, ow, total);
    else
    hipLaunchKernelGGL(col2im_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, cols, x, C, H, W, kh, kw,
                       stride, pad, dil, oh, ow, total);
    return hipGetLastError();
}

}  // namespace amr
