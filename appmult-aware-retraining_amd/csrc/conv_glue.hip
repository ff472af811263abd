// Glue of the quantised LUT convolution on uint8 codes, gfx950: the steps either side of the LUT GEMM in the
// reference's ApproxConv2d.forward (micronet+/app_layers.py:147-183) and approx_conv2d_op
// (self_ops/ops_py/approx_ops.py:556-571), without the float32 code tensors the reference passes between them.
//
//   quantize_nhwc_kernel     x [B,C,H,W] float32 -> codes [B*H*W, C] uint8 (pixel-major: the C codes of a pixel are
//                            adjacent), inside [B,C,H,W] uint8 (1 where the rounded value lay in [0, qmax]: the mask of
//                            the straight-through backward), xs [B*H*W] float32 (sum of a pixel's codes over the channels:
//                            the operand of the zero-point term conv(X, Zw))
//   im2col_nhwc_kernel       codes -> A [B*oh*ow, kh*kw*C] uint8, column k = (i*kw + j)*C + c ("tap-major": a window row is
//                            kh*kw runs of C adjacent bytes, each a pixel's codes or zeros)
//   conv_input_grad_kernel   the adjoint, with the quantiser's backward in the same pass:
//                            gx[b,c,y,x] = inside ? (sum over taps of cols[b][tap*C + c][pos(tap)] + zw * sum over taps of
//                            t[b][pos(tap)]) / scale : 0
//   dequant_grad_rowsum      g [B,N,L] -> g_rows [B*L, N] = (s_a*s_w) * g (transposed) and t[m] = sum_n g_rows[m, n]
//
// The order of the GEMM's k index is free as long as A's columns and B's rows agree; the tap-major order makes a window
// row a concatenation of contiguous pixel-code runs (coalesced copies instead of a byte gather) and puts the C channels of
// one tap side by side.
#include "amr_common.h"

namespace amr {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Same arithmetic as quant_code of the float quantiser (quantize.hip): q = x / s - zp, round half to even, inside = the
// rounded value lies in [0, qmax], code = clamp.  A NaN (also the inf - inf of an infinite q) gives code 0, inside 0.
__device__ __forceinline__ uint32_t quant_code_u8(float x, float s, float zp, float qmax, uint32_t* inside) {
    const float q = x / s - zp;
    const float r = __builtin_isinf(q) ? __builtin_nanf("") : rintf(q);
    *inside = (r >= 0.f) && (r <= qmax) ? 1u : 0u;
    const float cl = fminf(fmaxf(r, 0.f), qmax);      // (fmaxf drops a NaN: 0)
    return (uint32_t)cl;
}

// grid: ceil(B*L / 64) workgroups of 256 threads; LDS 64 x (CB + 16) bytes, CB = min(C rounded up to 16, 512).
// Lane = one of 64 consecutive pixels m = b*L + pix, wave w takes channels w, w + 4, ... of a block of CB channels:
// a wave's load covers 64 neighbouring pixels of one channel (256 B), the codes go to LDS [pixel][channel] and leave as
// 16-byte pieces of the pixel rows.
constexpr int kQnCB = 512;
__global__ __launch_bounds__(256) void quantize_nhwc_kernel(const float* __restrict__ x, const float* __restrict__ scale,
                                                            const float* __restrict__ zp_neg, float qmax,
                                                            uint8_t* __restrict__ codes, uint8_t* __restrict__ inside,
                                                            float* __restrict__ xs, int C, int L, long M, int relu) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float part[4][64];
    const float s = *scale, zp = *zp_neg;
    const int lane = threadIdx.x & 63, wave = uniform(threadIdx.x >> 6);
    const long m0 = (long)blockIdx.x * 64;
    const long m = min(m0 + lane, M - 1);
    const bool live = m0 + lane < M;
    const long b = m / L;
    const int pix = (int)(m - b * L);
    const float* xp = x + (size_t)b * C * L + pix;
    uint8_t* ip = inside + (size_t)b * C * L + pix;
    float sum = 0.f;
    for (int cb = 0; cb < C; cb += kQnCB) {
        const int cn = min(kQnCB, C - cb);
        const int pitch = ((cn + 15) & ~15) + 16;
        if (cb) __syncthreads();
        for (int c0 = wave; c0 < cn; c0 += 16) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = xp[(size_t)(cb + min(c0 + 4 * u, cn - 1)) * L];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + 4 * u;
                if (c < cn) {
                    uint32_t in;
                    // relu: the quantiser of max(x, 0); its backward passes a gradient where x > 0 and the code was in range
                    const float xv = relu ? (v[u] < 0.f ? 0.f : v[u]) : v[u];
                    const uint32_t code = quant_code_u8(xv, s, zp, qmax, &in);
                    if (relu && !(v[u] > 0.f)) in = 0u;
                    smem[lane * pitch + c] = (unsigned char)code;
                    if (live) ip[(size_t)(cb + c) * L] = (unsigned char)in;
                    sum += (float)code;
                }
            }
        }
        __syncthreads();
        const int rows = (int)min((long)64, M - m0);
        if ((C & 15) == 0) {
            const int ppr = cn >> 4;                                  // 16-byte pieces per pixel row
            for (int p = threadIdx.x; p < rows * ppr; p += 256) {
                const int r = p / ppr, o = p - r * ppr;
                *reinterpret_cast<u32x4*>(codes + (size_t)(m0 + r) * C + cb + 16 * o) = *reinterpret_cast<const u32x4*>(smem + r * pitch + 16 * o);
            }
        } else {
            for (int p = threadIdx.x; p < rows * cn; p += 256) {
                const int r = p / cn, o = p - r * cn;
                codes[(size_t)(m0 + r) * C + cb + o] = smem[r * pitch + o];
            }
        }
    }
    // a pixel's codes summed over all channels: the four waves' shares, added in a fixed order (integers below 2^24: exact)
    part[wave][lane] = sum;
    __syncthreads();
    if (wave == 0 && live) xs[m] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}

hipError_t launch_quantize_nhwc(const float* x, const float* scale, const float* zp_neg, float qmax, uint8_t* codes, uint8_t* inside,
                                float* xs, long B, int C, int L, hipStream_t stream, int relu) {
    const long M = B * L;
    const int cn = C < kQnCB ? C : kQnCB;
    const size_t lds = 64 * (size_t)(((cn + 15) & ~15) + 16);
    hipLaunchKernelGGL(quantize_nhwc_kernel, dim3((unsigned)((M + 63) / 64)), dim3(256), lds, stream, x, scale, zp_neg, qmax, codes,
                       inside, xs, C, L, M, relu);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ im2col, pixel-major codes
// One thread per 16 bytes of A (C % 16 == 0) or per byte: row m = (b, oy, ox), run `tap`, bytes c..c+15 = the codes of input
// pixel (oy*stride - pad + i*dil, ox*stride - pad + j*dil), zeros outside the image (code 0, as F.pad(value=0) gives the
// reference, self_ops/ops_py/approx_ops.py:556).  Consecutive threads write consecutive pieces of A.
// blockIdx.y = a slab of `slab_rows` rows holding fewer than 2^23 pieces, so that every division of the index arithmetic
// runs on a small number through a reciprocal (the 64-bit divisions of a flat index cost more than the copy).
template <int VEC>
__global__ __launch_bounds__(256) void im2col_nhwc_kernel(const uint8_t* __restrict__ codes, uint8_t* __restrict__ A, int C, int H,
                                                          int W, int kh, int kw, int stride, int pad, int dil, int oh, int ow,
                                                          long M, int slab_rows) {
    const int cpp = C / VEC;                               // pieces per run
    const int ppr = kh * kw * cpp;                         // pieces per row of A
    const long m0 = (long)blockIdx.y * slab_rows;          // first row of the slab (uniform: scalar arithmetic)
    const int rows = (int)min((long)slab_rows, M - m0);
    const int e = (int)(blockIdx.x * 256u + threadIdx.x);
    if (e >= rows * ppr) return;
    const long line0 = m0 / ow;                            // (b, oy) of the slab's first row
    const int ox0 = (int)(m0 - line0 * ow);
    const long b0 = line0 / oh;
    const int oy0 = (int)(line0 - b0 * oh);
    const float inv_ppr = 1.0f / (float)ppr, inv_cpp = 1.0f / (float)cpp, inv_kw = 1.0f / (float)kw, inv_ow = 1.0f / (float)ow,
                inv_oh = 1.0f / (float)oh;
    const int ml = div_small(e, ppr, inv_ppr);
    const int p = e - ml * ppr;
    const int tap = div_small(p, cpp, inv_cpp);
    const int piece = p - tap * cpp;
    const int i = div_small(tap, kw, inv_kw), j = tap - i * kw;
    const int xs = ox0 + ml;                               // < 2^23 + ow
    const int dl = div_small(xs, ow, inv_ow);
    const int ox = xs - dl * ow;
    const int ys = oy0 + dl;
    const int db = div_small(ys, oh, inv_oh);
    const int oy = ys - db * oh;
    const size_t b = (size_t)(b0 + db);
    const int y = oy * stride - pad + i * dil, xx = ox * stride - pad + j * dil;
    const bool in = y >= 0 && y < H && xx >= 0 && xx < W;
    const size_t src = ((b * H + (in ? y : 0)) * W + (in ? xx : 0)) * C + (size_t)piece * VEC;
    const size_t dst = ((size_t)m0 * ppr + (size_t)e) * VEC;
    if constexpr (VEC == 16) {
        u32x4 v = *reinterpret_cast<const u32x4*>(codes + src);
        if (!in) v = u32x4{0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(A + dst) = v;
    } else {
        A[dst] = in ? codes[src] : (uint8_t)0;
    }
}

hipError_t launch_im2col_nhwc(const uint8_t* codes, uint8_t* A, long B, int C, int H, int W, int kh, int kw, int stride, int pad,
                              int dil, int oh, int ow, hipStream_t stream) {
    const size_t bytes = (size_t)B * oh * ow * kh * kw * C;
    const long M = B * oh * ow;
    if (bytes == 0) return hipSuccess;
    // slabs of rows with at most 2^22 pieces each (the reciprocal divisions are exact below 2^23; ox0 + row stays below it)
    const bool vec = (C & 15) == 0 && (((uintptr_t)codes | (uintptr_t)A) & 15) == 0;
    const long ppr = (long)kh * kw * (vec ? C / 16 : C);
    if (ppr > (1L << 22) || ow > (1 << 20) || oh > (1 << 20)) return hipErrorInvalidValue;
    long slab_rows = (1L << 22) / ppr;
    if (slab_rows > M) slab_rows = M;
    const long slabs = (M + slab_rows - 1) / slab_rows;
    if (slabs > 65535) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((slab_rows * ppr + 255) / 256), (unsigned)slabs);
    if (vec)
        hipLaunchKernelGGL((im2col_nhwc_kernel<16>), grid, dim3(256), 0, stream, codes, A, C, H, W, kh, kw, stride, pad, dil, oh, ow, M,
                           (int)slab_rows);
    else
        hipLaunchKernelGGL((im2col_nhwc_kernel<1>), grid, dim3(256), 0, stream, codes, A, C, H, W, kh, kw, stride, pad, dil, oh, ow, M,
                           (int)slab_rows);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ input gradient
// One thread per input pixel (b, c, y, x), consecutive threads along x: the loads of all taps are issued at once
// (addresses of taps that do not exist are clamped and their values dropped), fixed summation order, no atomics.
//   cols   [B][kh*kw*C][L] float32, tap-major k (what the GEMM's gradA writes image-major), or nullptr: `gx` already holds
//          the sum over the taps (the convolution-shaped gradA kernel wrote it) and is finished in place
//   t      [B][L] float32, the row sums of the GEMM's output gradient; zw: device scalar
//   inside [B,C,H,W] uint8, scale: device scalar (the quantiser's)
template <int KH, int KW, int STRIDE>
__global__ __launch_bounds__(256) void conv_input_grad_kernel(const float* __restrict__ cols, const float* __restrict__ t,
                                                              const float* __restrict__ zw_p, const uint8_t* __restrict__ inside,
                                                              const float* __restrict__ scale_p, float* __restrict__ gx, int C,
                                                              int H, int W, int kh_rt, int kw_rt, int stride_rt, int pad, int dil,
                                                              int oh, int ow, size_t total, const uint32_t* __restrict__ gate,
                                                              int gate_mode) {
    // (32-bit index arithmetic inside an image; the images of the batch on blockIdx.y, strided when there are more than the grid holds)
    const uint32_t per_image = (uint32_t)C * (uint32_t)H * (uint32_t)W;
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= per_image) return;
    const int kh = KH ? KH : kh_rt, kw = KW ? KW : kw_rt, stride = STRIDE ? STRIDE : stride_rt;
    const int xx = (int)(e % (uint32_t)W);
    const uint32_t r = e / (uint32_t)W;
    const int yy = (int)(r % (uint32_t)H);
    const int c = (int)(r / (uint32_t)H);
    const size_t L = (size_t)oh * ow;
    for (size_t b = blockIdx.y; b * per_image < total; b += gridDim.y) {
    const size_t idx = b * per_image + e;
    // gate_mode 1: the pass behind a kernel that left the tap sums in gx -- when *gate says that kernel could not do its work,
    // this pass leaves gx alone (a recomputation is queued behind, gate_mode 2) or, gate_mode 3, marks every element NaN;
    // gate_mode 2: runs only when *gate is set.
    if (gate_mode != 0) {
        const bool raised = *gate != 0u;
        if (gate_mode == 2 && !raised) return;
        if (gate_mode == 1 && raised) return;
        if (gate_mode == 3 && raised) { gx[idx] = __builtin_nanf(""); continue; }
    }
    const float* base = cols ? cols + (b * (size_t)(kh * kw) * C + c) * L : nullptr;
    const float* tb = t + b * L;
    float acc = 0.f, tsum = 0.f;
    if constexpr (KH != 0) {
        float v[KH * KW], tv[KH * KW];
        bool ok[KH * KW];
#pragma unroll
        for (int i = 0; i < KH; ++i) {
            const int ty = yy + pad - i * dil;
            const int oy = ty / stride;
            const bool oky = ty >= 0 && (stride == 1 || ty % stride == 0) && oy < oh;
#pragma unroll
            for (int j = 0; j < KW; ++j) {
                const int tx = xx + pad - j * dil;
                const int ox = tx / stride;
                const int tap = i * KW + j;
                ok[tap] = oky && tx >= 0 && (stride == 1 || tx % stride == 0) && ox < ow;
                const size_t pos = ok[tap] ? (size_t)oy * ow + ox : 0;
                v[tap] = base ? base[(size_t)tap * C * L + pos] : 0.f;
                tv[tap] = tb[pos];
            }
        }
#pragma unroll
        for (int tap = 0; tap < KH * KW; ++tap) {
            acc += ok[tap] ? v[tap] : 0.f;
            tsum += ok[tap] ? tv[tap] : 0.f;
        }
    } else {
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
                const size_t pos = (size_t)oy * ow + ox;
                if (base) acc += base[(size_t)(i * kw + j) * C * L + pos];
                tsum += tb[pos];
            }
        }
    }
    if (!cols) acc = gx[idx];
    const float total_g = acc + *zw_p * tsum;
    gx[idx] = inside[idx] ? total_g / *scale_p : 0.f;
    }
}

// Stride 2 with an even image (3x3 / padding 1 or 1x1 / padding 0, no dilation): a thread owns one output position of one
// channel and the 2 x 2 input pixels it maps to.  Every tap's column is loaded exactly once (nine loads for the four
// pixels: the even/even pixel has one tap, the mixed ones two, the odd/odd one four), the pixels leave as two 8-byte
// stores.  Taps are added in ascending order like the general kernel.
template <int K>
__global__ __launch_bounds__(256) void conv_input_grad_s2_kernel(const float* __restrict__ cols, const float* __restrict__ t,
                                                                 const float* __restrict__ zw_p, const uint8_t* __restrict__ inside,
                                                                 const float* __restrict__ scale_p, float* __restrict__ gx, int C,
                                                                 int oh, int ow, long B) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const uint32_t per_image = (uint32_t)C * (uint32_t)oh * (uint32_t)ow;
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= per_image) return;
    const int ox = (int)(e % (uint32_t)ow);
    const uint32_t r = e / (uint32_t)ow;
    const int oy = (int)(r % (uint32_t)oh);
    const int c = (int)(r / (uint32_t)oh);
    const size_t L = (size_t)oh * ow, CL = (size_t)C * L;
    const int W = 2 * ow;
    const float zw = *zw_p, scale = *scale_p;
    const bool right = ox + 1 < ow, down = oy + 1 < oh;
    const size_t p00 = (size_t)oy * ow + ox;
    const size_t p01 = right ? p00 + 1 : p00, p10 = down ? p00 + ow : p00, p11 = p10 + (right ? 1 : 0);
    for (long b = blockIdx.y; b < B; b += gridDim.y) {
        const float* base = cols + ((size_t)b * (K * K) * C + c) * L;
        const float* tb = t + (size_t)b * L;
        float a00, a01, a10, a11, s00, s01, s10, s11;
        if constexpr (K == 1) {
            a00 = base[p00];
            s00 = tb[p00];
            a01 = a10 = a11 = s01 = s10 = s11 = 0.f;
        } else {
            // tap (i, j) reaches pixel (2*oy' + i - 1, 2*ox' + j - 1) from output position (oy', ox')
            const float v0 = base[0 * CL + p11], v1 = base[1 * CL + p10], v2 = base[2 * CL + p10];
            const float v3 = base[3 * CL + p01], v4 = base[4 * CL + p00], v5 = base[5 * CL + p00];
            const float v6 = base[6 * CL + p01], v7 = base[7 * CL + p00], v8 = base[8 * CL + p00];
            const float t00 = tb[p00], t01 = right ? tb[p01] : 0.f, t10 = down ? tb[p10] : 0.f, t11 = right && down ? tb[p11] : 0.f;
            a00 = v4;
            s00 = t00;
            a01 = (right ? v3 : 0.f) + v5;                      // pixel (2oy, 2ox+1): taps (1,0) from ox+1 and (1,2) from ox
            s01 = t01 + t00;
            a10 = (down ? v1 : 0.f) + v7;                       // pixel (2oy+1, 2ox): taps (0,1) from oy+1 and (2,1) from oy
            s10 = t10 + t00;
            a11 = (((right && down ? v0 : 0.f) + (down ? v2 : 0.f)) + (right ? v6 : 0.f)) + v8;
            s11 = ((t11 + t10) + t01) + t00;
        }
        const size_t o = (((size_t)b * C + c) * (2 * oh) + 2 * oy) * W + 2 * ox;
        const uint16_t in0 = *reinterpret_cast<const uint16_t*>(inside + o), in1 = *reinterpret_cast<const uint16_t*>(inside + o + W);
        f32x2 r0, r1;
        r0.x = (in0 & 0xff) ? (a00 + zw * s00) / scale : 0.f;
        r0.y = (in0 >> 8) ? (a01 + zw * s01) / scale : 0.f;
        r1.x = (in1 & 0xff) ? (a10 + zw * s10) / scale : 0.f;
        r1.y = (in1 >> 8) ? (a11 + zw * s11) / scale : 0.f;
        *reinterpret_cast<f32x2*>(gx + o) = r0;
        *reinterpret_cast<f32x2*>(gx + o + W) = r1;
    }
}

hipError_t launch_conv_input_grad(const float* cols, const float* t, const float* zw, const uint8_t* inside, const float* scale,
                                  float* gx, long B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil, int oh, int ow,
                                  hipStream_t stream, const uint32_t* gate = nullptr, int gate_mode = 0) {
    const size_t total = (size_t)B * C * H * W;
    if (total == 0) return hipSuccess;
    const unsigned rows = (unsigned)(B < 32768 ? B : 32768);
    if ((size_t)C * H * W > 0x7fffffffull) return hipErrorInvalidValue;      // (32-bit index inside an image)
    if (cols && gate_mode == 0 && stride == 2 && dil == 1 && H == 2 * oh && W == 2 * ow && kh == kw &&
        ((kh == 3 && pad == 1) || (kh == 1 && pad == 0)) && ((uintptr_t)gx & 7) == 0 && ((uintptr_t)inside & 1) == 0) {
        const dim3 g2((unsigned)(((size_t)C * oh * ow + 255) / 256), rows);
        if (kh == 3) hipLaunchKernelGGL((conv_input_grad_s2_kernel<3>), g2, dim3(256), 0, stream, cols, t, zw, inside, scale, gx, C, oh, ow, B);
        else hipLaunchKernelGGL((conv_input_grad_s2_kernel<1>), g2, dim3(256), 0, stream, cols, t, zw, inside, scale, gx, C, oh, ow, B);
        return hipGetLastError();
    }
    const dim3 grid((unsigned)(((size_t)C * H * W + 255) / 256), rows);
#define AMR_CIG(KH, KW, S)                                                                                                        \
    hipLaunchKernelGGL((conv_input_grad_kernel<KH, KW, S>), grid, dim3(256), 0, stream, cols, t, zw, inside, scale, gx, C, H, W, kh, kw, \
                       stride, pad, dil, oh, ow, total, gate, gate_mode)
    if (kh == 3 && kw == 3 && stride == 1) AMR_CIG(3, 3, 1);
    else if (kh == 3 && kw == 3 && stride == 2) AMR_CIG(3, 3, 2);
    else if (kh == 1 && kw == 1 && stride == 1) AMR_CIG(1, 1, 1);
    else if (kh == 1 && kw == 1 && stride == 2) AMR_CIG(1, 1, 2);
    else AMR_CIG(0, 0, 0);
#undef AMR_CIG
    return hipGetLastError();
}

// zt[b][y][x] = sum of t[b][pos] over the output positions a 3x3 / stride 1 / padding 1 window connects pixel (y, x) to
// (ascending tap order): the channel-independent part of the input gradient, for the kernel that finishes the gradient in
// its own store.
__global__ __launch_bounds__(256) void window_sums_3x3_kernel(const float* __restrict__ t, float* __restrict__ zt, int H, int W, size_t total) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int x = (int)(idx % W);
    const int y = (int)((idx / W) % H);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int oy = y + 1 - i, ox = x + 1 - j;
            const bool ok = oy >= 0 && oy < H && ox >= 0 && ox < W;
            const float v = t[ok ? idx + (size_t)((1 - i) * W + (1 - j)) : idx];
            acc += ok ? v : 0.f;
        }
    zt[idx] = acc;
}

hipError_t launch_window_sums_3x3(const float* t, float* zt, long B, int H, int W, hipStream_t stream) {
    const size_t total = (size_t)B * H * W;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(window_sums_3x3_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, t, zt, H, W, total);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ weight side of the layer
// Weight operand of the quantised LUT convolution in one launch (the reference: quantize_v2 on the weights, the cast and the
// transposes in front of the GEMM, and the zero-point convolution conv(Za, W); micronet+/app_layers.py:173,179 and
// self_ops/ops_py/approx_ops.py:560-561):
//   Bt[(tap*C + c)*N + n] = code of w[n][c][tap]            (uint8, rows in tap-major order)
//   inside[n][c][tap]     = the rounded value lay in [0, qmax] (mask of the straight-through backward)
//   w_resp[n][pos]        = sum over taps of (sum over c of the codes) * tapmask[tap][pos]
// One workgroup per output channel n.  The sums are integers below 2^24: exact in float32 in any order.
constexpr int kWpMaxTaps = 64;
__global__ __launch_bounds__(256) void conv_weight_prepare_kernel(const float* __restrict__ w, const float* __restrict__ scale,
                                                                  const float* __restrict__ zp_neg, float qmax,
                                                                  const float* __restrict__ tapmask, uint8_t* __restrict__ Bt,
                                                                  uint8_t* __restrict__ inside, float* __restrict__ w_resp, int N, int C,
                                                                  int T, int L) {
    __shared__ float wsum[kWpMaxTaps];
    const int n = blockIdx.x;
    const float s = *scale, zp = *zp_neg;
    if (threadIdx.x < kWpMaxTaps) wsum[threadIdx.x] = 0.f;
    __syncthreads();
    const int per_n = C * T;
    const float* wn = w + (size_t)n * per_n;
    for (int idx = threadIdx.x; idx < per_n; idx += 256) {
        const int c = idx / T, tap = idx - c * T;
        uint32_t in;
        const uint32_t code = quant_code_u8(wn[idx], s, zp, qmax, &in);
        Bt[((size_t)tap * C + c) * N + n] = (uint8_t)code;
        inside[(size_t)n * per_n + idx] = (uint8_t)in;
        atomicAdd(&wsum[tap], (float)code);         // (LDS; integer-valued: any order gives the same float)
    }
    __syncthreads();
    for (int pos = threadIdx.x; pos < L; pos += 256) {
        float acc = 0.f;
        for (int tap = 0; tap < T; ++tap) acc += wsum[tap] * tapmask[(size_t)tap * L + pos];
        w_resp[(size_t)n * L + pos] = acc;
    }
}

hipError_t launch_conv_weight_prepare(const float* w, const float* scale, const float* zp_neg, float qmax, const float* tapmask,
                                      uint8_t* Bt, uint8_t* inside, float* w_resp, int N, int C, int T, int L, hipStream_t stream) {
    hipLaunchKernelGGL(conv_weight_prepare_kernel, dim3(N), dim3(256), 0, stream, w, scale, zp_neg, qmax, tapmask, Bt, inside, w_resp, N, C,
                       T, L);
    return hipGetLastError();
}

// Gradient of the zero-point term Za * w_resp, summed over the batch and folded onto the taps:
//   g_wr[n][pos] = (*z_a * (*s_a * *s_w)) * sum over b of g[b][n][pos]
//   gz[p][n][tap] = sum over the positions pos of block p (64 positions each) of g_wr[n][pos] * tapmask[tap][pos]
// (the consumer, the weight-gradient kernel below, adds the blocks in ascending order).  Two launches, fixed summation order.  First S segments of the batch into partial sums (a thread owns four neighbouring
// elements and walks its segment with four loads in flight); then one workgroup per output channel n and block of positions adds the
// segments in ascending order (threads side by side along the positions, segment lanes beside them when the block is
// short), scales, and reduces against the tap masks, one tap per wave at a time.
__global__ __launch_bounds__(256) void batch_sum_partial_kernel(const float* __restrict__ g, float* __restrict__ partial, int B, size_t inner,
                                                                int seg_len) {
    const size_t j4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (j4 >= inner) return;
    const int b0 = blockIdx.y * seg_len, b1 = min(B, b0 + seg_len);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const bool vec = j4 + 3 < inner && (inner & 3) == 0;
    if (vec) {
        int b = b0;
        for (; b + 3 < b1; b += 4) {
            f32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f32x4*>(g + (size_t)(b + u) * inner + j4);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc = acc + v[u];
        }
        for (; b < b1; ++b) acc = acc + *reinterpret_cast<const f32x4*>(g + (size_t)b * inner + j4);
        *reinterpret_cast<f32x4*>(partial + (size_t)blockIdx.y * inner + j4) = acc;
    } else {
        for (int e = 0; e < 4 && j4 + e < inner; ++e) {
            float a = 0.f;
            for (int b = b0; b < b1; ++b) a += g[(size_t)b * inner + j4 + e];
            partial[(size_t)blockIdx.y * inner + j4 + e] = a;
        }
    }
}

constexpr int kBsChunk = 64;        // positions of one channel per workgroup of the folding kernel (four lanes of segments beside them)
__global__ __launch_bounds__(256) void batch_sum_taps_kernel(const float* __restrict__ partial, const float* __restrict__ za_p,
                                                             const float* __restrict__ sa_p, const float* __restrict__ sw_p,
                                                             const float* __restrict__ tapmask, float* __restrict__ g_wr,
                                                             float* __restrict__ gz_parts, size_t inner, int N, int L, int T, int segs) {
    __shared__ float part[256];
    __shared__ float v[kBsChunk];
    const int n = blockIdx.x, lane = threadIdx.x & 63, wave = uniform(threadIdx.x >> 6);
    const int p0 = blockIdx.y * kBsChunk;
    const int cn = min(kBsChunk, L - p0);
    const float scale = __fmul_rn(*za_p, __fmul_rn(*sa_p, *sw_p));
    // P threads along the positions (a power of two, 16..64), SP = 256 / P lanes of segments beside them
    int P = 16;
    while (P < cn) P <<= 1;
    const int SP = 256 / P;
    const int pp = threadIdx.x & (P - 1), sp = threadIdx.x / P;
    {
        float acc = 0.f;
        if (pp < cn) {
            const float* src = partial + (size_t)n * L + p0 + pp;
            int sgm = sp;
            for (; sgm + 3 * SP < segs; sgm += 4 * SP) {
                const float a0 = src[(size_t)sgm * inner], a1 = src[(size_t)(sgm + SP) * inner];
                const float a2 = src[(size_t)(sgm + 2 * SP) * inner], a3 = src[(size_t)(sgm + 3 * SP) * inner];
                acc = (((acc + a0) + a1) + a2) + a3;
            }
            for (; sgm < segs; sgm += SP) acc += src[(size_t)sgm * inner];
        }
        part[threadIdx.x] = acc;                                    // = part[sp * P + pp]
    }
    __syncthreads();
    if (threadIdx.x < cn) {
        float acc = part[threadIdx.x];
        for (int q = 1; q < SP; ++q) acc += part[q * P + threadIdx.x];
        acc = __fmul_rn(scale, acc);
        v[threadIdx.x] = acc;
        if (g_wr) g_wr[(size_t)n * L + p0 + threadIdx.x] = acc;
    }
    __syncthreads();
    for (int tap = wave; tap < T; tap += 4) {
        float acc = 0.f;
        for (int pos = lane; pos < cn; pos += 64) acc += v[pos] * tapmask[(size_t)tap * L + p0 + pos];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
        if (lane == 0) gz_parts[((size_t)blockIdx.y * N + n) * T + tap] = acc;
    }
}

int batch_sum_parts(int L) { return (L + kBsChunk - 1) / kBsChunk; }

int batch_sum_segments(int B, size_t inner, int n_cu) {
    // enough workgroups to fill the device, at least 8 images per segment, at most 32 segments
    const size_t wg_per_seg = (inner / 4 + 255) / 256;
    int segs = (int)((4 * (size_t)n_cu + wg_per_seg - 1) / (wg_per_seg ? wg_per_seg : 1));
    if (segs > B / 8) segs = B / 8;
    if (segs > 32) segs = 32;
    return segs < 1 ? 1 : segs;
}

hipError_t launch_batch_sum_taps(const float* g, const float* za, const float* sa, const float* sw, const float* tapmask, float* g_wr,
                                 float* gz, float* partial, int B, int N, int L, int T, int n_cu, hipStream_t stream) {
    const size_t inner = (size_t)N * L;
    const int segs = batch_sum_segments(B, inner, n_cu);
    const int seg_len = (B + segs - 1) / segs;
    const int used = (B + seg_len - 1) / seg_len;
    hipLaunchKernelGGL(batch_sum_partial_kernel, dim3((unsigned)((inner / 4 + 256) / 256), used), dim3(256), 0, stream, g, partial, B, inner,
                       seg_len);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(batch_sum_taps_kernel, dim3(N, batch_sum_parts(L)), dim3(256), 0, stream, partial, za, sa, sw, tapmask, g_wr, gz, inner,
                       N, L, T, used);
    return hipGetLastError();
}

// Weight gradient of the layer, finished in one launch: the LUT gradient gBt [T*C][N] (tap-major rows, what gradB wrote), the
// zero-point term gz [parts][N][T] (blocks of positions, added here in ascending order) and the quantiser's straight-through
// backward:   gw[n][c][tap] = inside[n][c][tap] ? (gBt[(tap*C + c)*N + n] + sum over p of gz[p][n][tap]) / *scale : 0.
// A workgroup transposes a tile of all T taps x cb channels x 16 output channels through LDS: reads run along n (64 B per
// row of gBt), writes along (c, tap), T*cb adjacent floats per output channel.  cb shrinks until the grid fills the device.
constexpr int kWgRows = 128, kWgCols = 16;
__global__ __launch_bounds__(256) void conv_weight_grad_kernel(const float* __restrict__ gBt, const float* __restrict__ gz, int parts,
                                                               const uint8_t* __restrict__ inside, const float* __restrict__ scale,
                                                               float* __restrict__ gw, int N, int C, int T, int cb) {
    __shared__ float tile[kWgRows][kWgCols + 1];
    __shared__ float gzs[kWgCols][kWpMaxTaps];
    const int lane = threadIdx.x & 63, wave = uniform(threadIdx.x >> 6);
    const int n0 = blockIdx.x * kWgCols, c0 = blockIdx.y * cb;
    const int cn = min(cb, C - c0), rows = T * cn;
    const int n_here = min(kWgCols, N - n0);
    {
        const int nl = threadIdx.x & (kWgCols - 1);
        for (int rr = threadIdx.x / kWgCols; rr < rows; rr += 256 / kWgCols) {
            const int tap = rr / cn, cc = rr - tap * cn;
            tile[rr][nl] = nl < n_here ? gBt[((size_t)tap * C + c0 + cc) * N + n0 + nl] : 0.f;
        }
        for (int e = threadIdx.x; e < n_here * T; e += 256) {
            const int q = e / T, tap = e - q * T;
            float acc = gz[(size_t)(n0 + q) * T + tap];
            for (int p = 1; p < parts; ++p) acc += gz[((size_t)p * N + n0 + q) * T + tap];
            gzs[q][tap] = acc;
        }
    }
    __syncthreads();
    const float s = *scale;
    for (int nl = wave; nl < n_here; nl += 4) {
        const size_t row = ((size_t)(n0 + nl) * C + c0) * T;
        for (int j = lane; j < rows; j += 64) {
            const int cc = j / T, tap = j - cc * T;
            const float val = tile[tap * cn + cc][nl] + gzs[nl][tap];
            gw[row + j] = inside[row + j] ? val / s : 0.f;
        }
    }
}

hipError_t launch_conv_weight_grad(const float* gBt, const float* gz, int parts, const uint8_t* inside, const float* scale, float* gw,
                                   int N, int C, int T, int n_cu, hipStream_t stream) {
    const int n_tiles = (N + kWgCols - 1) / kWgCols;
    int cb = T >= kWgRows ? 1 : kWgRows / T;
    const long fill = (long)C * n_tiles / (n_cu > 0 ? n_cu : 256);           // channels per workgroup that still give one workgroup per CU
    if (cb > fill) cb = (int)(fill < 1 ? 1 : fill);
    if (cb > C) cb = C;
    hipLaunchKernelGGL(conv_weight_grad_kernel, dim3(n_tiles, (C + cb - 1) / cb), dim3(256), 0, stream, gBt, gz, parts, inside, scale, gw, N,
                       C, T, cb);
    return hipGetLastError();
}

// Queued behind a kernel that finished gx itself: marks every element NaN when *gate says that kernel met what it cannot
// serve (and nobody queued a recomputation); otherwise its few workgroups leave at once.
__global__ __launch_bounds__(256) void poison_if_raised_kernel(float* __restrict__ gx, size_t total, const uint32_t* __restrict__ gate) {
    if (*gate == 0u) return;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) gx[i] = __builtin_nanf("");
}

hipError_t launch_poison_if_raised(float* gx, size_t total, const uint32_t* gate, hipStream_t stream) {
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(poison_if_raised_kernel, dim3(256), dim3(256), 0, stream, gx, total, gate);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ output gradient to GEMM rows
// g [B,N,L] -> gc [B*L, N] = (s_a*s_w) * g transposed, t[m] = sum over n of gc[m, n] (added in ascending n).  A workgroup
// owns 128 rows m and walks all column blocks of 32 through 32 x 32 LDS tiles (reads run along pos, writes along n).
__global__ __launch_bounds__(256) void dequant_grad_rowsum_kernel(const float* __restrict__ g, const float* __restrict__ sa_p,
                                                                  const float* __restrict__ sw_p, float* __restrict__ gc,
                                                                  float* __restrict__ t, int M, int N, int L) {
    __shared__ float tile[4][32][33];
    __shared__ float rsum[128];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int m0 = blockIdx.x * 128;
    const float s = __fmul_rn(*sa_p, *sw_p);
    if (threadIdx.x < 128) rsum[threadIdx.x] = 0.f;
    for (int n0 = 0; n0 < N; n0 += 32) {
        float v[4][4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const int m = min(m0 + 32 * tt + tx, M - 1);
            const int b = m / L, pos = m - b * L;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = min(n0 + ty + 8 * r, N - 1);
                v[tt][r] = g[((size_t)b * N + n) * L + pos];
            }
        }
        __syncthreads();                      // the previous block's tiles have been read
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) tile[tt][tx][ty + 8 * r] = __fmul_rn(s, v[tt][r]);
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + 32 * tt + ty + 8 * r, n = n0 + tx;
                if (m < M && n < N) gc[(size_t)m * N + n] = tile[tt][ty + 8 * r][tx];
            }
        // row sums of this column block: thread = row, ascending n (every row's running sum has one owner)
        if (threadIdx.x < 128) {
            const int tt = threadIdx.x >> 5, row = threadIdx.x & 31;
            float acc = rsum[threadIdx.x];
            const int nn = min(32, N - n0);
            for (int e = 0; e < nn; ++e) acc += tile[tt][row][e];
            rsum[threadIdx.x] = acc;
        }
    }
    __syncthreads();
    if (threadIdx.x < 128 && m0 + (int)threadIdx.x < M) t[m0 + threadIdx.x] = rsum[threadIdx.x];
}

// The same with the batch sums of the zero-point gradient formed on the way (L % 128 == 0, N <= 32 NB): a workgroup owns 128
// positions and a segment of the batch, walks its images one after the other and keeps, per thread, the sums over those
// images of the 16 NB elements it loads per image; partial[seg][n][pos] is what batch_sum_partial_kernel would have written
// (raw sums of g, images in ascending order), so that the output gradient is read once instead of twice.
template <int NB>
__global__ __launch_bounds__(256) void dequant_grad_rowsum_batch_kernel(const float* __restrict__ g, const float* __restrict__ sa_p,
                                                                        const float* __restrict__ sw_p, float* __restrict__ gc,
                                                                        float* __restrict__ t, float* __restrict__ partial, int B, int N,
                                                                        int L, int seg_len) {
    __shared__ float tile[4][32][33];
    __shared__ float rsum[128];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int p0 = blockIdx.x * 128;
    const int b0 = blockIdx.y * seg_len, b1 = min(B, b0 + seg_len);
    const float s = __fmul_rn(*sa_p, *sw_p);
    float acc[NB][4][4];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[nb][tt][r] = 0.f;
    for (int b = b0; b < b1; ++b) {
        const size_t m0 = (size_t)b * L + p0;
        if (threadIdx.x < 128) rsum[threadIdx.x] = 0.f;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int n0 = 32 * nb;
            float v[4][4];
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = min(n0 + ty + 8 * r, N - 1);
                    v[tt][r] = g[((size_t)b * N + n) * L + p0 + 32 * tt + tx];
                }
            __syncthreads();                      // the previous block's tiles have been read
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    acc[nb][tt][r] += v[tt][r];
                    tile[tt][tx][ty + 8 * r] = __fmul_rn(s, v[tt][r]);
                }
            __syncthreads();
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + tx;
                    if (n < N) gc[(m0 + 32 * tt + ty + 8 * r) * N + n] = tile[tt][ty + 8 * r][tx];
                }
            if (threadIdx.x < 128) {
                const int tt = threadIdx.x >> 5, row = threadIdx.x & 31;
                float a = rsum[threadIdx.x];
                const int nn = min(32, N - n0);
                for (int e = 0; e < nn; ++e) a += tile[tt][row][e];
                rsum[threadIdx.x] = a;
            }
        }
        if (threadIdx.x < 128) t[m0 + threadIdx.x] = rsum[threadIdx.x];
    }
    float* out = partial + (size_t)blockIdx.y * N * L;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = 32 * nb + ty + 8 * r;
                if (n < N) out[(size_t)n * L + p0 + 32 * tt + tx] = acc[nb][tt][r];
            }
}

// Segments of the batch for the sums of the zero-point gradient, and whether the rows kernel forms them on the way.
int output_grad_segments(int B, int N, int L, int n_cu, bool* fused) {
    *fused = (L % 128) == 0 && N <= 128 && B >= 8;
    if (!*fused) return batch_sum_segments(B, (size_t)N * L, n_cu);
    const int pos_blocks = L / 128;
    int segs = (2 * n_cu + pos_blocks - 1) / pos_blocks;
    if (segs > B / 4) segs = B / 4;
    if (segs > 128) segs = 128;
    return segs < 1 ? 1 : segs;
}

// g_rows, t and (tapmask != nullptr) gz of one layer's output gradient: two launches where the rows kernel can form the
// batch sums, three otherwise.
hipError_t launch_output_grad(const float* g, const float* za, const float* sa, const float* sw, const float* tapmask, float* gc, float* t,
                              float* gz, float* partial, int B, int N, int L, int T, int n_cu, hipStream_t stream) {
    bool fused = false;
    const int segs = output_grad_segments(B, N, L, n_cu, &fused);
    if (!tapmask || !fused) {
        hipLaunchKernelGGL(dequant_grad_rowsum_kernel, dim3((B * L + 127) / 128), dim3(256), 0, stream, g, sa, sw, gc, t, B * L, N, L);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess || !tapmask) return e;
        return launch_batch_sum_taps(g, za, sa, sw, tapmask, nullptr, gz, partial, B, N, L, T, n_cu, stream);
    }
    const int seg_len = (B + segs - 1) / segs;
    const int used = (B + seg_len - 1) / seg_len;
    const dim3 grid(L / 128, used);
    if (N <= 32) hipLaunchKernelGGL((dequant_grad_rowsum_batch_kernel<1>), grid, dim3(256), 0, stream, g, sa, sw, gc, t, partial, B, N, L, seg_len);
    else if (N <= 64) hipLaunchKernelGGL((dequant_grad_rowsum_batch_kernel<2>), grid, dim3(256), 0, stream, g, sa, sw, gc, t, partial, B, N, L, seg_len);
    else hipLaunchKernelGGL((dequant_grad_rowsum_batch_kernel<4>), grid, dim3(256), 0, stream, g, sa, sw, gc, t, partial, B, N, L, seg_len);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(batch_sum_taps_kernel, dim3(N, batch_sum_parts(L)), dim3(256), 0, stream, partial, za, sa, sw, tapmask, (float*)nullptr, gz,
                       (size_t)N * L, N, L, T, used);
    return hipGetLastError();
}

hipError_t launch_dequant_grad_rowsum(const float* g, const float* sa, const float* sw, float* gc, float* t, int M, int N, int L,
                                      hipStream_t stream) {
    hipLaunchKernelGGL(dequant_grad_rowsum_kernel, dim3((M + 127) / 128), dim3(256), 0, stream, g, sa, sw, gc, t, M, N, L);
    return hipGetLastError();
}

}  // namespace amr
