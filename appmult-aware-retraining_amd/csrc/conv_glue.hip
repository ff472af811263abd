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
                                                            float* __restrict__ xs, int C, int L, long M) {
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
                    const uint32_t code = quant_code_u8(v[u], s, zp, qmax, &in);
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
                                float* xs, long B, int C, int L, hipStream_t stream) {
    const long M = B * L;
    const int cn = C < kQnCB ? C : kQnCB;
    const size_t lds = 64 * (size_t)(((cn + 15) & ~15) + 16);
    hipLaunchKernelGGL(quantize_nhwc_kernel, dim3((unsigned)((M + 63) / 64)), dim3(256), lds, stream, x, scale, zp_neg, qmax, codes,
                       inside, xs, C, L, M);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ im2col, pixel-major codes
// One thread per 16 bytes of A (C % 16 == 0) or per byte: row m = (b, oy, ox), run `tap`, bytes c..c+15 = the codes of input
// pixel (oy*stride - pad + i*dil, ox*stride - pad + j*dil), zeros outside the image (code 0, as F.pad(value=0) gives the
// reference, self_ops/ops_py/approx_ops.py:556).  Consecutive threads write consecutive pieces of A.
template <int VEC>
__global__ __launch_bounds__(256) void im2col_nhwc_kernel(const uint8_t* __restrict__ codes, uint8_t* __restrict__ A, int C, int H,
                                                          int W, int kh, int kw, int stride, int pad, int dil, int oh, int ow,
                                                          size_t total) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cpp = C / VEC;                               // pieces per run
    const int taps = kh * kw;
    const int piece = (int)(idx % cpp);
    size_t r = idx / cpp;
    const int tap = (int)(r % taps);
    r /= taps;                                             // = m
    const int ox = (int)(r % ow);
    size_t r2 = r / ow;
    const int oy = (int)(r2 % oh);
    const size_t b = r2 / oh;
    const int i = tap / kw, j = tap - i * kw;
    const int y = oy * stride - pad + i * dil, xx = ox * stride - pad + j * dil;
    const bool in = y >= 0 && y < H && xx >= 0 && xx < W;
    const size_t src = ((b * H + (in ? y : 0)) * W + (in ? xx : 0)) * C + (size_t)piece * VEC;
    if constexpr (VEC == 16) {
        u32x4 v = *reinterpret_cast<const u32x4*>(codes + src);
        if (!in) v = u32x4{0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(A + idx * 16) = v;
    } else {
        A[idx] = in ? codes[src] : (uint8_t)0;
    }
}

hipError_t launch_im2col_nhwc(const uint8_t* codes, uint8_t* A, long B, int C, int H, int W, int kh, int kw, int stride, int pad,
                              int dil, int oh, int ow, hipStream_t stream) {
    const size_t bytes = (size_t)B * oh * ow * kh * kw * C;
    if (bytes == 0) return hipSuccess;
    if ((C & 15) == 0 && (((uintptr_t)codes | (uintptr_t)A) & 15) == 0) {
        const size_t total = bytes / 16;
        hipLaunchKernelGGL((im2col_nhwc_kernel<16>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, codes, A, C, H, W, kh,
                           kw, stride, pad, dil, oh, ow, total);
    } else {
        hipLaunchKernelGGL((im2col_nhwc_kernel<1>), dim3((unsigned)((bytes + 255) / 256)), dim3(256), 0, stream, codes, A, C, H, W, kh,
                           kw, stride, pad, dil, oh, ow, bytes);
    }
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
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    // gate_mode 1: the pass behind a kernel that left the tap sums in gx -- when *gate says that kernel could not do its work,
    // this pass leaves gx alone (a recomputation is queued behind, gate_mode 2) or, gate_mode 3, marks every element NaN;
    // gate_mode 2: runs only when *gate is set.
    if (gate_mode != 0) {
        const bool raised = *gate != 0u;
        if (gate_mode == 2 && !raised) return;
        if (gate_mode == 1 && raised) return;
        if (gate_mode == 3 && raised) { gx[idx] = __builtin_nanf(""); return; }
    }
    const int kh = KH ? KH : kh_rt, kw = KW ? KW : kw_rt, stride = STRIDE ? STRIDE : stride_rt;
    const int xx = (int)(idx % W);
    size_t r = idx / W;
    const int yy = (int)(r % H);
    r /= H;                                   // = b * C + c
    const int c = (int)(r % C);
    const size_t b = r / C;
    const size_t L = (size_t)oh * ow;
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

hipError_t launch_conv_input_grad(const float* cols, const float* t, const float* zw, const uint8_t* inside, const float* scale,
                                  float* gx, long B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil, int oh, int ow,
                                  hipStream_t stream, const uint32_t* gate = nullptr, int gate_mode = 0) {
    const size_t total = (size_t)B * C * H * W;
    if (total == 0) return hipSuccess;
    const dim3 grid((unsigned)((total + 255) / 256));
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

hipError_t launch_dequant_grad_rowsum(const float* g, const float* sa, const float* sw, float* gc, float* t, int M, int N, int L,
                                      hipStream_t stream) {
    hipLaunchKernelGGL(dequant_grad_rowsum_kernel, dim3((M + 127) / 128), dim3(256), 0, stream, g, sa, sw, gc, t, M, N, L);
    return hipGetLastError();
}

}  // namespace amr
