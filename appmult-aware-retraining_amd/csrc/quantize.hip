// Quantiser of the layer in front of the LUT GEMM, gfx950: real values -> integer codes in one pass.
//
// Forward: codes = clamp(round(x / scale - zp_neg), 0, qmax), the value of the reference's quantize_v2 with
// its straight-through rounding (micronet+/app_layers.py:147-160: "x / s - zpn", Round.apply, clamp); scale and
// zp_neg are read from device memory (they come out of the observers without a host round trip).
// Backward of that expression: the rounding passes the gradient through, the clamp passes it where the
// rounded value lies inside [0, qmax], and x / scale contributes 1 / scale:  gx = inside ? g / scale : 0.
// Both kernels are a single streaming pass (16 bytes per lane and access); the tail is done element-wise.
#include "amr_common.h"

namespace amr {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float quant_code(float x, float s, float zp, float qmax, bool* inside) {
    const float q = x / s - zp;
    // round half to even, as torch.round; the reference's straight-through form q - q.detach() + round(q) turns an
    // infinite q into a NaN (inf - inf), so does this
    const float r = __builtin_isinf(q) ? __builtin_nanf("") : rintf(q);
    *inside = (r >= 0.f) && (r <= qmax);
    // (a NaN stays a NaN, as in torch.clamp; fminf / fmaxf alone would turn it into a code)
    return r != r ? r : fminf(fmaxf(r, 0.f), qmax);
}

__global__ __launch_bounds__(256) void quantize_codes_kernel(const float* __restrict__ x, const float* __restrict__ scale,
                                                             const float* __restrict__ zp_neg, float qmax,
                                                             float* __restrict__ codes, size_t n, int vec) {
    const float s = *scale, zp = *zp_neg;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    bool in;
    if (vec) {
        if (4 * i + 3 < n) {
            const f32x4 v = reinterpret_cast<const f32x4*>(x)[i];
            f32x4 o = {quant_code(v.x, s, zp, qmax, &in), quant_code(v.y, s, zp, qmax, &in), quant_code(v.z, s, zp, qmax, &in),
                       quant_code(v.w, s, zp, qmax, &in)};
            reinterpret_cast<f32x4*>(codes)[i] = o;
        } else {
            for (size_t j = 4 * i; j < n; ++j) codes[j] = quant_code(x[j], s, zp, qmax, &in);
        }
    } else if (i < n) {
        codes[i] = quant_code(x[i], s, zp, qmax, &in);
    }
}

__global__ __launch_bounds__(256) void quantize_codes_backward_kernel(const float* __restrict__ g, const float* __restrict__ x,
                                                                      const float* __restrict__ scale,
                                                                      const float* __restrict__ zp_neg, float qmax,
                                                                      float* __restrict__ gx, size_t n, int vec) {
    const float s = *scale, zp = *zp_neg;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    auto one = [&](float gv, float xv) {
        bool in;
        (void)quant_code(xv, s, zp, qmax, &in);
        return in ? gv / s : 0.f;
    };
    if (vec) {
        if (4 * i + 3 < n) {
            const f32x4 gv = reinterpret_cast<const f32x4*>(g)[i];
            const f32x4 xv = reinterpret_cast<const f32x4*>(x)[i];
            f32x4 o = {one(gv.x, xv.x), one(gv.y, xv.y), one(gv.z, xv.z), one(gv.w, xv.w)};
            reinterpret_cast<f32x4*>(gx)[i] = o;
        } else {
            for (size_t j = 4 * i; j < n; ++j) gx[j] = one(g[j], x[j]);
        }
    } else if (i < n) {
        gx[i] = one(g[i], x[i]);
    }
}

// Observer step + quantisation parameters in one launch (one thread): the scalar updates the reference spreads over a
// dozen tensor operations per layer and step (micronet+/app_layers.py:21-53 observers, :154-160 scale / zero point).
//   mode 0: first batch, min/max := current;  mode 1: running extremes;  mode 2: keep * old + momentum * current
//   (keep = 1 - momentum, rounded by the caller the way the tensor expression rounds it)
//   scale = max((max - min) / qmax, eps)  [or (max - min) * inv_qmax when inv_qmax != 0];  zp_neg = round(min / scale)
// Same operations in the same order as the tensor expressions, each rounded on its own.
__global__ void observer_update_kernel(const float* __restrict__ cur_min, const float* __restrict__ cur_max, float* __restrict__ min_val,
                                       float* __restrict__ max_val, float* __restrict__ scale, float* __restrict__ zp_neg, int mode,
                                       float keep, float momentum, float qmax, float inv_qmax, float eps) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    float lo = *cur_min, hi = *cur_max;
    if (mode == 1) {
        // torch.min / torch.max hand a NaN on; fminf / fmaxf would drop it
        const float old_lo = *min_val, old_hi = *max_val;
        lo = (lo != lo || old_lo != old_lo) ? __builtin_nanf("") : fminf(lo, old_lo);
        hi = (hi != hi || old_hi != old_hi) ? __builtin_nanf("") : fmaxf(hi, old_hi);
    } else if (mode == 2) {
        lo = __fadd_rn(__fmul_rn(keep, *min_val), __fmul_rn(momentum, lo));
        hi = __fadd_rn(__fmul_rn(keep, *max_val), __fmul_rn(momentum, hi));
    }
    *min_val = lo;
    *max_val = hi;
    // (a division by a host-side scalar is a multiplication by its rounded reciprocal in the tensor library: inv_qmax != 0)
    const float range = __fsub_rn(hi, lo);
    const float raw = inv_qmax != 0.f ? __fmul_rn(range, inv_qmax) : __fdiv_rn(range, qmax);
    const float s = raw != raw ? raw : fmaxf(raw, eps);
    *scale = s;
    *zp_neg = rintf(__fdiv_rn(lo, s));
}

hipError_t launch_observer_update(const float* cur_min, const float* cur_max, float* min_val, float* max_val, float* scale,
                                  float* zp_neg, int mode, float keep, float momentum, float qmax, float inv_qmax, float eps,
                                  hipStream_t stream) {
    hipLaunchKernelGGL(observer_update_kernel, dim3(1), dim3(64), 0, stream, cur_min, cur_max, min_val, max_val, scale, zp_neg, mode,
                       keep, momentum, qmax, inv_qmax, eps);
    return hipGetLastError();
}

hipError_t launch_quantize_codes(const float* x, const float* scale, const float* zp_neg, float qmax, float* codes, size_t n,
                                 hipStream_t stream) {
    const int vec = ((((uintptr_t)x) | ((uintptr_t)codes)) & 15) == 0;
    const size_t items = vec ? (n + 3) / 4 : n;
    hipLaunchKernelGGL(quantize_codes_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, x, scale, zp_neg, qmax,
                       codes, n, vec);
    return hipGetLastError();
}

hipError_t launch_quantize_codes_backward(const float* g, const float* x, const float* scale, const float* zp_neg, float qmax,
                                          float* gx, size_t n, hipStream_t stream) {
    const int vec = ((((uintptr_t)x) | ((uintptr_t)g) | ((uintptr_t)gx)) & 15) == 0;
    const size_t items = vec ? (n + 3) / 4 : n;
    hipLaunchKernelGGL(quantize_codes_backward_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, g, x, scale,
                       zp_neg, qmax, gx, n, vec);
    return hipGetLastError();
}

}  // namespace amr
