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
// The scalar part of an observer step: range update (mode 0 first batch, 1 running extremes, 2 moving average), then
// scale = max((max - min) / qmax, eps) [or (max - min) * inv_qmax], zp_neg = round(min / scale); every operation rounded on
// its own, in the order of the tensor expressions (micronet+/app_layers.py:21-53, :154-160).
__device__ __forceinline__ void observer_update_scalars(float lo, float hi, float* __restrict__ min_val, float* __restrict__ max_val,
                                                        float* __restrict__ scale, float* __restrict__ zp_neg, int mode, float keep,
                                                        float momentum, float qmax, float inv_qmax, float eps) {
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

// Extremes of a tensor and the observer step that follows, in ONE launch (the reference: torch.min, torch.max and a dozen
// one-element tensor operations per layer and step).  Every workgroup folds its share (eight 16-byte loads in flight per
// thread, grid-stride) and leaves its three results -- smallest, largest, "saw a NaN" -- in a slot of its own in `state`
// (plain stores), then draws a ticket from state[0], the only atomic; the workgroup that draws the last ticket folds the
// slots, does the scalar update and puts the ticket counter back to 0 for the next call.  torch.aminmax hands a NaN on:
// so does this.  state: 4 + 3 * kObserveMaxBlocks words, all zero before the first call.
constexpr int kObserveMaxBlocks = 1024;

__global__ __launch_bounds__(256) void observe_minmax_kernel(const float* __restrict__ x, size_t n, uint32_t* __restrict__ state,
                                                             float* __restrict__ min_val, float* __restrict__ max_val,
                                                             float* __restrict__ scale, float* __restrict__ zp_neg, int mode, float keep,
                                                             float momentum, float qmax, float inv_qmax, float eps, int vec) {
    __shared__ float s_lo[4], s_hi[4];
    __shared__ uint32_t s_nan[4], s_last;
    float lo = __builtin_inff(), hi = -__builtin_inff();
    bool nan = false;
    const size_t stride = (size_t)gridDim.x * 256, tid = (size_t)blockIdx.x * 256 + threadIdx.x;
    auto take = [&](float v) {
        nan |= v != v;
        lo = fminf(lo, v);          // (fminf / fmaxf drop a NaN: it is carried by `nan`)
        hi = fmaxf(hi, v);
    };
    if (vec) {
        const size_t n4 = n >> 2;
        const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
        size_t i = tid;
        for (; i + 7 * stride < n4; i += 8 * stride) {
            f32x4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = x4[i + u * stride];
#pragma unroll
            for (int u = 0; u < 8; ++u) { take(v[u].x); take(v[u].y); take(v[u].z); take(v[u].w); }
        }
        for (; i < n4; i += stride) {
            const f32x4 v = x4[i];
            take(v.x); take(v.y); take(v.z); take(v.w);
        }
        for (size_t j = (n4 << 2) + tid; j < n; j += stride) take(x[j]);
    } else {
        for (size_t i = tid; i < n; i += stride) take(x[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    const bool wave_nan = __builtin_amdgcn_ballot_w64(nan) != 0;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { s_lo[wave] = lo; s_hi[wave] = hi; s_nan[wave] = wave_nan; }
    __syncthreads();
    uint32_t* slots = state + 4;
    if (threadIdx.x == 0) {
        lo = fminf(fminf(s_lo[0], s_lo[1]), fminf(s_lo[2], s_lo[3]));
        hi = fmaxf(fmaxf(s_hi[0], s_hi[1]), fmaxf(s_hi[2], s_hi[3]));
        // (atomic exchanges instead of plain stores: they are performed in the L2, where the last workgroup reads them)
        atomicExch(&slots[3 * blockIdx.x], __float_as_uint(lo));
        atomicExch(&slots[3 * blockIdx.x + 1], __float_as_uint(hi));
        atomicExch(&slots[3 * blockIdx.x + 2], s_nan[0] | s_nan[1] | s_nan[2] | s_nan[3]);
        __threadfence();
        s_last = atomicAdd(&state[0], 1u) == gridDim.x - 1 ? 1u : 0u;
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    lo = __builtin_inff(), hi = -__builtin_inff();
    uint32_t any_nan = 0;
    for (int b = threadIdx.x; b < (int)gridDim.x; b += 256) {
        lo = fminf(lo, __uint_as_float(atomicOr(&slots[3 * b], 0u)));
        hi = fmaxf(hi, __uint_as_float(atomicOr(&slots[3 * b + 1], 0u)));
        any_nan |= atomicOr(&slots[3 * b + 2], 0u);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        lo = fminf(lo, __shfl_xor(lo, o));
        hi = fmaxf(hi, __shfl_xor(hi, o));
    }
    const bool nan2 = __builtin_amdgcn_ballot_w64(any_nan != 0) != 0;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) { s_lo[wave] = lo; s_hi[wave] = hi; s_nan[wave] = nan2; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float t_lo = fminf(fminf(s_lo[0], s_lo[1]), fminf(s_lo[2], s_lo[3]));
        float t_hi = fmaxf(fmaxf(s_hi[0], s_hi[1]), fmaxf(s_hi[2], s_hi[3]));
        // (mode bit 2: the extremes of max(x, 0) -- the maximum with zero is monotone, so it is taken on the two results)
        if (mode & 4) { t_lo = fmaxf(t_lo, 0.f); t_hi = fmaxf(t_hi, 0.f); }
        if (s_nan[0] | s_nan[1] | s_nan[2] | s_nan[3]) t_lo = t_hi = __builtin_nanf("");
        observer_update_scalars(t_lo, t_hi, min_val, max_val, scale, zp_neg, mode & 3, keep, momentum, qmax, inv_qmax, eps);
        atomicExch(&state[0], 0u);
    }
}

hipError_t launch_observe_minmax(const float* x, size_t n, uint32_t* state, float* min_val, float* max_val, float* scale, float* zp_neg,
                                 int mode, float keep, float momentum, float qmax, float inv_qmax, float eps, int n_cu, hipStream_t stream) {
    const int vec = (((uintptr_t)x) & 15) == 0;
    size_t blocks = (n + 256 * 32 - 1) / (256 * 32);         // at least 32 values per thread
    // one workgroup per CU at most (measured on MI355X for 134 MB: 28 us with 256 workgroups, 37 with 512, 57 with 1024 -- the
    // tickets and the slots cost more than the extra loads in flight gain)
    size_t cap = (size_t)(n_cu > 0 ? n_cu : 256);
    if (cap > kObserveMaxBlocks) cap = kObserveMaxBlocks;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(observe_minmax_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, n, state, min_val, max_val, scale, zp_neg,
                       mode, keep, momentum, qmax, inv_qmax, eps, vec);
    return hipGetLastError();
}

__global__ void observer_update_kernel(const float* __restrict__ cur_min, const float* __restrict__ cur_max, float* __restrict__ min_val,
                                       float* __restrict__ max_val, float* __restrict__ scale, float* __restrict__ zp_neg, int mode,
                                       float keep, float momentum, float qmax, float inv_qmax, float eps) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    observer_update_scalars(*cur_min, *cur_max, min_val, max_val, scale, zp_neg, mode, keep, momentum, qmax, inv_qmax, eps);
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
