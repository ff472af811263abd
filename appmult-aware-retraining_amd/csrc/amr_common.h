// Internal helpers shared by the gfx950 LUT-GEMM translation units (not part of the public C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <atomic>

namespace amr {

constexpr int kWave = 64;  // CDNA4 wavefront width

// Padded-table geometry for a bit-width: rows = 2^b + 1, cols = 2^b + 2, entry (a,b) at a*cols + b
// (reference layout: self_ops/src/approx_mult.h:12-40).
struct LutGeom {
    int bits;
    int rows;
    int cols;
    int64_t elems;   // rows*cols + tail padding
    int pad_code;    // 2^bits: indexes the all-zero pad row / column
};

inline bool lut_geom_from_bits(int bits, LutGeom* g) {
    int tail;
    switch (bits) {
        case 4: tail = 718; break;
        case 6: tail = 830; break;
        case 7: tail = 638; break;
        case 8: tail = 0; break;
        default: return false;
    }
    const int n = 1 << bits;
    g->bits = bits;
    g->rows = n + 1;
    g->cols = n + 2;
    g->elems = (int64_t)g->rows * g->cols + tail;
    g->pad_code = n;
    return true;
}

inline bool lut_geom_from_elems(int64_t elems, LutGeom* g) {
    for (int bits : {4, 6, 7, 8}) {
        if (lut_geom_from_bits(bits, g) && g->elems == elems) return true;
    }
    return false;
}

// Lets a kernel use up to 160 KB of dynamic LDS: set once per kernel and device (bit d of `done` = device d), from
// whichever host thread gets there first; setting it twice is harmless, so concurrent first calls need no lock.
inline hipError_t allow_full_lds(const void* kernel, std::atomic<uint64_t>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

// Operands of the dequantising store (the zero-point terms, scaling and bias of the reference's ApproxConv2d.forward,
// micronet+/app_layers.py:175-183, see dequant.hip): out == nullptr selects the plain store.
struct SlabDequant {
    const float* xs;      // [M] box sums of the input codes
    const float* wr;      // [N][L] response of the weight codes to an all-ones image
    const float* tp;      // [L] taps inside the image x input channels
    const float* za;      // device scalars
    const float* zw;
    const float* sa;
    const float* sw;
    const float* bias;    // [N] or nullptr
    float* out;           // [M / L][N][L]
    int L;                // positions per image
};

// Convolution-shaped forward pass (3x3, stride 1, padding 1): the rows of the GEMM are the pixels of pixel-major codes
// [B*H*W][C]; column k = tap*C + c of row m is the code of channel c of the pixel tap (ti, tj) reaches from pixel m, or the
// code 0 of the padding (zero: 16 zero bytes, 16-byte aligned).
struct SlabConv {
    const uint8_t* zero;
    int C, H, W;
};

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Four consecutive bytes starting at an arbitrary byte address (global memory accepts unaligned
// dword loads on gfx9-family hardware; memcpy keeps the compiler from assuming 4-byte alignment).
__device__ __forceinline__ uint32_t load_u32_unaligned(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}

// Four codes row[k..k+3]; positions at or beyond `end` repeat the last valid code row[end-1]
// (callers never consume them; the clamp only keeps the load inside the row).
__device__ __forceinline__ uint32_t load_codes4_clamped(const uint8_t* row, int k, int end) {
    if (k + 4 <= end) return load_u32_unaligned(row + k);
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int kk = k + i;
        kk = kk < end ? kk : end - 1;
        v |= (uint32_t)row[kk] << (8 * i);
    }
    return v;
}

// Copies n_dwords dwords of a table from global memory into LDS with all THREADS threads of the workgroup.  A thread
// has eight loads in flight before it stores the first (a plain copy loop compiles to load / wait / store, i.e. one
// memory latency per element and thread: 10 us for a 34 KB table and 256 threads); 16 bytes per load when the table is
// 16-byte aligned.  `lds` must be 16-byte aligned.  The caller synchronises the workgroup afterwards.
template <int THREADS>
__device__ __forceinline__ void stage_table_dwords(void* lds, const void* __restrict__ table, int n_dwords) {
    constexpr int U = 8;
    const int tid = threadIdx.x;
    int done = 0;
    const int n4 = n_dwords >> 2;
    if ((reinterpret_cast<uintptr_t>(table) & 15) == 0 && n4 > 0) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4* s4 = reinterpret_cast<const u32x4*>(table);
        u32x4* d4 = reinterpret_cast<u32x4*>(lds);
        for (int base = 0; base < n4; base += U * THREADS) {
            u32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = s4[min(base + u * THREADS + tid, n4 - 1)];
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (base + u * THREADS + tid < n4) d4[base + u * THREADS + tid] = v[u];
        }
        done = n4 << 2;
    }
    const uint32_t* s32 = reinterpret_cast<const uint32_t*>(table);
    uint32_t* d32 = reinterpret_cast<uint32_t*>(lds);
    for (int base = done; base < n_dwords; base += U * THREADS) {
        uint32_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = s32[min(base + u * THREADS + tid, n_dwords - 1)];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (base + u * THREADS + tid < n_dwords) d32[base + u * THREADS + tid] = v[u];
    }
}

// j / d for 0 <= j < 2^23 and a divisor d whose reciprocal inv = 1.0f / d the caller computed once.
__device__ __forceinline__ int div_small(int j, int d, float inv) {
    int q = (int)((float)j * inv);
    if (q * d > j) --q;
    else if ((q + 1) * d <= j) ++q;
    return q;
}

// Tile coordinates of a workgroup whose (x, y) tile grid is folded into blockIdx.x, x fastest -- the order in which a
// two-dimensional grid is dealt out, without its limit of 65535 workgroups along y.
__device__ __forceinline__ void folded_tile_xy(int tiles_x, int* x, int* y) {
    const uint32_t id = blockIdx.x;
    const uint32_t q = id / (uint32_t)tiles_x;
    *y = (int)q;
    *x = (int)(id - q * (uint32_t)tiles_x);
}

}  // namespace amr
