// Internal helpers shared by the gfx950 LUT-GEMM translation units (not part of the public C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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

}  // namespace amr
