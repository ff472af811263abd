// Backward LUT-GEMM, gradient of A, for large M on gfx950: "expanded-table" kernel (7-bit tables and
// narrower).
//
// Same result (to fp32 summation order) as lutgemm_gradA_kernel and as the reference's
// ApproxGemmBackwardKernelForGA (self_ops/src/approx_gemm_backward.cu:44-267):
//       gA[m,k] = 1/16 * sum_n gC[m,n] * G[A[m,k]][B[k,n]]
//
//   step 1  expand_gradA_kernel:  S[k][a][n] = half(G[a][B[k,n]] - 1024) for every code a
//   step 2  lutgemm_gradA_slab_kernel:  gA[m,k] = dot(gC[m,:], S[k][A[m,k]][:]) + 1024 * sum_n gC[m,n]
//
// In step 2 a lane owns one row m: it keeps 32 values of gC[m,:] in registers and, for every k of its
// workgroup, reads ROW a = A[m,k] of S[k] (64 B, four 128-bit LDS reads) instead of gathering 32 single
// entries, so the LDS moves eight entries per lane and instruction.  The multiply-add takes the half
// straight into an fp32 fma (v_fma_mix_f32); a half holds every integer of magnitude <= 2048, so table
// entries in [-1024, 3072] are exact (16 x the gradient of a 7-bit multiplier is about 16*b <= 2032) and
// products and sums are the fp32 values an fp32 table would give.  An entry a half cannot hold, or a masked
// code 128 in A (not addressable here), raises flags[2] and the direct kernel, queued behind and gated on
// that flag, recomputes gA.
//
// Layout of S in HBM: S[n_tile][k][a (128 rows)][40 halves]: 32 columns + 16 B of padding, so that the rows
// of the 16 codes a mod 16 start in 16 different groups of four banks (lanes read the same columns of
// different rows at the same time; with 64 B rows they would all meet in the same few banks).
// A workgroup (8 waves = 512 rows; two per CU, so that one computes while the other waits) owns 16 or 32 consecutive k and walks all column tiles; the slabs of four k
// (40 KB) are double buffered in LDS and filled by LDS-direct loads while the previous four are consumed.
#include <type_traits>

#include "amr_common.h"

namespace amr {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kGaCols = 32;                               // columns per tile
constexpr int kGaRowBytes = 2 * kGaCols + 16;             // 80
constexpr int kGaSlabBytes = 128 * kGaRowBytes;           // one k: 10 KB
constexpr int kGaChunkK = 4;
constexpr int kGaChunkBytes = kGaChunkK * kGaSlabBytes;   // 40 KB
constexpr float kGaHalfOffset = 1024.f;
constexpr int kGaWaves = 8;                               // 512 rows per workgroup; two workgroups share a CU (80 KB of LDS each)

// ------------------------------------------------------------------------------------------ expand
// grid (n_tiles, K / 8), 256 threads.  Requires N % 32 == 0 and K % 8 == 0.
constexpr int kGaExpandK = 8;

__global__ __launch_bounds__(256) void expand_gradA_kernel(const uint8_t* __restrict__ B, const uint32_t* __restrict__ lut32,
                                                           int lut_dwords, int lut_cols, int n_codes,
                                                           uint32_t* __restrict__ S, uint32_t* __restrict__ flags, int K, int N) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* s32 = reinterpret_cast<uint32_t*>(smem);
    for (int i = threadIdx.x; i < lut_dwords; i += 256) s32[i] = lut32[i];
    __syncthreads();
    const int16_t* s16 = reinterpret_cast<const int16_t*>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // 16 lanes write the 64 B of one row: lane = (k within a group of four, column pair), one dword (two columns) per lane
    const int ks = lane >> 4, cp = lane & 15;
    const int n = blockIdx.x * kGaCols + 2 * cp;
    bool inexact = false;
    for (int pp = 0; pp < kGaExpandK / 4; ++pp) {
        const int k = blockIdx.y * kGaExpandK + 4 * pp + ks;
        const int b0 = (int)B[(size_t)k * N + n], b1 = (int)B[(size_t)k * N + n + 1];
        uint32_t* slab = S + ((size_t)blockIdx.x * K + k) * (kGaSlabBytes / 4);
        for (int a = wave; a < 128; a += 4) {
            // codes beyond the table (only the pad code 2^b of a narrower table can occur) contribute zero
            const float v0 = (a < n_codes) ? (float)s16[a * lut_cols + b0] : 0.f;
            const float v1 = (a < n_codes) ? (float)s16[a * lut_cols + b1] : 0.f;
            const _Float16 h0 = (_Float16)(v0 - kGaHalfOffset), h1 = (_Float16)(v1 - kGaHalfOffset);
            inexact |= ((float)h0 != v0 - kGaHalfOffset) | ((float)h1 != v1 - kGaHalfOffset);
            const uint32_t w = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
            slab[a * (kGaRowBytes / 4) + cp] = w;
        }
    }
    if (__builtin_amdgcn_ballot_w64(inexact) != 0 && lane == 0) atomicOr(&flags[2], 1u);
}

// Four 128-bit LDS reads at consecutive 16 B offsets, issued and NOT waited for.  Inline assembly: the
// compiler must not make these reads wait for the LDS-direct loads that fill the other buffer (same LDS
// array to it), the waves of the two workgroups of a CU overlap each other's waits.
__device__ __forceinline__ void ga_issue4(u32x4 (&d)[4], uint32_t addr) {
    asm volatile(
        "ds_read_b128 %0, %4\n ds_read_b128 %1, %4 offset:16\n ds_read_b128 %2, %4 offset:32\n ds_read_b128 %3, %4 offset:48"
        : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3])
        : "v"(addr)
        : "memory");
}

// Waits until at most PENDING LDS operations are outstanding; the four results pass through as in/out
// operands so that every use of them is ordered after the wait.
template <int PENDING>
__device__ __forceinline__ void ga_wait4(u32x4 (&d)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]) : "n"(PENDING) : "memory");
}

// ------------------------------------------------------------------------------------------ consume
// grid ceil(M / 512) * K / KT workgroups, 512 threads, KT = 16 or 32 k per workgroup.  Requires M >= 64, N % 32 == 0,
// K % KT == 0, M*K < 2^31.
// rows_per_image = 0: gA row-major [M,K]; L > 0: image-major transposed gA[m / L][k][m % L].
template <bool VEC, int kGaKT>
__global__ __launch_bounds__(kGaWaves * 64, 2) void lutgemm_gradA_slab_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const u32x4* __restrict__ S, float* __restrict__ gA,
    uint32_t* __restrict__ flags, int M, int K, int N, float scale, int rows_per_image, int row_blocks, int xcd_order) {
    __shared__ __align__(16) unsigned char smem[2 * kGaChunkBytes];
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    // A wave whose rows would stick out of M is shifted up so that all its rows exist; the rows it then
    // shares with the wave above are not stored twice (a wave entirely beyond M stores nothing but still
    // takes part in the copies and barriers).
    // Workgroup order: 32 neighbouring row blocks, then all k groups, then the next 32 row blocks, so that the workgroups
    // in flight at one time share their slabs (same k group) and their rows of gC (same row block) in the caches.
    // The hardware deals workgroups to the 8 XCDs round-robin by index; the workgroups of one XCD (same index mod 8)
    // take consecutive positions of that order when there are few row blocks (xcd_order), so that the row blocks of
    // one k group meet in ONE L2 and its slabs are fetched from memory once: with 8 row blocks every workgroup
    // fetched its own copy otherwise.  With many row blocks each XCD already holds several per k group, and keeping
    // a k group on one XCD measured a little slower.
    const int k_groups = K / kGaKT;
    const int total_wgs = row_blocks * k_groups;
    const int per_xcd = (total_wgs + 7) / 8;
    const int logical = xcd_order ? (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8) : (int)blockIdx.x;
    if (logical >= total_wgs) return;
    const int band = logical / (32 * k_groups);                    // 32 row blocks x all k groups
    const int band_rows = min(32, row_blocks - 32 * band);
    const int in_band = logical - band * 32 * k_groups;
    const int k_group = in_band / band_rows;
    const int row_block = 32 * band + (in_band - k_group * band_rows);
    const int m_first = (row_block * kGaWaves + wave) * 64;
    const int m = min(m_first, M - 64) + lane;
    const int k0 = k_group * kGaKT;
    const int n_tiles = N / kGaCols;
    const int total = n_tiles * (kGaKT / kGaChunkK);           // chunks this workgroup walks: (tile, four k)

    uint32_t codes[kGaKT / 4];
#pragma unroll
    for (int d = 0; d < kGaKT / 4; ++d) codes[d] = load_u32_unaligned(A + (size_t)m * K + k0 + 4 * d);
    uint32_t any_code = 0;
#pragma unroll
    for (int d = 0; d < kGaKT / 4; ++d) any_code |= codes[d];
    if (__builtin_amdgcn_ballot_w64((any_code & 0x80808080u) != 0) != 0) {
        if (lane == 0) atomicOr(&flags[2], 1u);
    }

    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // chunk q = (tile, four k of the workgroup's range): 40 KB = 40 wave-wide 16-byte loads, spread over the waves
    auto request = [&](int q, int buf) {
        const int nt = q / (kGaKT / kGaChunkK), kc = q % (kGaKT / kGaChunkK);
        const u32x4* src = S + ((size_t)nt * K + k0 + kGaChunkK * kc) * (kGaSlabBytes / 16);
        for (int i = wave; i < kGaChunkBytes / 1024; i += kGaWaves)
            __builtin_amdgcn_global_load_lds((gptr_t)(src + i * 64 + lane), (lptr_t)(smem + buf * kGaChunkBytes + i * 1024), 16, 0, 0);
    };

    float acc[kGaKT];
#pragma unroll
    for (int kk = 0; kk < kGaKT; ++kk) acc[kk] = 0.f;
    float row_sum = 0.f;

    request(0, 0);
    const float* grow = gC + (size_t)m * N;
    for (int nt = 0; nt < n_tiles; ++nt) {
        float g[kGaCols];
#pragma unroll
        for (int kc = 0; kc < kGaKT / kGaChunkK; ++kc) {
            const int q = nt * (kGaKT / kGaChunkK) + kc;
            // chunk q, requested one step ago, has landed for every wave; the other buffer is free again
            asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
            if (kc == 0) {
#pragma unroll
                for (int i = 0; i < kGaCols / 4; ++i) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(grow + nt * kGaCols + 4 * i);
                    g[4 * i] = v.x; g[4 * i + 1] = v.y; g[4 * i + 2] = v.z; g[4 * i + 3] = v.w;
                }
#pragma unroll
                for (int i = 0; i < kGaCols; ++i) row_sum += g[i];
                // the values of gC have arrived here; only now is the next chunk requested, so that the wait the
                // compiler places in front of the first use of gC does not also wait for that request
                asm volatile("" : "+v"(row_sum));
            }
            if (q + 1 < total) request(q + 1, (kc + 1) & 1);
            auto slab_addr = [&](int kk) {
                const uint32_t a = (codes[kc] >> (8 * kk)) & 0xffu;
                return a * (uint32_t)kGaRowBytes + (uint32_t)((kc & 1) * kGaChunkBytes + kk * kGaSlabBytes);
            };
#pragma unroll
            for (int kk = 0; kk < kGaChunkK; ++kk) {
                u32x4 d[4];
                ga_issue4(d, slab_addr(kk));
                ga_wait4<0>(d);
                float s = acc[kGaChunkK * kc + kk];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f16x8 h = __builtin_bit_cast(f16x8, d[i]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) s = __builtin_fmaf(g[8 * i + e], (float)h[e], s);
                }
                // pin: the sum is finished before the next volatile read block starts (otherwise the compiler keeps
                // the results of several blocks live and runs out of registers)
                asm volatile("" : "+v"(s));
                acc[kGaChunkK * kc + kk] = s;
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (m < m_first) return;     // row stored by the wave above
    const float corr = kGaHalfOffset * row_sum;
    if (rows_per_image > 0) {
        const int img = m / rows_per_image, l = m - img * rows_per_image;
        float* o = gA + ((size_t)img * K + k0) * rows_per_image + l;
#pragma unroll
        for (int kk = 0; kk < kGaKT; ++kk) o[(size_t)kk * rows_per_image] = (acc[kk] + corr) * scale;
    } else if (VEC) {
#pragma unroll
        for (int d = 0; d < kGaKT / 4; ++d) {
            f32x4 v = {(acc[4 * d] + corr) * scale, (acc[4 * d + 1] + corr) * scale, (acc[4 * d + 2] + corr) * scale,
                       (acc[4 * d + 3] + corr) * scale};
            *reinterpret_cast<f32x4*>(gA + (size_t)m * K + k0 + 4 * d) = v;
        }
    } else {
#pragma unroll
        for (int kk = 0; kk < kGaKT; ++kk) gA[(size_t)m * K + k0 + kk] = (acc[kk] + corr) * scale;
    }
}

// ------------------------------------------------------------------------------------------ host
hipError_t launch_gradA(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                        const LutGeom& g, int M, int K, int N, float scale, int n_cu, hipStream_t stream,
                        const uint32_t* gate, int rows_per_image);

// Bytes of the expanded table S, or 0 when the expanded-table gradA does not apply.
size_t gradA_slab_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    // (below about 4096 rows, or 8192 for short K, the expansion, 2^b / M of the work but all of it HBM writes plus two
    // more launches, costs more than it saves)
    if (!force && M < 8192 && K < 1024) return 0;
    if (g.bits > 7 || M < (force ? 2048 : 4096) || (N % kGaCols) != 0 || (K % 8) != 0 || ((K % 16) != 0 && (K % 24) != 0) || (size_t)M * K >= (1ull << 31)) return 0;
    return (size_t)(N / kGaCols) * K * kGaSlabBytes;
}

hipError_t launch_gradA_slab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                             const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                             int rows_per_image, hipStream_t stream) {
    const int lut_dwords = g.rows * g.cols / 2;
    hipLaunchKernelGGL(expand_gradA_kernel, dim3(N / kGaCols, K / kGaExpandK), dim3(256), (size_t)lut_dwords * 4, stream, B,
                       reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols, 1 << g.bits, reinterpret_cast<uint32_t*>(S),
                       flags, K, N);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int rows_per_wg = kGaWaves * 64;
    const bool vec = (((uintptr_t)gA & 15) == 0);
    if (((uintptr_t)gC & 15) != 0) return hipErrorInvalidValue;   // callers check: rows of gC are read 16 bytes at a time
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const unsigned row_blocks = (unsigned)((M + rows_per_wg - 1) / rows_per_wg);
    // k per workgroup: 32 halve the gC reloads and the start-up cost per multiply-add against 16 (measured better
    // also where the last round of workgroups is half empty); 24 for few row blocks (measured).
    const int xcd_order = row_blocks <= 16;
    auto launch = [&](auto kt_tag) {
        constexpr int KT = decltype(kt_tag)::value;
        const dim3 grid(8 * ((row_blocks * (K / KT) + 7) / 8));
        if (vec) hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<true, KT>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale, rows_per_image, (int)row_blocks, xcd_order);
        else hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<false, KT>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale, rows_per_image, (int)row_blocks, xcd_order);
    };
    (void)n_cu;
    int kt = (K % 32) == 0 ? 32 : 16;
    if (row_blocks <= 16 && (K % 24) == 0) kt = 24;    // few row blocks: more, shorter workgroups fill the last round better
    if ((K % kt) != 0) kt = (K % 24) == 0 ? 24 : 16;
    if (kt == 32) launch(std::integral_constant<int, 32>{});
    else if (kt == 24) launch(std::integral_constant<int, 24>{});
    else launch(std::integral_constant<int, 16>{});
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // masked codes in A or table entries a half cannot hold: the gated direct kernel recomputes gA
    return launch_gradA(gC, A, B, gA, lut, g, M, K, N, scale, n_cu, stream, flags + 2, rows_per_image);
}

}  // namespace amr
