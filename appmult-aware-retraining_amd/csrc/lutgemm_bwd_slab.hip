// Backward LUT-GEMM, gradient of B, for large M on gfx950: "expanded-table" kernel (7-bit tables and
// narrower).
//
// Same result (to fp32 summation order) as lutgemm_gradB_kernel and as the reference's
// ApproxGemmBackwardKernelForGB (self_ops/src/approx_gemm_backward.cu:269-492).
//
// A workgroup owns KT values of k and one 64-column tile of B.  It first expands the gradient table
// along its B codes into LDS as fp32,
//       S[kk][a][c] = (float) G[a][ B[k0+kk, n0+c] ]          (a = every operand code, 256 B per row)
// and then streams rows m of A / gC.  For one (m, k) everything a lane needs sits in ROW a = A[m,k]
// of S, next to each other, so it is fetched with 128-bit LDS reads instead of one gather per
// multiply-add:
//   lane = (row slot l/16, column group l%16 of 4 columns); acc[kk][c] += gC[m,c] * S[kk][a][c];
//   partial sums of the 4 row slots, 16 waves and M splits are added at the end.
// Every wave-level 128-bit read touches all 64 banks exactly four times, i.e. it is conflict-free.
// The LDS address (slab<<16 | a<<8 | lane part) is assembled from the code byte by one v_perm_b32,
// which needs a < 128: a masked code (128 in a 7-bit operand) raises flags[1] and the direct kernel,
// queued behind this one and gated on that flag, recomputes the result.
// (The gradient of A has no such formulation that pays off: its reduction runs over n, so the rows of
// gC would have to be re-read once per k tile; it stays with the direct gather kernel.)
#include <type_traits>

#include "amr_common.h"

namespace amr {

constexpr int kBwdSlabRows = 128;
constexpr int kBwdSlabBytes = kBwdSlabRows * 256;   // one k: 128 codes x 64 columns x fp32 = 32 KB
constexpr int kBwdKT = 4;                            // k per workgroup (128 KB of LDS)
constexpr int kBwdRU = 2;                            // row groups (of 4 rows) per wave and iteration in gradB
constexpr int kBwdRowsPerIter = 16 * kBwdRU * 4;      // rows a workgroup consumes per iteration

typedef float f32x4 __attribute__((ext_vector_type(4)));

// S[kk][a][c] for kk < KT, built by all 1024 threads straight from the table in global memory (it is
// 33 KB and stays in the L2; the expansion is 2^b / M of the streaming work).
// (T: int16 entries of the reference's tables, or float32 entries)
template <typename T>
__device__ __forceinline__ void build_bwd_slab(float* slab, const T* __restrict__ G, int lut_cols, int n_codes,
                                               const uint8_t* __restrict__ B, int K, int N, int k0, int n0, int kt) {
    const int col = threadIdx.x & 63;
    const int a0 = threadIdx.x >> 6;
    // all loads of one k are issued before the first is used (the table sits in L2; a dependent
    // load-convert-store chain would pay that latency once per entry)
    for (int kk = 0; kk < kt; ++kk) {
        const bool live = (k0 + kk < K) && (n0 + col < N);
        const int b = live ? (int)B[(size_t)(k0 + kk) * N + n0 + col] : 0;
        float* s = slab + kk * (kBwdSlabBytes / 4);
        T e[kBwdSlabRows / 16];
#pragma unroll
        for (int i = 0; i < kBwdSlabRows / 16; ++i) e[i] = G[min(a0 + 16 * i, n_codes - 1) * lut_cols + b];
#pragma unroll
        for (int i = 0; i < kBwdSlabRows / 16; ++i) {
            const int a = a0 + 16 * i;
            s[a * 64 + col] = (live && a < n_codes) ? (float)e[i] : 0.f;
        }
    }
}

// ------------------------------------------------------------------------------------------ gradB
// grid (n_tiles, ceil(K/KT), m_splits), 1024 threads.  out: gB itself (m_splits == 1) or the partial
// buffer [split][K][N].
// FAST: K % 4 == 0, N % 64 == 0, M % 128 == 0, gC 16-byte aligned and M*K, 4*M*N < 2^31, so every
// operand load is an unconditional dword / 128-bit load at a 32-bit offset (no tail handling in the
// streaming loop).
template <bool FAST, typename T>
__global__ __launch_bounds__(1024) void lutgemm_gradB_slab_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ out,
    const T* __restrict__ G, int lut_cols, int n_codes, uint32_t* __restrict__ flags, int M, int K, int N,
    int m_chunk, float scale, int vec_ok) {
    __shared__ __align__(16) unsigned char smem[kBwdKT * kBwdSlabBytes];
    float* slab = reinterpret_cast<float*>(smem);
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 4, cg = lane & 15;
    const int n0 = blockIdx.x * 64;
    const int k0 = blockIdx.y * kBwdKT;
    const int mb = blockIdx.z * m_chunk;
    const int me = min(M, mb + m_chunk);

    build_bwd_slab(slab, G, lut_cols, n_codes, B, K, N, k0, n0, kBwdKT);
    __syncthreads();

    // address pieces: byte0 = 16*cg, byte1 = code (v_perm), byte2 = slab pair (kk>>1), +32768 for odd kk
    const uint32_t base_lo = (uint32_t)(cg << 4), base_hi = base_lo | 0x10000u;
    const bool k_full = (k0 + 4 <= K);
    const bool cols_vec = vec_ok && (n0 + 64 <= N);
    const int ncol = n0 + 4 * cg;

    float acc[kBwdKT][4];
#pragma unroll
    for (int kk = 0; kk < kBwdKT; ++kk)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[kk][c] = 0.f;
    uint32_t seen = 0;

    constexpr int RU = kBwdRU;   // row groups (of 4 rows) per wave and iteration

    // one row group: four 128-bit slab reads (one per k) and 16 multiply-adds
    auto consume = [&](uint32_t a, const f32x4& gvec) {
        seen |= a;
        f32x4 s[kBwdKT];
#pragma unroll
        for (int kk = 0; kk < kBwdKT; ++kk) {
            const uint32_t addr = __builtin_amdgcn_perm(a, (kk & 2) ? base_hi : base_lo, 0x0c020400u + ((uint32_t)kk << 8));
            s[kk] = *reinterpret_cast<const f32x4*>(smem + addr + (kk & 1) * kBwdSlabBytes);
        }
#pragma unroll
        for (int kk = 0; kk < kBwdKT; ++kk) {
            acc[kk][0] = __builtin_fmaf(gvec.x, s[kk].x, acc[kk][0]);
            acc[kk][1] = __builtin_fmaf(gvec.y, s[kk].y, acc[kk][1]);
            acc[kk][2] = __builtin_fmaf(gvec.z, s[kk].z, acc[kk][2]);
            acc[kk][3] = __builtin_fmaf(gvec.w, s[kk].w, acc[kk][3]);
        }
    };

    if (FAST) {
        // Every row of the chunk exists (M % 128 == 0) and offsets fit 32 bits: the operands of a row
        // group are one unaligned dword of codes and one 16-byte piece of gC at per-lane 32-bit offsets
        // that advance by a wave-uniform stride.  Two register sets alternate (no copies); the loads of
        // the next iteration are in flight while the current one is consumed.
        const int iters = (me - mb) / (16 * RU * 4);
        uint32_t aoff[RU], goff[RU];
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const uint32_t m = (uint32_t)(mb + 4 * (wave * RU + u) + rs);
            aoff[u] = m * (uint32_t)K + (uint32_t)k0;
            goff[u] = (m * (uint32_t)N + (uint32_t)ncol) * 4u;
        }
        const uint32_t astep = (uint32_t)(16 * RU * 4) * (uint32_t)K;
        const uint32_t gstep = (uint32_t)(16 * RU * 4) * (uint32_t)N * 4u;
        const unsigned char* gbytes = reinterpret_cast<const unsigned char*>(gC);
        uint32_t a0[RU], a1[RU];
        f32x4 g0[RU], g1[RU];
        auto load = [&](uint32_t (&a)[RU], f32x4 (&g)[RU]) {
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                a[u] = load_u32_unaligned(A + aoff[u]);
                g[u] = *reinterpret_cast<const f32x4*>(gbytes + goff[u]);
                aoff[u] += astep;
                goff[u] += gstep;
            }
        };
        if (iters > 0) load(a0, g0);
        for (int it = 0; it < iters; it += 2) {
            if (it + 1 < iters) load(a1, g1);
#pragma unroll
            for (int u = 0; u < RU; ++u) consume(a0[u], g0[u]);
            if (it + 1 < iters) {
                if (it + 2 < iters) load(a0, g0);
#pragma unroll
                for (int u = 0; u < RU; ++u) consume(a1[u], g1[u]);
            }
        }
    } else {
        for (int g0 = wave * RU; mb + 4 * g0 < me; g0 += 16 * RU) {
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                const int m = mb + 4 * (g0 + u) + rs;
                const bool valid = m < me;
                const int mc = valid ? m : me - 1;
                const uint8_t* arow = A + (size_t)mc * K;
                const uint32_t a = k_full ? load_u32_unaligned(arow + k0) : load_codes4_clamped(arow, k0, K);
                const float* grow = gC + (size_t)mc * N;
                f32x4 v;
                if (cols_vec) {
                    v = *reinterpret_cast<const f32x4*>(grow + ncol);
                } else {
                    v.x = (ncol + 0 < N) ? grow[ncol + 0] : 0.f;
                    v.y = (ncol + 1 < N) ? grow[ncol + 1] : 0.f;
                    v.z = (ncol + 2 < N) ? grow[ncol + 2] : 0.f;
                    v.w = (ncol + 3 < N) ? grow[ncol + 3] : 0.f;
                }
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                consume(valid ? a : 0u, valid ? v : zero);
            }
        }
    }
    if (__builtin_amdgcn_ballot_w64((seen & 0x80808080u) != 0) != 0) {
        if (lane == 0) atomicOr(&flags[1], 1u);
    }

    // sum the four row slots of the wave, then the 16 waves through LDS (the slabs are no longer needed)
#pragma unroll
    for (int kk = 0; kk < kBwdKT; ++kk)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float v = acc[kk][c];
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            acc[kk][c] = v;
        }
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);   // [wave][kk][64]
    if (rs == 0) {
#pragma unroll
        for (int kk = 0; kk < kBwdKT; ++kk)
#pragma unroll
            for (int c = 0; c < 4; ++c) red[(wave * kBwdKT + kk) * 64 + 4 * cg + c] = acc[kk][c];
    }
    __syncthreads();
    if (tid < kBwdKT * 64) {
        const int kk = tid >> 6, col = tid & 63;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < 16; ++w) v += red[(w * kBwdKT + kk) * 64 + col];
        if (k0 + kk < K && n0 + col < N) out[((size_t)blockIdx.z * K + k0 + kk) * N + n0 + col] = v * scale;
    }
}


// ------------------------------------------------------------------------------------------ gradB, half-precision slab
// Same scheme with the expanded table held as IEEE half, S16[kk][a][c] = half(G[a][b] - offset), so that
// eight k fit the 128 KB (half the gC traffic per multiply-add: every row of gC a workgroup streams is
// used for 8 instead of 4 values of k) and one 64-bit LDS read brings four entries.  Exact: a half holds
// every integer of magnitude <= 2048, i.e. table entries in [-2048, 2048] with offset 0 and in [-1024, 3072] with
// offset 1024, picked from the table's extremes by bwd_header_kernel (16 x the gradient of a 7-bit
// multiplier is about 16*b <= 2032); an entry outside that range raises flags[1] like a masked code does
// and the direct kernel recomputes.  The multiply-add takes the half straight into an fp32 fma
// (v_fma_mix_f32), products and sums are the same fp32 values as with an fp32 table, and the offset is
// undone at the end with the column sums of gC:  sum_m g*(G-offset) + offset * sum_m g (nothing to undo and no
// column sums for offset 0).
//
// LDS layout: byte address = (kk>>1)*32768 + a*256 + (kk&1)*128 + 2*pos(c): the two k of a pair share a 256 B
// row; column c of the tile sits at position pos(c) = 8*((c%32)/4) + 4*(c/32) + c%4 of its 128 B half-row, so that the
// 16 bytes a lane reads (column group cg) hold columns 4cg..4cg+3 and 32+4cg..32+4cg+3 and its two 16-byte loads of
// a row of gC belong to two instructions that each cover 128 contiguous bytes per row.
// Lane = (row slot rs of 4, k half kh, column group cg of 8): per row of A it reads the four k of its half with
// 128-bit reads (one v_perm_b32 per eight multiply-adds).  The LDS serves 16 lanes of such a read together, i.e. the
// two k halves of one row slot: half 1 visits the two k of every pair in the other order than half 0, so that one
// reads a 128 B half-row in banks 0-31 and the other one in banks 32-63.
// Requires K % 8 == 0, N % 64 == 0, row counts that are multiples of the rows per iteration, gC 16-byte
// aligned and 32-bit offsets (the launcher checks).
constexpr int kBwdKT16 = 8;
constexpr int kBwdColsumSplits = 64;      // the most M splits the launcher picks

__global__ __launch_bounds__(1024) void lutgemm_gradB_slab16_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ out,
    const int16_t* __restrict__ G, int lut_cols, int n_codes, uint32_t* __restrict__ flags, int M, int K, int N,
    int m_chunk, float scale, int n_tiles, int k_tiles, int splits, float* __restrict__ colsum) {
    constexpr int KT = kBwdKT16;
    __shared__ __align__(16) unsigned char smem[KT * 16384 + 32768];     // slabs + the table as halves
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 4, kh = (lane >> 3) & 1, cg = lane & 7;
    const uint32_t swap = (uint32_t)kh;
    // Workgroups are dealt to the 8 XCDs round-robin by their index; the workgroups of one XCD (same index mod 8) take
    // consecutive k tiles of one (column tile, M split), so that the rows of gC and A they all stream are shared in
    // that XCD's L2 instead of being fetched once per XCD.
    // A workgroup keeps its CU and takes every (gridDim.x / 8)-th unit of its XCD's share: the copy of the table in LDS is made
    // once per workgroup, not once per unit (a unit of 4096 rows lasts 34 us, 3 of them were that copy and the start-up).
    const int total = n_tiles * k_tiles * splits;
    const int per_xcd = (total + 7) / 8;
    if (flags[6] != 0u) return;                  // the table cannot be held as halves (bwd_header_kernel): the direct kernel does it
    const float offset = (float)(int)flags[4];   // bwd_header_kernel
    {   // The table itself goes to LDS, as halves, 128 x 128 without the padding (32 KB behind the slabs; codes the table
        // does not have read as zero): 16 independent loads per thread, one trip to L2.
        _Float16* tab = reinterpret_cast<_Float16*>(smem + KT * 16384);
        bool inexact = false;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int idx = tid + 1024 * i, a = idx >> 7, b = idx & 127;
            const float v = (a < n_codes && b < n_codes) ? (float)G[a * lut_cols + b] - offset : -offset;
            const _Float16 h = (_Float16)v;
            inexact |= ((float)h != v);
            tab[idx] = h;
        }
        if (__builtin_amdgcn_ballot_w64(inexact) != 0 && lane == 0) atomicOr(&flags[1], 1u);
    }
    // the codes of B of a unit (lanes = its 64 columns, eight k) are loaded while the previous unit is being finished
    auto load_b_codes = [&](int logical_u, int (&bc)[KT]) {
        const int lu = min(logical_u, total - 1);
        const int kt_u = lu % k_tiles, nt_u = (lu / k_tiles) % n_tiles;
#pragma unroll
        for (int kk = 0; kk < KT; ++kk) bc[kk] = (int)B[(size_t)(kt_u * KT + kk) * N + nt_u * 64 + lane];
    };
    int bnext[KT];
    load_b_codes((int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8), bnext);
    for (int slot = (int)(blockIdx.x / 8); slot < per_xcd; slot += (int)(gridDim.x / 8)) {
    const int logical = (int)(blockIdx.x % 8) * per_xcd + slot;
    if (logical >= total) break;
    const int k_tile = logical % k_tiles;
    const int n_tile = (logical / k_tiles) % n_tiles;
    const int split = logical / (k_tiles * n_tiles);
    const int n0 = n_tile * 64;
    const int k0 = k_tile * KT;
    const int mb = split * m_chunk;
    const int me = min(M, mb + m_chunk);

    {   // The slabs are gathered from the copy of the table: wave-uniform code a, lanes = columns.  (Gathering them from
        // the table in global memory took 64 loads per thread in 8 dependent rounds: 5 of the 12 us a workgroup
        // spent outside its streaming loop.)
        const _Float16* tab = reinterpret_cast<const _Float16*>(smem + KT * 16384);
        const int col = lane;
        int bcode[KT];
#pragma unroll
        for (int kk = 0; kk < KT; ++kk) bcode[kk] = bnext[kk];
        __syncthreads();
        const _Float16 zero = (_Float16)(-offset);
#pragma unroll
        for (int kk = 0; kk < KT; ++kk) {
            unsigned char* s = smem + (kk >> 1) * 32768 + (kk & 1) * 128 + 2 * (8 * ((col & 31) >> 2) + 4 * (col >> 5) + (col & 3));
            const bool masked = bcode[kk] > 127;           // the masked code of a 7-bit operand: the table's zero column
            const _Float16* t = tab + min(bcode[kk], 127);
#pragma unroll
            for (int i = 0; i < kBwdSlabRows / 16; ++i) {
                const int a = wave + 16 * i;
                const _Float16 h = t[a * 128];
                *reinterpret_cast<_Float16*>(s + a * 256) = masked ? zero : h;
            }
        }
    }
    __syncthreads();

    // address pieces: byte0 = half-row (pair member) and column group, byte1 = code (v_perm), byte2 = k half
    const uint32_t lo_even = (swap << 7) | (uint32_t)(cg << 4) | (swap << 16);          // reads 0, 2
    const uint32_t lo_odd = ((swap ^ 1u) << 7) | (uint32_t)(cg << 4) | (swap << 16);    // reads 1, 3
    uint32_t sel[4];                                                                     // code byte of read j: j ^ swap
#pragma unroll
    for (int j = 0; j < 4; ++j) sel[j] = 0x0c020400u + ((uint32_t)(j ^ (int)swap) << 8);
    const int ncol = n0 + 4 * cg;

    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    float acc[4][8];       // acc[j]: k = k0 + 4 kh + (j ^ kh); columns 4cg..4cg+3, 32+4cg..32+4cg+3
    float gsum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[j][c] = 0.f;
    uint32_t seen = 0;

    constexpr int RU = kBwdRU;
    auto consume = [&](auto sums_tag, uint32_t a4, const f32x4& g0, const f32x4& g1) __attribute__((always_inline)) {
        seen |= a4;
        f16x8 s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t addr = __builtin_amdgcn_perm(a4, (j & 1) ? lo_odd : lo_even, sel[j]);
            s[j] = *reinterpret_cast<const f16x8*>(smem + addr + (j >> 1) * 32768);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[j][0] = __builtin_fmaf(g0.x, (float)s[j][0], acc[j][0]);
            acc[j][1] = __builtin_fmaf(g0.y, (float)s[j][1], acc[j][1]);
            acc[j][2] = __builtin_fmaf(g0.z, (float)s[j][2], acc[j][2]);
            acc[j][3] = __builtin_fmaf(g0.w, (float)s[j][3], acc[j][3]);
            acc[j][4] = __builtin_fmaf(g1.x, (float)s[j][4], acc[j][4]);
            acc[j][5] = __builtin_fmaf(g1.y, (float)s[j][5], acc[j][5]);
            acc[j][6] = __builtin_fmaf(g1.z, (float)s[j][6], acc[j][6]);
            acc[j][7] = __builtin_fmaf(g1.w, (float)s[j][7], acc[j][7]);
        }
        if (decltype(sums_tag)::value) {
            gsum[0] += g0.x; gsum[1] += g0.y; gsum[2] += g0.z; gsum[3] += g0.w;
            gsum[4] += g1.x; gsum[5] += g1.y; gsum[6] += g1.z; gsum[7] += g1.w;
        }
    };

    auto stream_rows = [&](auto sums_tag) __attribute__((always_inline)) {
        const int iters = (me - mb) / (16 * RU * 4);
        uint32_t aoff[RU], goff[RU];
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const uint32_t m = (uint32_t)(mb + 4 * (wave * RU + u) + rs);
            aoff[u] = m * (uint32_t)K + (uint32_t)(k0 + 4 * kh);
            goff[u] = (m * (uint32_t)N + (uint32_t)ncol) * 4u;
        }
        const uint32_t astep = (uint32_t)(16 * RU * 4) * (uint32_t)K;
        const uint32_t gstep = (uint32_t)(16 * RU * 4) * (uint32_t)N * 4u;
        const unsigned char* gbytes = reinterpret_cast<const unsigned char*>(gC);
        uint32_t ca[RU], cb[RU];
        f32x4 ga0[RU], ga1[RU], gb0[RU], gb1[RU];
        // Every load batch is issued unconditionally (beyond the end: the last rows again, nobody consumes them): behind
        // a branch around the loads the compiler's wait in front of the consumer has to cover the path without new
        // loads too, and on the other path it then waits for the first of the loads it has just issued -- no prefetch
        // at all (measured: the waves spent half their time in s_waitcnt).
        int next = 0;
        auto load = [&](uint32_t (&c4)[RU], f32x4 (&g0)[RU], f32x4 (&g1)[RU]) {
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                c4[u] = load_u32_unaligned(A + aoff[u]);
                g0[u] = *reinterpret_cast<const f32x4*>(gbytes + goff[u]);
                g1[u] = *reinterpret_cast<const f32x4*>(gbytes + goff[u] + 128);
            }
            ++next;
            const uint32_t as = next < iters ? astep : 0u, gs = next < iters ? gstep : 0u;
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                aoff[u] += as;
                goff[u] += gs;
            }
            // (the scheduler would otherwise start on the consumer first, i.e. wait for the previous batch, and issue
            // these loads behind that wait)
            __builtin_amdgcn_sched_barrier(0);
        };
        if (iters > 0) {
            load(ca, ga0, ga1);
            int it = 0;
            for (; it + 2 <= iters; it += 2) {
                load(cb, gb0, gb1);
#pragma unroll
                for (int u = 0; u < RU; ++u) consume(sums_tag, ca[u], ga0[u], ga1[u]);
                load(ca, ga0, ga1);
#pragma unroll
                for (int u = 0; u < RU; ++u) consume(sums_tag, cb[u], gb0[u], gb1[u]);
            }
            if (it < iters) {
#pragma unroll
                for (int u = 0; u < RU; ++u) consume(sums_tag, ca[u], ga0[u], ga1[u]);
            }
        }
    };
    // (two copies of the loop.  The column sums of gC, needed to undo a non-zero offset, are the same for all k tiles
    // of a (column tile, M split): only the workgroup of k tile 0 forms them (4 % more work in its loop) and leaves them
    // in colsum[split][n]; gradB_finish_kernel adds offset * colsum to every k afterwards.)
    const bool do_sums = offset != 0.f && k_tile == 0;
    if (do_sums) stream_rows(std::true_type{}); else stream_rows(std::false_type{});
    if (__builtin_amdgcn_ballot_w64((seen & 0x80808080u) != 0) != 0) {
        if (lane == 0) atomicOr(&flags[1], 1u);
    }
    load_b_codes(logical + (int)(gridDim.x / 8), bnext);       // (beyond the last unit: the last one again, unused)

    // The 4 row slots x 16 waves meet in LDS (the slabs are no longer needed; the copy of the table behind them stays):
    // every lane leaves its 32 sums there with eight 16-byte writes, red[wave][rs][k][64 columns] (128 KB), and the sums
    // over (wave, rs) are formed in a fixed order: two partial sums of 32 terms per output by all 1024 threads, then their
    // sum.  (Adding the row slots in registers first took 64 cross-lane operations per wave and unit.)  The lanes of k half
    // 1 keep the two halves of a row of 64 the other way round: the 16 lanes the LDS serves together then write 64
    // different banks.
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);
    {
        float* r = red + (size_t)((wave * 4 + rs) * KT) * 64 + 4 * cg;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int kk = 4 * kh + (j ^ kh);
            const f32x4 lo = {acc[j][0], acc[j][1], acc[j][2], acc[j][3]}, hi = {acc[j][4], acc[j][5], acc[j][6], acc[j][7]};
            *reinterpret_cast<f32x4*>(r + kk * 64 + 32 * kh) = lo;
            *reinterpret_cast<f32x4*>(r + kk * 64 + 32 * (kh ^ 1)) = hi;
        }
    }
    __syncthreads();
    float part = 0.f;
    {
        const int o = tid & 511, p = tid >> 9;          // output (k, column) and half of the (wave, rs) pairs
        const float* r = red + (size_t)(p * 32 * KT) * 64 + (o ^ (((o >> 8) & 1) << 5));      // (o >> 8 = k half of the output)
#pragma unroll 8
        for (int t = 0; t < 32; ++t) part += r[t * KT * 64];
    }
    __syncthreads();
    red[tid] = part;
    if (do_sums) {      // (same for every thread) the column sums of gC: row slots in registers, waves through LDS
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            gsum[c] += __shfl_xor(gsum[c], 32);
            gsum[c] += __shfl_xor(gsum[c], 16);
        }
        if (rs == 0 && kh == 0) {
#pragma unroll
            for (int c = 0; c < 8; ++c) red[1024 + wave * 64 + 32 * (c >> 2) + 4 * cg + (c & 3)] = gsum[c];
        }
    }
    __syncthreads();
    if (tid < KT * 64) {
        const int kk = tid >> 6, col = tid & 63;
        out[((size_t)split * K + k0 + kk) * N + n0 + col] = (red[tid] + red[512 + tid]) * scale;
        if (do_sums && kk == 0) {
            float gs = 0.f;
#pragma unroll
            for (int w = 0; w < 16; ++w) gs += red[1024 + w * 64 + col];
            colsum[(size_t)split * N + n0 + col] = gs;
        }
    }
    __syncthreads();     // the sums have been read: the slabs of the next unit may be written
    }
}

// gB[k][n] = sum over the M splits of the partial results (fixed order) + scale * offset * sum over the splits of the
// column sums of gC (offset = flags[4]; nothing to add for offset 0).  partial == nullptr: one split, the kernel wrote gB itself.
__global__ __launch_bounds__(256) void gradB_finish_kernel(const float* __restrict__ partial, float* __restrict__ gB,
                                                           const float* __restrict__ colsum, const uint32_t* __restrict__ flags,
                                                           int K, int N, int splits, float scale) {
    const float offset = (float)(int)flags[4];
    if (flags[6] != 0u || (partial == nullptr && offset == 0.f)) return;
    const size_t count = (size_t)K * N;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const int n = (int)(i % (size_t)N);
    float v = partial ? partial[i] : gB[i];
    if (partial) {
        // (eight loads in flight, added in the order of the splits: a load-add chain pays the memory latency once per split)
        int p = 1;
        for (; p + 8 <= splits; p += 8) {
            float t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = partial[(size_t)(p + u) * count + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) v += t[u];
        }
        for (; p < splits; ++p) v += partial[(size_t)p * count + i];
    }
    if (offset != 0.f) {
        float cs = colsum[n];
        int p = 1;
        for (; p + 8 <= splits; p += 8) {
            float t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = colsum[(size_t)(p + u) * N + n];
#pragma unroll
            for (int u = 0; u < 8; ++u) cs += t[u];
        }
        for (; p < splits; ++p) cs += colsum[(size_t)p * N + n];
        v += scale * offset * cs;
    }
    gB[i] = v;
}

// ------------------------------------------------------------------------------------------ scratch header
// One workgroup: clears the 64 flag words of the backward scratch and decides how the half-precision tables are stored.
// A half holds every integer of magnitude <= 2048.  offset (flags[3] for the table of gradA, flags[4] for the table of
// gradB, as int32): 0 when the whole table lies in [-2048, 2048] (the correction term with the sums of gC then drops out
// of the kernels); else the value of smallest magnitude that brings every entry into that range, max - 2048 or
// min + 2048 (rounded up to a power of two when that still fits), when the table spans no more than 4096.  The kernels then compute sum g * (entry - offset) + offset * sum g,
// whose rounding errors grow with |offset| while the true terms have the size of the entries: the offset is only taken
// when |offset| <= 8 x the mean magnitude of the entries.  A table that fails either test is not held as halves at all:
// flags[5] (gradA) / flags[6] (gradB) tell the expanded-table kernels to leave at once, and flags[2] / flags[1] make the
// direct kernels queued behind them compute the result.
__global__ __launch_bounds__(1024) void bwd_header_kernel(const uint32_t* __restrict__ lut_a, const uint32_t* __restrict__ lut_b,
                                                          int lut_dwords, int n_entries, uint32_t* __restrict__ flags) {
    __shared__ int extremes[4];
    __shared__ unsigned int magnitude[2];      // sum of |entry|: at most 65536 x 32768 < 2^32, added as integers (any order, same sum)
    if (threadIdx.x < 4) extremes[threadIdx.x] = 0;
    if (threadIdx.x < 2) magnitude[threadIdx.x] = 0u;
    __syncthreads();
    // all loads of both tables are issued before the first is used (one dependent load at a time would pay the
    // memory latency 66 times: 19 us instead of 5)
    constexpr int PER = 9;                       // 9 x 1024 dwords cover a 7-bit table (8385) in one round; an 8-bit table takes four
    uint32_t w[2][PER];
    for (int base = 0; base < lut_dwords; base += PER * 1024) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t* lut = t ? lut_b : lut_a;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const int idx = base + i * 1024 + (int)threadIdx.x;
                w[t][i] = (lut && idx < lut_dwords) ? lut[idx] : 0u;
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            int lo = 0, hi = 0, mag = 0;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const int v0 = (int)(int16_t)(w[t][i] & 0xffffu), v1 = (int)(int16_t)(w[t][i] >> 16);
                lo = min(lo, min(v0, v1));
                hi = max(hi, max(v0, v1));
                mag += abs(v0) + abs(v1);
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                lo = min(lo, __shfl_xor(lo, o));
                hi = max(hi, __shfl_xor(hi, o));
                mag += __shfl_xor(mag, o);           // at most 64 lanes x 18 entries x 32768: fits 32 bits
            }
            if ((threadIdx.x & 63) == 0) {
                atomicMin(&extremes[2 * t], lo);
                atomicMax(&extremes[2 * t + 1], hi);
                atomicAdd(&magnitude[t], (unsigned int)mag);
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        int off[2], unusable[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int lo = extremes[2 * t], hi = extremes[2 * t + 1];
            off[t] = 0;
            unusable[t] = 0;
            if (lo < -2048 || hi > 2048) {
                if (hi - lo > 4096) unusable[t] = 1;
                else {
                    // the value of smallest magnitude that works, rounded up to a power of two when one fits: g * 2^j is
                    // exact, so a row of zeros (the pad row a masked code reads) still sums to exactly -offset * sum g and
                    // cancels against the correction term
                    const int need = hi > 2048 ? hi - 2048 : -(lo + 2048), room = hi > 2048 ? lo + 2048 : -(hi - 2048);
                    int p = 1;
                    while (p < need) p <<= 1;
                    const int mag_off = p <= room ? p : need;
                    off[t] = hi > 2048 ? mag_off : -mag_off;
                }
                if ((unsigned long long)abs(off[t]) * (unsigned long long)n_entries > 8ull * magnitude[t]) unusable[t] = 1;
            }
            if (unusable[t]) off[t] = 0;
        }
        uint32_t v = 0;
        const int i = threadIdx.x;
        if (i == 3) v = (uint32_t)off[0];
        if (i == 4) v = (uint32_t)off[1];
        if (i == 5 || i == 2) v = lut_a ? (uint32_t)unusable[0] : 0u;
        if (i == 6 || i == 1) v = lut_b ? (uint32_t)unusable[1] : 0u;
        flags[i] = v;
    }
}

hipError_t launch_bwd_header(const int16_t* lut_a, const int16_t* lut_b, const LutGeom& g, uint32_t* flags, hipStream_t stream) {
    hipLaunchKernelGGL(bwd_header_kernel, dim3(1), dim3(1024), 0, stream, reinterpret_cast<const uint32_t*>(lut_a),
                       reinterpret_cast<const uint32_t*>(lut_b), g.rows * g.cols / 2, (1 << g.bits) * (1 << g.bits), flags);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ host
hipError_t launch_gradB_gated(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                              const LutGeom& g, int M, int K, int N, float scale, const uint32_t* gate, hipStream_t stream);
__global__ void reduce_partials_kernel(const float* __restrict__ partial, float* __restrict__ out, size_t count, int splits);

// Floats of scratch the half-slab kernel keeps in front of its partial results (column sums of gC per M split).
size_t gradB_slab_colsum_floats(int N) { return kBwdColsumSplits * (size_t)N; }

bool bwd_slab_applies(const LutGeom& g, int M, int K, int N) {
    (void)N;
    // (measured cross-over against the direct kernel on MI355X: between 512 and 1024 rows)
    return g.bits <= 7 && M >= 1024 && K >= 4;
}

// M splits of the expanded-table gradB.  A workgroup fills a CU (128 KB of LDS), so the grid runs in rounds
// of n_cu workgroups: pick the split count whose (rounds x rows per workgroup) is smallest, charging every
// workgroup the cost of expanding its slabs (about that of streaming 512 rows) and keeping at least 1024
// rows per workgroup.
static int gradB_slab_splits_kt(int M, int K, int N, int n_cu, int kt) {
    const long per_split = (long)((N + 63) / 64) * ((K + kt - 1) / kt);
    long max_s = M / 1024;
    if (max_s > 64) max_s = 64;
    if (max_s < 1) max_s = 1;
    long best_s = 1, best_cost = -1;
    for (long sp = 1; sp <= max_s; ++sp) {
        long chunk = (M + sp - 1) / sp;
        chunk = (chunk + 255) & ~255L;
        const long zs = (M + chunk - 1) / chunk;
        const long rounds = (per_split * zs + n_cu - 1) / n_cu;
        const long cost = rounds * (chunk + 512);
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_s = sp; }
    }
    return (int)best_s;
}

// Upper bound over the kernels launch_gradB_slab may pick (sizes the partial-sum scratch).
int gradB_slab_splits(int M, int K, int N, int n_cu) {
    const int s4 = gradB_slab_splits_kt(M, K, N, n_cu, kBwdKT), s8 = gradB_slab_splits_kt(M, K, N, n_cu, kBwdKT16);
    return s4 > s8 ? s4 : s8;
}

hipError_t launch_gradB_slab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                             const LutGeom& g, int M, int K, int N, float scale, uint32_t* flags, float* partials,
                             int n_cu, hipStream_t stream, int split_cap) {
    const int vec_ok = ((N & 3) == 0) && (((uintptr_t)gC & 15) == 0);
    const bool small = (size_t)M * K < (1ull << 31) && (size_t)M * N * 4 < (1ull << 31);
    const bool regular = vec_ok && small && (N & 63) == 0 && (M % kBwdRowsPerIter) == 0;
    const bool half_slab = regular && (K & 7) == 0;
    const int kt = half_slab ? kBwdKT16 : kBwdKT;
    // split_cap > 0: the most M splits the caller's scratch has room for
    int splits = gradB_slab_splits_kt(M, K, N, n_cu, kt);
    if (split_cap > 0 && splits > split_cap) splits = split_cap;
    int m_chunk = (M + splits - 1) / splits;
    m_chunk = (m_chunk + 255) & ~255;
    const int zs = (M + m_chunk - 1) / m_chunk;
    float* out = zs > 1 ? partials : gB;
    dim3 grid((N + 63) / 64, (K + kt - 1) / kt, zs);
    if (half_slab) {
        // scratch of this kernel: [column sums of gC: 64 splits x N][partial results]
        float* colsum = partials;
        float* part16 = partials + kBwdColsumSplits * (size_t)N;
        out = zs > 1 ? part16 : gB;
        const int total = (int)(grid.x * grid.y * grid.z);
        // (one workgroup per CU at most; the workgroups of an XCD walk their share of the units in steps of that many)
        const int per_xcd16 = (total + 7) / 8, cus_per_xcd16 = n_cu >= 8 ? n_cu / 8 : 1;
        hipLaunchKernelGGL(lutgemm_gradB_slab16_kernel, dim3(8 * (per_xcd16 < cus_per_xcd16 ? per_xcd16 : cus_per_xcd16)), dim3(1024), 0, stream, gC, A, B, out, lut, g.cols,
                           1 << g.bits, flags, M, K, N, m_chunk, scale, (int)grid.x, (int)grid.y, (int)grid.z, colsum);
        hipError_t e16 = hipGetLastError();
        if (e16 != hipSuccess) return e16;
        const size_t count = (size_t)K * N;
        hipLaunchKernelGGL(gradB_finish_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream,
                           zs > 1 ? (const float*)part16 : (const float*)nullptr, gB, colsum, flags, K, N, zs, scale);
        e16 = hipGetLastError();
        if (e16 != hipSuccess) return e16;
        return launch_gradB_gated(gC, A, B, gB, lut, g, M, K, N, scale, flags + 1, stream);
    }
    else if (regular && (K & 3) == 0)
        hipLaunchKernelGGL((lutgemm_gradB_slab_kernel<true, int16_t>), grid, dim3(1024), 0, stream, gC, A, B, out, lut, g.cols, 1 << g.bits,
                           flags, M, K, N, m_chunk, scale, vec_ok);
    else
        hipLaunchKernelGGL((lutgemm_gradB_slab_kernel<false, int16_t>), grid, dim3(1024), 0, stream, gC, A, B, out, lut, g.cols, 1 << g.bits,
                           flags, M, K, N, m_chunk, scale, vec_ok);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (zs > 1) {
        const size_t count = (size_t)K * N;
        hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, partials, gB,
                           count, zs);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    // 7-bit operands can hold the masked code 128, and any table can hold an entry a half cannot: the gated
    // direct kernel covers both (for narrower tables a code 2^b is an ordinary slab row of zeros)
    if (g.bits == 7 || half_slab) return launch_gradB_gated(gC, A, B, gB, lut, g, M, K, N, scale, flags + 1, stream);
    return hipSuccess;
}

// The same for float32 tables: the fp32 slab holds the entries themselves, so the products and sums are the ones the
// direct kernel forms (the half-precision slab cannot hold arbitrary float entries).  flags[1] is cleared here; the
// direct float-table kernel queued behind is gated on it (7-bit operands holding the masked code 128).
hipError_t launch_gradB_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut, const LutGeom& g,
                               int M, int K, int N, float scale, void* workspace, int n_cu, hipStream_t stream,
                               const uint32_t* gate);
hipError_t launch_gradB_slab_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut,
                                    const LutGeom& g, int M, int K, int N, float scale, uint32_t* flags, float* partials,
                                    int n_cu, hipStream_t stream) {
    hipError_t e;
    const int vec_ok = ((N & 3) == 0) && (((uintptr_t)gC & 15) == 0);
    const bool small = (size_t)M * K < (1ull << 31) && (size_t)M * N * 4 < (1ull << 31);
    const bool regular = vec_ok && small && (N & 63) == 0 && (M % kBwdRowsPerIter) == 0;
    const int splits = gradB_slab_splits_kt(M, K, N, n_cu, kBwdKT);
    int m_chunk = (M + splits - 1) / splits;
    m_chunk = (m_chunk + 255) & ~255;
    const int zs = (M + m_chunk - 1) / m_chunk;
    float* out = zs > 1 ? partials : gB;
    dim3 grid((N + 63) / 64, (K + kBwdKT - 1) / kBwdKT, zs);
    if (regular && (K & 3) == 0)
        hipLaunchKernelGGL((lutgemm_gradB_slab_kernel<true, float>), grid, dim3(1024), 0, stream, gC, A, B, out, lut, g.cols, 1 << g.bits,
                           flags, M, K, N, m_chunk, scale, vec_ok);
    else
        hipLaunchKernelGGL((lutgemm_gradB_slab_kernel<false, float>), grid, dim3(1024), 0, stream, gC, A, B, out, lut, g.cols, 1 << g.bits,
                           flags, M, K, N, m_chunk, scale, vec_ok);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (zs > 1) {
        const size_t count = (size_t)K * N;
        hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, partials, gB,
                           count, zs);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (g.bits == 7) return launch_gradB_f32tab(gC, A, B, gB, lut, g, M, K, N, scale, nullptr, n_cu, stream, flags + 1);
    return hipSuccess;
}

}  // namespace amr
