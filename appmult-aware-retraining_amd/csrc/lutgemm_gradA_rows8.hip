// Backward LUT-GEMM, gradient of A, 8-bit tables (int16 or float32), for layers of 2048 to 8192 rows on gfx950.
//
// Same result (to fp32 summation order) as lutgemm_gradA_kernel and as the reference's
// ApproxGemmBackwardKernelForGA (self_ops/src/approx_gemm_backward.cu:21-258):
//       gA[m,k] = 1/16 * sum_n gC[m,n] * G[A[m,k]][B[k,n]]
//
// The expanded-table kernel of lutgemm_gradA_slab.hip writes K*N*512 B of table to memory whatever M is: with 2048 rows
// that is 1.2 GB for a 4608 x 512 layer, a third of the kernel's time, and every 512 rows stream all of it.  Here the
// table is expanded per workgroup in LDS instead, exactly as lutgemm_gradB_slab8_kernel does it: a workgroup owns four
// k and one 64-column tile of B, S[kk][a][c] = G[a][B[k0+kk, n0+c]] as int16 (128 KB), and streams rows of A and gC
// through it.  Per row it forms the four sums over its 64 columns -- eight columns per lane, then across the eight
// lanes of the row slot -- and leaves them in a buffer of partial results P[column tile][k tile][m][4]; a second kernel
// adds the column tiles in a fixed order and writes gA (row-major or image-major).  One conversion
// (v_cvt_f32_i32 on a 16-bit half of a register) per entry as in the other 8-bit kernels: exact for any table.
//
// LDS layout, lane mapping and bank behaviour are those of lutgemm_gradB_slab8_kernel (lutgemm_bwd_slab8.hip): byte address
// = (kk>>1)*65536 + a*256 + (kk&1)*128 + 2*pos(c), lane = (row slot rs of 8, column group cg of 8), odd row slots visit
// the two k of a pair in the other order.
// Requires K % 4 == 0, N % 64 == 0, M % 256 == 0, gC 16-byte aligned and 32-bit offsets (the launcher checks).
#include "amr_common.h"

namespace amr {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kR8KT = 4;                              // k per workgroup (128 KB of LDS)
constexpr int kR8RU = 2;                              // row groups (of 8 rows) per wave and iteration
constexpr int kR8RowsPerIter = 16 * kR8RU * 8;        // rows a workgroup consumes per iteration

// the value lane (l ^ 1) / (l ^ 2) of the quad holds
__device__ __forceinline__ float r8_quad_xor1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
}
__device__ __forceinline__ float r8_quad_xor2(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
}

// P: [n_tiles][k_tiles][M][4] floats.
__global__ __launch_bounds__(1024) void lutgemm_gradA_rows8_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ P,
    const int16_t* __restrict__ G, int lut_cols, int M, int K, int N, int m_chunk, int n_tiles, int k_tiles, int splits) {
    constexpr int KT = kR8KT;
    __shared__ __align__(16) unsigned char smem[2 * 65536 + 16 * 1024];   // slabs + 1 KB per wave for the slab build
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 3, cg = lane & 7;
    const uint32_t swap = (uint32_t)(rs & 1);
    // Workgroups are dealt to the 8 XCDs round-robin by their index; the workgroups of one XCD (same index mod 8) take
    // consecutive k tiles of one (column tile, M split), so that the rows of gC and A they all stream are shared in
    // that XCD's L2.  A workgroup keeps its CU and takes every (gridDim.x / 8)-th unit of its XCD's share.
    const int total = n_tiles * k_tiles * splits;
    const int per_xcd = (total + 7) / 8;
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

        {   // slab build: table rows staged in LDS, see lutgemm_gradB_slab8_kernel
            const int col = lane;
            __syncthreads();
            const unsigned char* gbytes8 = reinterpret_cast<const unsigned char*>(G);
            uint32_t* stage = reinterpret_cast<uint32_t*>(smem + 2 * 65536 + wave * 1024);
            unsigned char* s_col = smem + 2 * (8 * ((col & 31) >> 2) + 4 * (col >> 5) + (col & 3));
#pragma unroll 1
            for (int half = 0; half < 2; ++half) {
                uint32_t r0[8], r1[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const unsigned char* row = gbytes8 + (size_t)(wave + 16 * (8 * half + i)) * (size_t)lut_cols * 2 + 4 * lane;
                    r0[i] = load_u32_unaligned(row);
                    r1[i] = load_u32_unaligned(row + 256);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    uint32_t* st = stage + (i & 1) * 128;
                    st[lane] = r0[i];
                    st[64 + lane] = r1[i];
                    typedef uint16_t __attribute__((may_alias)) u16_alias;
                    const u16_alias* s16 = reinterpret_cast<const u16_alias*>(st);
                    const int a = wave + 16 * (8 * half + i);
#pragma unroll
                    for (int kk = 0; kk < KT; ++kk)
                        *reinterpret_cast<uint16_t*>(s_col + (kk >> 1) * 65536 + (kk & 1) * 128 + a * 256) = s16[bnext[kk]];
                }
            }
        }
        __syncthreads();

        const uint32_t lo_even = (swap << 7) | (uint32_t)(cg << 4) | 0x01000000u;          // reads 0, 2
        const uint32_t lo_odd = ((swap ^ 1u) << 7) | (uint32_t)(cg << 4) | 0x01000000u;    // reads 1, 3
        uint32_t sel[4];                                                                    // code byte of read j: j ^ swap
#pragma unroll
        for (int j = 0; j < 4; ++j) sel[j] = (j >= 2 ? 0x0c030400u : 0x0c0c0400u) + ((uint32_t)(j ^ (int)swap) << 8);
        const int ncol = n0 + 4 * cg;
        // the partial results of this unit: rows mb .. me - 1 of block (n_tile, k_tile), four floats (k0 .. k0 + 3) per row.
        // After the sums have met, lane cg < 4 of a row slot holds the one of index 2 (cg % 2) + (cg / 2) % 2, which is
        // k = k0 + (index ^ swap).
        float* pu = P + ((size_t)(n_tile * k_tiles + k_tile) * (size_t)M) * 4;
        const bool bit0 = (cg & 1) != 0, bit1 = (cg & 2) != 0;
        const uint32_t kl = (uint32_t)((2 * (cg & 1) + ((cg >> 1) & 1)) ^ (int)swap);

        constexpr int RU = kR8RU;
        // one row: four 128-bit slab reads (one per k), 32 conversions and multiply-adds, the sums over the eight lanes
        auto consume = [&](uint32_t a4, const f32x4& g0, const f32x4& g1, int m) __attribute__((always_inline)) {
            u32x4 s[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t addr = __builtin_amdgcn_perm(a4, (j & 1) ? lo_odd : lo_even, sel[j]);
                s[j] = *reinterpret_cast<const u32x4*>(smem + addr);
            }
            float d[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // (entries 2q and 2q+1 of the 16 bytes are the halves of dword q, sign-extended by the conversion; two chains)
                float lo = g0.x * (float)(int16_t)(s[j].x & 0xffffu);
                float hi = g1.x * (float)(int16_t)(s[j].z & 0xffffu);
                lo = __builtin_fmaf(g0.y, (float)((int32_t)s[j].x >> 16), lo);
                hi = __builtin_fmaf(g1.y, (float)((int32_t)s[j].z >> 16), hi);
                lo = __builtin_fmaf(g0.z, (float)(int16_t)(s[j].y & 0xffffu), lo);
                hi = __builtin_fmaf(g1.z, (float)(int16_t)(s[j].w & 0xffffu), hi);
                lo = __builtin_fmaf(g0.w, (float)((int32_t)s[j].y >> 16), lo);
                hi = __builtin_fmaf(g1.w, (float)((int32_t)s[j].w >> 16), hi);
                d[j] = lo + hi;
            }
            // four sums over eight lanes in three exchanges: lanes l and l ^ 1 split the four indices between them (even
            // lanes keep 0 and 1), lanes l and l ^ 2 the two each is left with, lanes l and l ^ 4 add what remains
            const float keep0 = bit0 ? d[2] : d[0], keep1 = bit0 ? d[3] : d[1];
            const float send0 = bit0 ? d[0] : d[2], send1 = bit0 ? d[1] : d[3];
            const float r0 = keep0 + r8_quad_xor1(send0), r1 = keep1 + r8_quad_xor1(send1);
            float q = (bit1 ? r1 : r0) + r8_quad_xor2(bit1 ? r0 : r1);
            q += __shfl_xor(q, 4);
            if (cg < 4) pu[(size_t)m * 4 + kl] = q;
        };

        {
            const int iters = (me - mb) / kR8RowsPerIter;
            uint32_t aoff[RU], goff[RU];
            int mrow[RU];
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                mrow[u] = mb + 8 * (wave * RU + u) + rs;
                aoff[u] = (uint32_t)mrow[u] * (uint32_t)K + (uint32_t)k0;
                goff[u] = ((uint32_t)mrow[u] * (uint32_t)N + (uint32_t)ncol) * 4u;
            }
            const uint32_t astep = (uint32_t)kR8RowsPerIter * (uint32_t)K;
            const uint32_t gstep = (uint32_t)kR8RowsPerIter * (uint32_t)N * 4u;
            const unsigned char* gbytes = reinterpret_cast<const unsigned char*>(gC);
            uint32_t ca[RU], cb[RU];
            f32x4 ga0[RU], ga1[RU], gb0[RU], gb1[RU];
            // (every load batch is issued unconditionally, beyond the end the last rows again, which nobody consumes)
            int next = 0, done = 0;
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
                __builtin_amdgcn_sched_barrier(0);
            };
            auto consume_batch = [&](uint32_t (&c4)[RU], f32x4 (&g0)[RU], f32x4 (&g1)[RU]) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < RU; ++u) consume(c4[u], g0[u], g1[u], mrow[u] + done * kR8RowsPerIter);
                ++done;
            };
            if (iters > 0) {
                load(ca, ga0, ga1);
                int it = 0;
                for (; it + 2 <= iters; it += 2) {
                    load(cb, gb0, gb1);
                    consume_batch(ca, ga0, ga1);
                    load(ca, ga0, ga1);
                    consume_batch(cb, gb0, gb1);
                }
                if (it < iters) consume_batch(ca, ga0, ga1);
            }
        }
        load_b_codes(logical + (int)(gridDim.x / 8), bnext);       // (beyond the last unit: the last one again, unused)
        // (the barrier at the top of the next unit's slab build keeps the slab reads of this unit ahead of its writes)
    }
}

// gA[m][KT kt .. KT kt + KT - 1] = scale * sum over the column tiles, in their order, of P[nt][kt][m][0 .. KT - 1].
// grid (ceil(M / 256), k_tiles), 256 threads; rows_per_image = 0: gA row-major [M,K]; L > 0: gA[m / L][k][m % L].
template <int KT>
__global__ __launch_bounds__(256) void gradA_rows8_finish_kernel(const float* __restrict__ P, float* __restrict__ gA, int M, int K,
                                                                 int n_tiles, int k_tiles, float scale, int rows_per_image) {
    typedef float vec_t __attribute__((ext_vector_type(KT)));
    const int m = (int)blockIdx.x * 256 + (int)threadIdx.x;
    const int kt = (int)blockIdx.y;
    if (m >= M) return;
    const vec_t* p = reinterpret_cast<const vec_t*>(P) + (size_t)kt * (size_t)M + m;
    vec_t v = p[0];
    for (int nt = 1; nt < n_tiles; ++nt) v += p[(size_t)nt * (size_t)k_tiles * (size_t)M];
    if (rows_per_image > 0) {
        const int img = m / rows_per_image, l = m - img * rows_per_image;
        float* o = gA + ((size_t)img * K + KT * kt) * rows_per_image + l;
#pragma unroll
        for (int i = 0; i < KT; ++i) o[(size_t)i * rows_per_image] = v[i] * scale;
    } else {
        float* o = gA + (size_t)m * K + KT * kt;
#pragma unroll
        for (int i = 0; i < KT; ++i) o[i] = v[i] * scale;
    }
}

// ------------------------------------------------------------------------------------------ float32 tables
// The same for an 8-bit table of float32 entries, with the slab and lane mapping of lutgemm_gradB_slab8f_kernel: two k per
// workgroup, S[kk][a][c] as float32 (256 B per code and k, natural column order), a v_fma_f32 per entry; odd row slots
// take the two halves of a row in the other order.  P: [n_tiles][k_tiles][M][2] floats.
constexpr int kR8fKT = 2;

__global__ __launch_bounds__(1024) void lutgemm_gradA_rows8f_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ P,
    const float* __restrict__ G, int lut_cols, int M, int K, int N, int m_chunk, int n_tiles, int k_tiles, int splits) {
    constexpr int KT = kR8fKT;
    __shared__ __align__(16) unsigned char smem[2 * 65536 + 16 * 1024];   // slabs + 1 KB per wave for the slab build
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 3, cg = lane & 7;
    const uint32_t swap = (uint32_t)(rs & 1);
    const int total = n_tiles * k_tiles * splits;
    const int per_xcd = (total + 7) / 8;
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

        {   // slab build: table rows (256 entries = 1 KB) staged in LDS, see lutgemm_gradB_slab8f_kernel
            const int col = lane;
            __syncthreads();
            float* stage = reinterpret_cast<float*>(smem + 2 * 65536 + wave * 1024);
            float* s_col = reinterpret_cast<float*>(smem) + col;
#pragma unroll 1
            for (int half = 0; half < 2; ++half) {
                float r[8][4];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float* row = G + (size_t)(wave + 16 * (8 * half + i)) * (size_t)lut_cols + lane;
#pragma unroll
                    for (int q = 0; q < 4; ++q) r[i][q] = row[64 * q];
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) stage[64 * q + lane] = r[i][q];
                    const int a = wave + 16 * (8 * half + i);
#pragma unroll
                    for (int kk = 0; kk < KT; ++kk) s_col[kk * 16384 + a * 64] = stage[bnext[kk]];
                }
            }
        }
        __syncthreads();

        const uint32_t lo_first = (swap << 7) | (uint32_t)(cg << 4) | 0x01000000u;          // reads 0, 2
        const uint32_t lo_second = ((swap ^ 1u) << 7) | (uint32_t)(cg << 4) | 0x01000000u;  // reads 1, 3
        const int ncol = n0 + 4 * cg;
        // partial results of this unit: two floats (k0, k0 + 1) per row; after the sums have met, lanes cg = 0, 1 of a row
        // slot hold those of k0 + cg
        float* pu = P + ((size_t)(n_tile * k_tiles + k_tile) * (size_t)M) * 2;
        const bool bit0 = (cg & 1) != 0;

        constexpr int RU = kR8RU;
        // a2: the codes of the two k in bytes 0 and 1; gf / gs: the lane's first and second piece of the row of gC
        auto consume = [&](uint32_t a2, const f32x4& gf, const f32x4& gs, int m) __attribute__((always_inline)) {
            f32x4 s[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t sel = (j >= 2 ? 0x0c030400u : 0x0c0c0400u) + ((uint32_t)(j >> 1) << 8);
                const uint32_t addr = __builtin_amdgcn_perm(a2, (j & 1) ? lo_second : lo_first, sel);
                s[j] = *reinterpret_cast<const f32x4*>(smem + addr);
            }
            float d[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4& gv = (j & 1) ? gs : gf;
                float t = gv.x * s[j].x;
                t = __builtin_fmaf(gv.y, s[j].y, t);
                t = __builtin_fmaf(gv.z, s[j].z, t);
                d[j] = __builtin_fmaf(gv.w, s[j].w, t);
            }
            const float d0 = d[0] + d[1], d1 = d[2] + d[3];       // k0 and k0 + 1 over the lane's eight columns
            float q = (bit0 ? d1 : d0) + r8_quad_xor1(bit0 ? d0 : d1);
            q += r8_quad_xor2(q);
            q += __shfl_xor(q, 4);
            if (cg < 2) pu[(size_t)m * 2 + cg] = q;
        };

        {
            const int iters = (me - mb) / kR8RowsPerIter;
            uint32_t aoff[RU], goff[RU];
            int mrow[RU];
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                mrow[u] = mb + 8 * (wave * RU + u) + rs;
                aoff[u] = (uint32_t)mrow[u] * (uint32_t)K + (uint32_t)k0;
                goff[u] = ((uint32_t)mrow[u] * (uint32_t)N + (uint32_t)ncol) * 4u;
            }
            const uint32_t astep = (uint32_t)kR8RowsPerIter * (uint32_t)K;
            const uint32_t gstep = (uint32_t)kR8RowsPerIter * (uint32_t)N * 4u;
            const uint32_t first = 128u * swap, second = 128u * (swap ^ 1u);      // byte offsets of the lane's two pieces of a row of gC
            const unsigned char* gbytes = reinterpret_cast<const unsigned char*>(gC);
            uint32_t ca[RU], cb[RU];
            f32x4 ga0[RU], ga1[RU], gb0[RU], gb1[RU];
            int next = 0, done = 0;
            auto load = [&](uint32_t (&c2)[RU], f32x4 (&g0)[RU], f32x4 (&g1)[RU]) {
#pragma unroll
                for (int u = 0; u < RU; ++u) {
                    uint16_t two;
                    __builtin_memcpy(&two, A + aoff[u], 2);
                    c2[u] = two;
                    g0[u] = *reinterpret_cast<const f32x4*>(gbytes + goff[u] + first);
                    g1[u] = *reinterpret_cast<const f32x4*>(gbytes + goff[u] + second);
                }
                ++next;
                const uint32_t as = next < iters ? astep : 0u, gs = next < iters ? gstep : 0u;
#pragma unroll
                for (int u = 0; u < RU; ++u) {
                    aoff[u] += as;
                    goff[u] += gs;
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            auto consume_batch = [&](uint32_t (&c2)[RU], f32x4 (&g0)[RU], f32x4 (&g1)[RU]) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < RU; ++u) consume(c2[u], g0[u], g1[u], mrow[u] + done * kR8RowsPerIter);
                ++done;
            };
            if (iters > 0) {
                load(ca, ga0, ga1);
                int it = 0;
                for (; it + 2 <= iters; it += 2) {
                    load(cb, gb0, gb1);
                    consume_batch(ca, ga0, ga1);
                    load(ca, ga0, ga1);
                    consume_batch(cb, gb0, gb1);
                }
                if (it < iters) consume_batch(ca, ga0, ga1);
            }
        }
        load_b_codes(logical + (int)(gridDim.x / 8), bnext);       // (beyond the last unit: the last one again, unused)
    }
}

// ------------------------------------------------------------------------------------------ host
// (measured on MI355X: from 2048 to 8192 rows this kernel beats both the direct kernel and the expanded-table kernel,
// whose table, written to memory, weighs most there -- 1.2 x at 2048 rows, level at 8192 with int16 tables, 1.35 x at 8192
// with float32 ones; at 32768 rows the expanded-table kernel is 1.2 x faster; `force` lowers the floor to 1024 rows and
// keeps the ceiling)
bool gradA_rows8_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force) {
    const bool small = (size_t)M * K < (1ull << 31) && (size_t)M * N * 4 < (1ull << 31) &&
                       (size_t)(N / 64) * (size_t)M * (size_t)K < (1ull << 32);
    // (the k tiles are gridDim.y of the second kernel: at most 65535 of the float variant's two k)
    return g.bits == 8 && M >= (force ? 1024 : 2048) && M < 16384 && (M % kR8RowsPerIter) == 0 && (K & 3) == 0 && (N & 63) == 0 &&
           K / kR8fKT <= 65535 && small && ((uintptr_t)gC & 15) == 0;
}

// Bytes of the partial results, or 0 when the kernel does not apply (gC's alignment is the caller's to check).
size_t gradA_rows8_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    if (!gradA_rows8_applies(g, M, K, N, nullptr, force)) return 0;
    return (size_t)(N / 64) * (size_t)M * (size_t)K * sizeof(float);
}

// P: gradA_rows8_workspace_bytes(...) bytes of scratch, p_bytes what the caller has there.
hipError_t launch_gradA_rows8(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                              const LutGeom& g, int M, int K, int N, float scale, int n_cu, void* P, size_t p_bytes,
                              int rows_per_image, hipStream_t stream) {
    const int n_tiles = N / 64, k_tiles = K / kR8KT;
    if (p_bytes < (size_t)n_tiles * (size_t)M * (size_t)K * sizeof(float) || ((uintptr_t)P & 15) != 0) return hipErrorInvalidValue;
    // rows per unit: as many units as keep every CU busy twice over, whole multiples of 256 rows, at least 2048
    int splits = 1;
    while (splits < 4 && (long)n_tiles * k_tiles * splits < 2L * n_cu && M / (splits * 2) >= 2048 && (M % (splits * 2 * kR8RowsPerIter)) == 0)
        splits *= 2;
    const int m_chunk = M / splits;
    const int total = n_tiles * k_tiles * splits;
    const int per_xcd = (total + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    hipLaunchKernelGGL(lutgemm_gradA_rows8_kernel, dim3(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd)), dim3(1024), 0,
                       stream, gC, A, B, reinterpret_cast<float*>(P), lut, g.cols, M, K, N, m_chunk, n_tiles, k_tiles, splits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((gradA_rows8_finish_kernel<kR8KT>), dim3((unsigned)((M + 255) / 256), (unsigned)k_tiles), dim3(256), 0, stream,
                       reinterpret_cast<const float*>(P), gA, M, K, n_tiles, k_tiles, scale, rows_per_image);
    return hipGetLastError();
}

// The same for 8-bit float32 tables (same conditions, same amount of scratch: two floats per row and pair of k).
bool gradA_rows8f_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force) {
    return gradA_rows8_applies(g, M, K, N, gC, force);
}
size_t gradA_rows8f_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    return gradA_rows8_workspace_bytes(g, M, K, N, force);
}
hipError_t launch_gradA_rows8f(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                               const LutGeom& g, int M, int K, int N, float scale, int n_cu, void* P, size_t p_bytes,
                               int rows_per_image, hipStream_t stream) {
    const int n_tiles = N / 64, k_tiles = K / kR8fKT;
    if (p_bytes < (size_t)n_tiles * (size_t)M * (size_t)K * sizeof(float) || ((uintptr_t)P & 15) != 0) return hipErrorInvalidValue;
    int splits = 1;
    while (splits < 4 && (long)n_tiles * k_tiles * splits < 2L * n_cu && M / (splits * 2) >= 2048 && (M % (splits * 2 * kR8RowsPerIter)) == 0)
        splits *= 2;
    const int m_chunk = M / splits;
    const int total = n_tiles * k_tiles * splits;
    const int per_xcd = (total + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    hipLaunchKernelGGL(lutgemm_gradA_rows8f_kernel, dim3(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd)), dim3(1024), 0,
                       stream, gC, A, B, reinterpret_cast<float*>(P), lut, g.cols, M, K, N, m_chunk, n_tiles, k_tiles, splits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((gradA_rows8_finish_kernel<kR8fKT>), dim3((unsigned)((M + 255) / 256), (unsigned)k_tiles), dim3(256), 0, stream,
                       reinterpret_cast<const float*>(P), gA, M, K, n_tiles, k_tiles, scale, rows_per_image);
    return hipGetLastError();
}

}  // namespace amr
