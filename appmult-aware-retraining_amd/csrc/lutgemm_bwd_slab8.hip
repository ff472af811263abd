// Backward LUT-GEMM, gradient of B, 8-bit tables, for large M on gfx950: "expanded-table" kernel with the entries held
// as the int16 values of the table.
//
// Same result (to fp32 summation order) as lutgemm_gradB_kernel and as the reference's
// ApproxGemmBackwardKernelForGB (self_ops/src/approx_gemm_backward.cu:269-492):
//       gB[k,n] = 1/16 * sum_m G[A[m,k]][B[k,n]] * gC[m,n]
//
// The gradient tables of an 8-bit multiplier span more than the 4096 consecutive integers a half can hold exactly
// (16 x the gradient is about 16 * 255), so the half-precision slab of the narrower tables does not apply; a float32
// slab would hold two k per 128 KB.  Here the slab keeps the int16 entries,
//       S[kk][a][c] = G[a][ B[k0+kk, n0+c] ]          (a = every operand code, kk < 4; 128 B per code and k)
// four k in 128 KB, and an entry costs one conversion (v_cvt_f32_i32 on a 16-bit half of a register) in front of
// its multiply-add: two vector instructions per multiply-add instead of one gather from LDS with 2.5 lanes per bank.
// Every entry is exact, whatever the table holds: no offset, no column sums of gC, no fall-back.  (uint8 operands
// cannot hold a masked code 256.)
//
// LDS layout: byte address = (kk>>1)*65536 + a*256 + (kk&1)*128 + 2*pos(c): the two k of a pair share a 256 B row;
// column c of the tile sits at position pos(c) = 8*((c%32)/4) + 4*(c/32) + c%4 of its 128 B half-row, so that the
// 16 bytes a lane reads (column group cg) hold columns 4cg..4cg+3 and 32+4cg..32+4cg+3 and its two 16-byte loads of
// a row of gC belong to two instructions that each cover 128 contiguous bytes per row.
// Lane = (row slot rs of 8, column group cg of 8): per row of A it reads its eight columns of all four k with 128-bit
// reads (one v_perm_b32 per eight multiply-adds).  The LDS serves 16 lanes of such a read together, i.e. two row slots:
// odd slots visit the two k of every pair in the other order than even ones, so that one reads a 128 B half-row in
// banks 0-31 and the other one in banks 32-63 whatever the codes are.
// Requires K % 4 == 0, N % 64 == 0, M % 256 == 0, gC 16-byte aligned and 32-bit offsets (the launcher checks).
#include "amr_common.h"

namespace amr {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kB8KT = 4;                              // k per workgroup (128 KB of LDS)
constexpr int kB8RU = 2;                              // row groups (of 8 rows) per wave and iteration
constexpr int kB8RowsPerIter = 16 * kB8RU * 8;        // rows a workgroup consumes per iteration

__global__ __launch_bounds__(1024) void lutgemm_gradB_slab8_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ out,
    const int16_t* __restrict__ G, int lut_cols, int M, int K, int N, int m_chunk, float scale, int n_tiles, int k_tiles,
    int splits) {
    constexpr int KT = kB8KT;
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
    // the codes of B of a unit (lanes = its 64 columns, four k) are loaded while the previous unit is being finished
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

        {   // The slabs are gathered from the table in global memory (132 KB: it stays in the L2), a table row (code a, 256
            // entries = 512 B) per wave at a time: the row comes in with two coalesced dword loads per lane, goes to a
            // 512 B spot of LDS that only this wave uses, and every lane (= column) picks the entries of its four codes of B
            // from there.  (Gathering from global memory itself, 64 two-byte loads per thread whose lanes scatter over a row,
            // took 14 us per unit: more than streaming 2048 rows.)
            const int col = lane;
            __syncthreads();
            const unsigned char* gbytes8 = reinterpret_cast<const unsigned char*>(G);
            uint32_t* stage = reinterpret_cast<uint32_t*>(smem + 2 * 65536 + wave * 1024);
            unsigned char* s_col = smem + 2 * (8 * ((col & 31) >> 2) + 4 * (col >> 5) + (col & 3));
#pragma unroll 1
            for (int half = 0; half < 2; ++half) {             // (eight rows = 16 loads of a thread in flight at a time)
                uint32_t r0[8], r1[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const unsigned char* row = gbytes8 + (size_t)(wave + 16 * (8 * half + i)) * (size_t)lut_cols * 2 + 4 * lane;
                    r0[i] = load_u32_unaligned(row);
                    r1[i] = load_u32_unaligned(row + 256);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    uint32_t* st = stage + (i & 1) * 128;      // (two spots in turn: the next row is written while this one is read)
                    st[lane] = r0[i];
                    st[64 + lane] = r1[i];
                    // (read back as 16-bit entries through a type that may alias the dwords just written: with plain uint16_t
                    // the compiler is free to move these reads in front of those writes)
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

        // address pieces: byte0 = half-row (pair member) and column group, byte1 = code (v_perm), byte2 = pair (byte 3 of
        // the lane's constant holds the 1 the second pair needs)
        const uint32_t lo_even = (swap << 7) | (uint32_t)(cg << 4) | 0x01000000u;          // reads 0, 2
        const uint32_t lo_odd = ((swap ^ 1u) << 7) | (uint32_t)(cg << 4) | 0x01000000u;    // reads 1, 3
        uint32_t sel[4];                                                                    // code byte of read j: j ^ swap
#pragma unroll
        for (int j = 0; j < 4; ++j) sel[j] = (j >= 2 ? 0x0c030400u : 0x0c0c0400u) + ((uint32_t)(j ^ (int)swap) << 8);
        const int ncol = n0 + 4 * cg;

        float acc[4][8];       // acc[j]: k = k0 + (j ^ swap); columns 4cg..4cg+3, 32+4cg..32+4cg+3
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[j][c] = 0.f;

        constexpr int RU = kB8RU;
        auto consume = [&](uint32_t a4, const f32x4& g0, const f32x4& g1) __attribute__((always_inline)) {
            u32x4 s[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t addr = __builtin_amdgcn_perm(a4, (j & 1) ? lo_odd : lo_even, sel[j]);
                s[j] = *reinterpret_cast<const u32x4*>(smem + addr);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // (entries 2q and 2q+1 of the 16 bytes are the halves of dword q, sign-extended by the conversion)
                acc[j][0] = __builtin_fmaf(g0.x, (float)(int16_t)(s[j].x & 0xffffu), acc[j][0]);
                acc[j][1] = __builtin_fmaf(g0.y, (float)((int32_t)s[j].x >> 16), acc[j][1]);
                acc[j][2] = __builtin_fmaf(g0.z, (float)(int16_t)(s[j].y & 0xffffu), acc[j][2]);
                acc[j][3] = __builtin_fmaf(g0.w, (float)((int32_t)s[j].y >> 16), acc[j][3]);
                acc[j][4] = __builtin_fmaf(g1.x, (float)(int16_t)(s[j].z & 0xffffu), acc[j][4]);
                acc[j][5] = __builtin_fmaf(g1.y, (float)((int32_t)s[j].z >> 16), acc[j][5]);
                acc[j][6] = __builtin_fmaf(g1.z, (float)(int16_t)(s[j].w & 0xffffu), acc[j][6]);
                acc[j][7] = __builtin_fmaf(g1.w, (float)((int32_t)s[j].w >> 16), acc[j][7]);
            }
        };

        {
            const int iters = (me - mb) / kB8RowsPerIter;
            uint32_t aoff[RU], goff[RU];
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                const uint32_t m = (uint32_t)(mb + 8 * (wave * RU + u) + rs);
                aoff[u] = m * (uint32_t)K + (uint32_t)k0;
                goff[u] = (m * (uint32_t)N + (uint32_t)ncol) * 4u;
            }
            const uint32_t astep = (uint32_t)kB8RowsPerIter * (uint32_t)K;
            const uint32_t gstep = (uint32_t)kB8RowsPerIter * (uint32_t)N * 4u;
            const unsigned char* gbytes = reinterpret_cast<const unsigned char*>(gC);
            uint32_t ca[RU], cb[RU];
            f32x4 ga0[RU], ga1[RU], gb0[RU], gb1[RU];
            // Every load batch is issued unconditionally (beyond the end: the last rows again, nobody consumes them): behind
            // a branch around the loads the compiler's wait in front of the consumer would have to cover the path without
            // new loads too, and no load would be in flight during the arithmetic.
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
                    for (int u = 0; u < RU; ++u) consume(ca[u], ga0[u], ga1[u]);
                    load(ca, ga0, ga1);
#pragma unroll
                    for (int u = 0; u < RU; ++u) consume(cb[u], gb0[u], gb1[u]);
                }
                if (it < iters) {
#pragma unroll
                    for (int u = 0; u < RU; ++u) consume(ca[u], ga0[u], ga1[u]);
                }
            }
        }
        load_b_codes(logical + (int)(gridDim.x / 8), bnext);       // (beyond the last unit: the last one again, unused)

        // The 8 row slots x 16 waves meet in LDS (the slabs are no longer needed): every lane leaves its 32 sums there with
        // eight 16-byte writes, red[wave][rs][k][64 columns] (128 KB), and the sums over (wave, rs) are formed in a fixed
        // order: four partial sums of 32 terms per output by all 1024 threads, then their sum.  (Adding the row slots in
        // registers first took 96 cross-lane operations per wave and unit.)
        __syncthreads();
        float* red = reinterpret_cast<float*>(smem);
        {
            float* r = red + (size_t)((wave * 8 + rs) * KT) * 64 + 4 * cg;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int kk = j ^ (int)swap;
                const f32x4 lo = {acc[j][0], acc[j][1], acc[j][2], acc[j][3]}, hi = {acc[j][4], acc[j][5], acc[j][6], acc[j][7]};
                // (odd row slots keep their two halves of a row of 64 the other way round: the 16 lanes the LDS serves
                // together then write 64 different banks)
                *reinterpret_cast<f32x4*>(r + kk * 64 + 32 * (int)swap) = lo;
                *reinterpret_cast<f32x4*>(r + kk * 64 + 32 * (int)(swap ^ 1u)) = hi;
            }
        }
        __syncthreads();
        float part = 0.f;
        {
            const int o = tid & 255, p = tid >> 8;          // output (k, column) and quarter of the (wave, rs) pairs
            const float* r = red + (size_t)(p * 32 * KT) * 64;
#pragma unroll 8
            for (int t = 0; t < 32; ++t) part += r[t * KT * 64 + (o ^ ((t & 1) << 5))];      // (t % 2 = parity of the row slot)
        }
        __syncthreads();
        red[tid] = part;
        __syncthreads();
        if (tid < KT * 64) {
            const int kk = tid >> 6, col = tid & 63;
            const float v = ((red[tid] + red[256 + tid]) + red[512 + tid]) + red[768 + tid];
            out[((size_t)split * K + k0 + kk) * N + n0 + col] = v * scale;
        }
        // (the barrier at the top of the next unit's slab build keeps these reads ahead of its writes)
    }
}

// ------------------------------------------------------------------------------------------ float32 tables, 8 bits
// The same for an 8-bit table of float32 entries (the direct kernel needs two passes over every gather there: the table,
// 258 KB, does not fit the LDS).  The slab keeps the entries themselves, S[kk][a][c] = G[a][B[k0+kk, n0+c]] as float32,
// 256 B per code and k in the natural column order, two k in 128 KB, and a multiply-add is one v_fma_f32 (no conversion);
// a 128-bit read brings four entries.  Lane = (row slot rs of 8, column group cg of 8): per row of A it reads columns
// 4cg..4cg+3 and 32+4cg..32+4cg+3 of both k; odd row slots take the two halves of a 256 B row in the other order (and
// load their two pieces of gC in that order), so that the 16 lanes the LDS serves together read 64 different banks.
// Requires K % 4 == 0, N % 64 == 0, M % 256 == 0, gC 16-byte aligned and 32-bit offsets (the launcher checks).
constexpr int kB8fKT = 2;

__global__ __launch_bounds__(1024) void lutgemm_gradB_slab8f_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ out,
    const float* __restrict__ G, int lut_cols, int M, int K, int N, int m_chunk, float scale, int n_tiles, int k_tiles,
    int splits) {
    constexpr int KT = kB8fKT;
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

        {   // Slab build: a table row (code a, 256 entries = 1 KB) per wave at a time comes in with four coalesced dword
            // loads per lane, goes to 1 KB of LDS that only this wave uses, and every lane (= column) picks the entries of
            // its two codes of B from there.  Eight rows = 32 loads of a thread are in flight at a time.
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

        // address pieces: byte0 = half of the row and column group, byte1 = code (v_perm), byte2 = k (byte 3 of the lane's
        // constant holds the 1 the second k needs)
        const uint32_t lo_first = (swap << 7) | (uint32_t)(cg << 4) | 0x01000000u;          // reads 0, 2
        const uint32_t lo_second = ((swap ^ 1u) << 7) | (uint32_t)(cg << 4) | 0x01000000u;  // reads 1, 3
        const int ncol = n0 + 4 * cg;

        float acc[4][4];       // acc[j]: k = k0 + j / 2; columns 32 ((j % 2) ^ swap) + 4cg .. + 3
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[j][c] = 0.f;

        constexpr int RU = kB8RU;
        // a2: the codes of the two k in bytes 0 and 1; gf / gs: the lane's first and second piece of the row of gC
        auto consume = [&](uint32_t a2, const f32x4& gf, const f32x4& gs) __attribute__((always_inline)) {
            f32x4 s[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t sel = (j >= 2 ? 0x0c030400u : 0x0c0c0400u) + ((uint32_t)(j >> 1) << 8);
                const uint32_t addr = __builtin_amdgcn_perm(a2, (j & 1) ? lo_second : lo_first, sel);
                s[j] = *reinterpret_cast<const f32x4*>(smem + addr);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4& gv = (j & 1) ? gs : gf;
                acc[j][0] = __builtin_fmaf(gv.x, s[j].x, acc[j][0]);
                acc[j][1] = __builtin_fmaf(gv.y, s[j].y, acc[j][1]);
                acc[j][2] = __builtin_fmaf(gv.z, s[j].z, acc[j][2]);
                acc[j][3] = __builtin_fmaf(gv.w, s[j].w, acc[j][3]);
            }
        };

        {
            const int iters = (me - mb) / kB8RowsPerIter;
            uint32_t aoff[RU], goff[RU];
#pragma unroll
            for (int u = 0; u < RU; ++u) {
                const uint32_t m = (uint32_t)(mb + 8 * (wave * RU + u) + rs);
                aoff[u] = m * (uint32_t)K + (uint32_t)k0;
                goff[u] = (m * (uint32_t)N + (uint32_t)ncol) * 4u;
            }
            const uint32_t astep = (uint32_t)kB8RowsPerIter * (uint32_t)K;
            const uint32_t gstep = (uint32_t)kB8RowsPerIter * (uint32_t)N * 4u;
            const uint32_t first = 128u * swap, second = 128u * (swap ^ 1u);      // byte offsets of the lane's two pieces of a row of gC
            const unsigned char* gbytes = reinterpret_cast<const unsigned char*>(gC);
            uint32_t ca[RU], cb[RU];
            f32x4 ga0[RU], ga1[RU], gb0[RU], gb1[RU];
            int next = 0;
            // (every load batch is issued unconditionally, beyond the end the last rows again: see the int16 kernel)
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
            if (iters > 0) {
                load(ca, ga0, ga1);
                int it = 0;
                for (; it + 2 <= iters; it += 2) {
                    load(cb, gb0, gb1);
#pragma unroll
                    for (int u = 0; u < RU; ++u) consume(ca[u], ga0[u], ga1[u]);
                    load(ca, ga0, ga1);
#pragma unroll
                    for (int u = 0; u < RU; ++u) consume(cb[u], gb0[u], gb1[u]);
                }
                if (it < iters) {
#pragma unroll
                    for (int u = 0; u < RU; ++u) consume(ca[u], ga0[u], ga1[u]);
                }
            }
        }
        load_b_codes(logical + (int)(gridDim.x / 8), bnext);       // (beyond the last unit: the last one again, unused)

        // The 8 row slots x 16 waves meet in LDS, red[wave][rs][k][64 columns] (64 KB): 16 partial sums of 8 terms per
        // output by all 1024 threads (2 k x 64 columns x 8 parts), then their sum, in a fixed order.
        __syncthreads();
        float* red = reinterpret_cast<float*>(smem);
        {
            float* r = red + (size_t)((wave * 8 + rs) * KT) * 64 + 4 * cg;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 v = {acc[j][0], acc[j][1], acc[j][2], acc[j][3]};
                *reinterpret_cast<f32x4*>(r + (j >> 1) * 64 + 32 * ((j & 1) ^ (int)swap)) = v;
            }
        }
        __syncthreads();
        float part = 0.f;
        {
            const int o = tid & 127, p = tid >> 7;          // output (k, column) and eighth of the (wave, rs) pairs
            const float* r = red + (size_t)(p * 16 * KT) * 64 + o;
#pragma unroll
            for (int t = 0; t < 16; ++t) part += r[t * KT * 64];
        }
        __syncthreads();
        red[tid] = part;
        __syncthreads();
        if (tid < KT * 64) {
            const int kk = tid >> 6, col = tid & 63;
            float v = 0.f;
#pragma unroll
            for (int p = 0; p < 8; ++p) v += red[128 * p + tid];
            out[((size_t)split * K + k0 + kk) * N + n0 + col] = v * scale;
        }
        // (the barrier at the top of the next unit's slab build keeps these reads ahead of its writes)
    }
}

// ------------------------------------------------------------------------------------------ host
__global__ void reduce_partials_kernel(const float* __restrict__ partial, float* __restrict__ out, size_t count, int splits);

// (measured on MI355X against the direct kernel: 2.9 x faster at 131072 rows, 2.1 x at 8192, 1.45 x at 2048; at 512 rows
// the build of the slabs outweighs the streaming; `force`: from 1024 rows)
bool gradB_slab8_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force) {
    const bool small = (size_t)M * K < (1ull << 31) && (size_t)M * N * 4 < (1ull << 31);
    return g.bits == 8 && M >= (force ? 1024 : 2048) && (M % kB8RowsPerIter) == 0 && (K & 3) == 0 && (N & 63) == 0 && small &&
           ((uintptr_t)gC & 15) == 0;
}

// M splits: as many as keep every CU busy, at least 2048 rows per workgroup (building the slabs of a unit costs about as
// much as streaming 700 rows).
int gradB_slab8_splits(int M, int K, int N, int n_cu) {
    const long per_split = (long)(N / 64) * (K / kB8KT);
    long max_s = M / 2048;
    if (max_s > 64) max_s = 64;
    if (max_s < 1) max_s = 1;
    long best_s = 1, best_cost = -1;
    for (long sp = 1; sp <= max_s; ++sp) {
        long chunk = (M + sp - 1) / sp;
        chunk = (chunk + kB8RowsPerIter - 1) / kB8RowsPerIter * kB8RowsPerIter;
        const long zs = (M + chunk - 1) / chunk;
        const long rounds = (per_split * zs + n_cu - 1) / n_cu;
        const long cost = rounds * (chunk + 700);
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_s = sp; }
    }
    return (int)best_s;
}

// partials: room for gradB_slab8_splits(...) x K x N floats when that is more than one.
hipError_t launch_gradB_slab8(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                              const LutGeom& g, int M, int K, int N, float scale, float* partials, int n_cu,
                              hipStream_t stream, int split_cap) {
    // split_cap > 0: the most M splits the caller's scratch has room for
    int splits = gradB_slab8_splits(M, K, N, n_cu);
    if (split_cap > 0 && splits > split_cap) splits = split_cap;
    int m_chunk = (M + splits - 1) / splits;
    m_chunk = (m_chunk + kB8RowsPerIter - 1) / kB8RowsPerIter * kB8RowsPerIter;
    const int zs = (M + m_chunk - 1) / m_chunk;
    float* out = zs > 1 ? partials : gB;
    const int n_tiles = N / 64, k_tiles = K / kB8KT;
    const int total = n_tiles * k_tiles * zs;
    const int per_xcd = (total + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    hipLaunchKernelGGL(lutgemm_gradB_slab8_kernel, dim3(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd)), dim3(1024), 0,
                       stream, gC, A, B, out, lut, g.cols, M, K, N, m_chunk, scale, n_tiles, k_tiles, zs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (zs > 1) {
        const size_t count = (size_t)K * N;
        hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, partials, gB,
                           count, zs);
        e = hipGetLastError();
    }
    return e;
}

bool gradB_slab8f_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force) {
    const bool small = (size_t)M * K < (1ull << 31) && (size_t)M * N * 4 < (1ull << 31);
    return g.bits == 8 && M >= (force ? 1024 : 2048) && (M % kB8RowsPerIter) == 0 && (K & 3) == 0 && (N & 63) == 0 && small &&
           ((uintptr_t)gC & 15) == 0;
}

// M splits of the float32 variant (two k per unit).
int gradB_slab8f_splits(int M, int K, int N, int n_cu) {
    const long per_split = (long)(N / 64) * (K / kB8fKT);
    long max_s = M / 2048;
    if (max_s > 64) max_s = 64;
    if (max_s < 1) max_s = 1;
    long best_s = 1, best_cost = -1;
    for (long sp = 1; sp <= max_s; ++sp) {
        long chunk = (M + sp - 1) / sp;
        chunk = (chunk + kB8RowsPerIter - 1) / kB8RowsPerIter * kB8RowsPerIter;
        const long zs = (M + chunk - 1) / chunk;
        const long rounds = (per_split * zs + n_cu - 1) / n_cu;
        const long cost = rounds * (chunk + 1400);
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_s = sp; }
    }
    return (int)best_s;
}

// partials: room for gradB_slab8f_splits(...) x K x N floats when that is more than one.
hipError_t launch_gradB_slab8f(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut,
                               const LutGeom& g, int M, int K, int N, float scale, float* partials, int n_cu,
                               hipStream_t stream) {
    const int splits = gradB_slab8f_splits(M, K, N, n_cu);
    int m_chunk = (M + splits - 1) / splits;
    m_chunk = (m_chunk + kB8RowsPerIter - 1) / kB8RowsPerIter * kB8RowsPerIter;
    const int zs = (M + m_chunk - 1) / m_chunk;
    float* out = zs > 1 ? partials : gB;
    const int n_tiles = N / 64, k_tiles = K / kB8fKT;
    const int total = n_tiles * k_tiles * zs;
    const int per_xcd = (total + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    hipLaunchKernelGGL(lutgemm_gradB_slab8f_kernel, dim3(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd)), dim3(1024), 0,
                       stream, gC, A, B, out, lut, g.cols, M, K, N, m_chunk, scale, n_tiles, k_tiles, zs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (zs > 1) {
        const size_t count = (size_t)K * N;
        hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, partials, gB,
                           count, zs);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace amr
