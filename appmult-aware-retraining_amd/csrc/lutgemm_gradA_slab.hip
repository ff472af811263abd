// Backward LUT-GEMM, gradient of A, for large M on gfx950: "expanded-table" kernel (7-bit tables and
// narrower).
//
// Same result (to fp32 summation order) as lutgemm_gradA_kernel and as the reference's
// ApproxGemmBackwardKernelForGA (self_ops/src/approx_gemm_backward.cu:21-258):
//       gA[m,k] = 1/16 * sum_n gC[m,n] * G[A[m,k]][B[k,n]]
//
//   step 1  expand_gradA_kernel:  S[k][a][n] = half(G[a][B[k,n]] - offset) for every code a
//   step 2  lutgemm_gradA_slab_kernel:  gA[m,k] = dot(gC[m,:], S[k][A[m,k]][:]) + offset * sum_n gC[m,n]
//
// In step 2 a lane owns one k in four (k = 4j + c, c = lane % 4) of two rows m: it keeps 32 values of gC[m,:]
// per row in registers and, for each of its k, reads ROW a = A[m,k] of S[k] (64 B, four 128-bit LDS reads)
// instead of gathering 32 single entries.  The multiply-add takes the half straight into an fp32 fma
// (v_fma_mix_f32); a half holds every integer of magnitude <= 2048, so with offset 0 table entries in
// [-2048, 2048] are exact (16 x the gradient of a 7-bit multiplier is about 16*b <= 2032), with offset 1024
// entries in [-1024, 3072]; the offset is picked from the extremes of the table (bwd_header_kernel) and sits in
// flags[3].  Products and sums are then the fp32 values an fp32 table would give.  An entry a half cannot
// hold, or a masked code 128 in A (not addressable here), raises flags[2] and the direct kernel, queued
// behind and gated on that flag, recomputes gA.
//
// Layout of S (HBM and LDS): chunks of four k, S[n_tile][k / 4][a (128 rows)][k % 4][32 columns] halves,
// 32 KB each: the four k of a code a share a 256 B row, k % 4 picks a 64 B window = 16 banks.  The four
// lanes of a quad (same m, c = 0..3) read in four different windows; the four quads that the LDS serves
// together read 16 B pieces (q + step) % 4 of their windows, q the quad number: 16 lanes x 4 banks, all
// different whatever the codes are, so the random rows cost no bank conflicts.  (A lane reading a whole
// 64 B row of its own at 80 B pitch, the previous layout, measured 11 LDS clocks per 128-bit read
// instead of 4.)  gC is kept in registers in the same rotated order.
//
// A workgroup (16 waves, one per CU, all 160 KB of LDS) owns 512 rows and KT = 16 or 32 consecutive k and walks
// all column tiles.  The chunks go from L2 to LDS by LDS-direct loads, three buffers, requested two chunks ahead, two
// wave-wide loads per wave and chunk; the rows of gC take the same road (64 KB staging area, every wave its own rows,
// requested a column tile ahead).  The only loads with a register destination are the codes of the next tile (one
// 16-byte load per lane and tile); all waiting is explicit.  The results of a tile leave through LDS as 16-byte
// stores of whole 128 B lines.
// Measured on MI355X: no LDS bank-conflict cycles (4.0 LDS clocks per 128-bit read); 0.77-0.80 us per chunk and
// CU against 0.5 us of v_fma_mix_f32 issue (72 VALU instructions per wave and chunk, four waves per SIMD), plus
// 4 us per tile.
//
// The same kernel serves two more table formats, 16 columns per tile and four chunk buffers each: float32 entries
// (7-bit float tables; a 128-bit read feeds four v_fma_f32) and the int16 entries of an 8-bit table (256 code rows of
// 128 B; a conversion in front of every multiply-add; exact for any table, no offset and no fall-back).
#include <type_traits>

#include "amr_common.h"

namespace amr {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kGaFmtHalf = 0, kGaFmtF32 = 1, kGaFmtI16 = 2, kGaFmtF32W = 3;   // how S holds the entries (W: float32 entries of an 8-bit table)
constexpr int kGaCols = 32;                               // columns per tile (half entries; 16 for float32 entries)
constexpr int kGaColsF32 = 16;
constexpr int kGaColsF32W = 8;                            // float32 entries of an 8-bit table: 256 code rows of 128 B in a 32 KB chunk
constexpr int kGaChunkK = 4;
constexpr int kGaChunkBytes = 128 * kGaChunkK * 2 * kGaCols;   // 32 KB (= 128 codes x 4 k x 16 columns x 4 bytes as well)
constexpr int kGaBufs = 3;
constexpr int kGaWaves = 16;
constexpr int kGaRowsPerWave = 32;                        // 16 quads x 2 rows
constexpr int kGaRows = kGaWaves * kGaRowsPerWave;        // 512 rows per workgroup
constexpr int kGaStageBase = kGaBufs * kGaChunkBytes;     // 96 KB: the rows of gC of one column tile, 128 B per row
constexpr int kGaStageBytes = kGaRows * kGaCols * 4;      // 64 KB (half of it used with float32 entries)
static_assert(kGaStageBase + kGaStageBytes == 160 * 1024, "the workgroup uses the whole LDS of a CU");

// ------------------------------------------------------------------------------------------ expand
// grid (n_tiles, ceil(K / 4 / quads_per_wg)), 256 threads.  Requires N % 32 == 0 and K % 4 == 0.

__global__ __launch_bounds__(256) void expand_gradA_kernel(const uint8_t* __restrict__ B, const uint32_t* __restrict__ lut32,
                                                           int lut_dwords, int lut_cols, int n_codes,
                                                           uint32_t* __restrict__ S, uint32_t* __restrict__ flags, int K, int N, int quads_per_wg) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* s32 = reinterpret_cast<uint32_t*>(smem);
    if (flags[5] != 0u) return;                  // the table cannot be held as halves (bwd_header_kernel): the direct kernel does it
    const float offset = (float)(int)flags[3];   // decided from the table's extremes by bwd_header_kernel
    // The table goes to LDS as halves, converted once per workgroup; what is left per entry of S is two 16-bit LDS
    // reads, one shift-or and the store (the kernel writes 256 B per code and k quad and should run at the speed of
    // the writes: 6.8 TB/s measured for a plain fill).
    bool inexact = false;
    // (eight loads of a thread in flight before the first is converted and stored)
    for (int base = 0; base < lut_dwords; base += 8 * 256) {
        uint32_t w8[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) w8[u] = lut32[min(base + u * 256 + (int)threadIdx.x, lut_dwords - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + u * 256 + (int)threadIdx.x;
            const uint32_t w = w8[u];
            const float v0 = (float)(int16_t)(w & 0xffffu) - offset, v1 = (float)(int16_t)(w >> 16) - offset;
            const _Float16 h0 = (_Float16)v0, h1 = (_Float16)v1;
            if (i < lut_dwords) {
                inexact |= ((float)h0 != v0) | ((float)h1 != v1);
                s32[i] = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
            }
        }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (__builtin_amdgcn_ballot_w64(inexact) != 0 && lane == 0) atomicOr(&flags[2], 1u);
    __syncthreads();
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(smem);
    // a wave writes the 256 B row of one code: lane = (k % 4, column pair), one dword (two columns) per lane
    const int ks = lane >> 4, cp = lane & 15;
    const int n = blockIdx.x * kGaCols + 2 * cp;
    // the codes of B for all k quads of the workgroup first (one trip to memory instead of one per quad)
    constexpr int kMaxQuads = 4;
    uint16_t bpair[kMaxQuads];
#pragma unroll
    for (int pp = 0; pp < kMaxQuads; ++pp) {
        const int kq = min(blockIdx.y * quads_per_wg + min(pp, quads_per_wg - 1), K / 4 - 1);
        const uint8_t* bp = B + (size_t)(4 * kq + ks) * N + n;
        bpair[pp] = (uint16_t)((uint32_t)bp[0] | ((uint32_t)bp[1] << 8));
    }
#pragma unroll
    for (int pp = 0; pp < kMaxQuads; ++pp) {
        if (pp >= quads_per_wg) break;
        const int kq = blockIdx.y * quads_per_wg + pp;
        if (4 * kq >= K) break;
        const uint16_t* p0 = s16 + (int)(bpair[pp] & 0xffu);
        const uint16_t* p1 = s16 + (int)(bpair[pp] >> 8);
        uint32_t* chunk = S + ((size_t)blockIdx.x * (K / 4) + kq) * (kGaChunkBytes / 4) + lane;
#pragma unroll 8
        for (int a = wave; a < 128; a += 4) {
            // codes beyond the table (only the pad code 2^b of a narrower table can occur) read its all-zero pad row
            const int row = min(a, n_codes) * lut_cols;
            chunk[a * 64] = (uint32_t)p0[row] | ((uint32_t)p1[row] << 16);
        }
    }
}

// The same for a float32 table: S[n_tile][k / 4][a][k % 4][16 columns] float32, the entries themselves (no offset, nothing
// inexact).  grid (N / 16, ceil(K / 4 / quads_per_wg)), 256 threads, the table (rows x cols floats) in dynamic LDS.
__global__ __launch_bounds__(256) void expand_gradA_f32_kernel(const uint8_t* __restrict__ B, const float* __restrict__ lut,
                                                               int lut_entries, int lut_cols, int n_codes, uint32_t* __restrict__ S,
                                                               int K, int N, int quads_per_wg) {
    extern __shared__ __align__(16) unsigned char smem[];
    stage_table_dwords<256>(smem, lut, lut_entries);
    __syncthreads();
    const uint32_t* s32 = reinterpret_cast<const uint32_t*>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // a wave writes the 256 B row of one code: lane = (k % 4, column), one dword per lane
    const int ks = lane >> 4, col = lane & 15;
    const int n = blockIdx.x * kGaColsF32 + col;
    // (the codes of B for all k quads of the workgroup first)
    constexpr int kMaxQuads = 4;
    int bcode[kMaxQuads];
#pragma unroll
    for (int pp = 0; pp < kMaxQuads; ++pp) {
        const int kq = min(blockIdx.y * quads_per_wg + min(pp, quads_per_wg - 1), K / 4 - 1);
        bcode[pp] = (int)B[(size_t)(4 * kq + ks) * N + n];
    }
#pragma unroll
    for (int pp = 0; pp < kMaxQuads; ++pp) {
        if (pp >= quads_per_wg) break;
        const int kq = blockIdx.y * quads_per_wg + pp;
        if (4 * kq >= K) break;
        const uint32_t* p0 = s32 + bcode[pp];
        uint32_t* chunk = S + ((size_t)blockIdx.x * (K / 4) + kq) * (kGaChunkBytes / 4) + lane;
#pragma unroll 8
        for (int a = wave; a < 128; a += 4) chunk[a * 64] = p0[min(a, n_codes) * lut_cols];
    }
}

// The same for an 8-bit int16 table held as it is: S[n_tile][k / 4][a (256 rows)][k % 4][16 columns] int16, 32 KB per chunk
// (every entry exact whatever the table holds: no offset, no flag).  grid (N / 16, ceil(K / 4 / quads_per_wg)), 256
// threads, the table (rows x cols int16) in dynamic LDS.
constexpr int kGaI16MaxQuads = 8;
__global__ __launch_bounds__(256) void expand_gradA_i16_kernel(const uint8_t* __restrict__ B, const uint32_t* __restrict__ lut32,
                                                               int lut_dwords, int lut_cols, uint32_t* __restrict__ S, int K, int N,
                                                               int quads_per_wg) {
    extern __shared__ __align__(16) unsigned char smem[];
    stage_table_dwords<256>(smem, lut32, lut_dwords);
    __syncthreads();
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // a wave writes the 128 B rows of two consecutive codes: lane = (code % 2, k % 4, column pair), one dword per lane
    const int ap = lane >> 5, ks = (lane >> 3) & 3, cp = lane & 7;
    const int n = blockIdx.x * kGaColsF32 + 2 * cp;
    // (the codes of B for all k quads of the workgroup first)
    uint16_t bpair[kGaI16MaxQuads];
#pragma unroll
    for (int pp = 0; pp < kGaI16MaxQuads; ++pp) {
        const int kq = min(blockIdx.y * quads_per_wg + min(pp, quads_per_wg - 1), K / 4 - 1);
        const uint8_t* bp = B + (size_t)(4 * kq + ks) * N + n;
        bpair[pp] = (uint16_t)((uint32_t)bp[0] | ((uint32_t)bp[1] << 8));
    }
#pragma unroll
    for (int pp = 0; pp < kGaI16MaxQuads; ++pp) {
        if (pp >= quads_per_wg) break;
        const int kq = blockIdx.y * quads_per_wg + pp;
        if (4 * kq >= K) break;
        const uint16_t* p0 = s16 + (int)(bpair[pp] & 0xffu);
        const uint16_t* p1 = s16 + (int)(bpair[pp] >> 8);
        uint32_t* chunk = S + ((size_t)blockIdx.x * (K / 4) + kq) * (kGaChunkBytes / 4) + (lane & 31);
#pragma unroll 8
        for (int a2 = wave; a2 < 128; a2 += 4) {
            const int a = 2 * a2 + ap, row = a * lut_cols;
            chunk[a * 32] = (uint32_t)p0[row] | ((uint32_t)p1[row] << 16);
        }
    }
}

// The same for an 8-bit table of float32 entries: S[n_tile][k / 4][a (256 rows)][k % 4][8 columns] float32, 32 KB per chunk.
// The table (258 KB) does not fit the LDS: the entries are gathered from global memory (it stays in the L2; the expansion
// is 256 / M of the multiply-adds).  grid (N / 8, ceil(K / 4 / quads_per_wg)), 256 threads.
__global__ __launch_bounds__(256) void expand_gradA_f32w_kernel(const uint8_t* __restrict__ B, const float* __restrict__ lut, int lut_cols,
                                                                float* __restrict__ S, int K, int N, int quads_per_wg) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // a wave writes the 128 B rows of two consecutive codes: lane = (code % 2, k % 4, column), one float per lane
    const int ap = lane >> 5, ks = (lane >> 3) & 3, col = lane & 7;
    const int n = blockIdx.x * kGaColsF32W + col;
    for (int pp = 0; pp < quads_per_wg; ++pp) {
        const int kq = blockIdx.y * quads_per_wg + pp;
        if (4 * kq >= K) break;
        const float* p0 = lut + (int)B[(size_t)(4 * kq + ks) * N + n];
        float* chunk = S + ((size_t)blockIdx.x * (K / 4) + kq) * (kGaChunkBytes / 4) + (lane & 31);
#pragma unroll 8
        for (int a2 = wave; a2 < 128; a2 += 4) {
            const int a = 2 * a2 + ap;
            chunk[a * 32] = p0[a * lut_cols];
        }
    }
}

// ------------------------------------------------------------------------------------------ consume
// One 128-bit LDS read of a chunk, issued and NOT waited for.  The address comes out of ONE v_perm_b32:
// byte 0 = the lane's constant (window and piece), byte 1 = the code (BYTE of codeword; < 128), byte 2 = 1 for
// the third and fourth buffer (byte 3 of the lane's constant holds that 1), the odd buffers go into the offset field.
// Inline assembly: the compiler must not make these reads wait for the LDS-direct loads that fill the other
// buffers (same LDS array to it).
template <int BYTE, int BUF>
__device__ __forceinline__ void ga_read(u32x4& d, uint32_t codeword, uint32_t lane_const) {
    constexpr uint32_t sel = (BUF >= 2 ? 0x0c030000u : 0x0c020000u) | ((4u + BYTE) << 8);
    uint32_t addr;
    // (the address computation sits inside the volatile block so that it stays where it is used: computed ahead
    // of the loop, as the compiler would, the addresses of all reads of a workgroup occupy registers that do not exist)
    asm volatile("v_perm_b32 %1, %2, %3, %4\n ds_read_b128 %0, %1 offset:%5"
                 : "=v"(d), "=&v"(addr)
                 : "v"(codeword), "v"(lane_const), "s"(sel), "n"((BUF & 1) ? kGaChunkBytes : 0)
                 : "memory");
}

// The same for chunks of int16 entries of an 8-bit table: 256 rows of 128 B (window c 32 B, two pieces), four buffers of
// 32 KB.  v_perm_b32 assembles twice the address -- byte 0 = twice the lane's offset, byte 1 = the code, byte 2 = the
// buffer number (byte BUF of the lane's constant; none for buffer 0) -- and a shift halves it.
template <int BYTE, int BUF>
__device__ __forceinline__ void ga_read_i16(u32x4& d, uint32_t codeword, uint32_t lane_const) {
    constexpr uint32_t sel = 0x0c000000u | ((BUF == 0 ? 0x0cu : (uint32_t)BUF) << 16) | ((4u + BYTE) << 8);
    uint32_t addr;
    asm volatile("v_perm_b32 %1, %2, %3, %4\n v_lshrrev_b32 %1, 1, %1\n ds_read_b128 %0, %1"
                 : "=v"(d), "=&v"(addr)
                 : "v"(codeword), "v"(lane_const), "s"(sel)
                 : "memory");
}

// One piece (eight floats) of the two rows of gC a lane works on, from the staging area (the rows are 2 KB apart: 16 rows
// of 128 B): four 128-bit reads, NOT waited for ...
__device__ __forceinline__ void ga_issue_piece(u32x4 (&t)[4], uint32_t addr) {
    asm volatile("ds_read_b128 %0, %4\n ds_read_b128 %1, %4 offset:16\n ds_read_b128 %2, %4 offset:2048\n ds_read_b128 %3, %4 offset:2064"
                 : "=&v"(t[0]), "=&v"(t[1]), "=&v"(t[2]), "=&v"(t[3])
                 : "v"(addr)
                 : "memory");
}
// ... and, once they have landed, into piece S of the register copy of the rows.
template <int S, int COLS>
__device__ __forceinline__ void ga_take_piece(float (&g0)[COLS], float (&g1)[COLS], const u32x4 (&t)[4]) {
    static_assert(8 * S + 7 < COLS, "piece index");
    const f32x4 a0 = __builtin_bit_cast(f32x4, t[0]), a1 = __builtin_bit_cast(f32x4, t[1]);
    const f32x4 b0 = __builtin_bit_cast(f32x4, t[2]), b1 = __builtin_bit_cast(f32x4, t[3]);
    g0[8 * S] = a0.x; g0[8 * S + 1] = a0.y; g0[8 * S + 2] = a0.z; g0[8 * S + 3] = a0.w;
    g0[8 * S + 4] = a1.x; g0[8 * S + 5] = a1.y; g0[8 * S + 6] = a1.z; g0[8 * S + 7] = a1.w;
    g1[8 * S] = b0.x; g1[8 * S + 1] = b0.y; g1[8 * S + 2] = b0.z; g1[8 * S + 3] = b0.w;
    g1[8 * S + 4] = b1.x; g1[8 * S + 5] = b1.y; g1[8 * S + 6] = b1.z; g1[8 * S + 7] = b1.w;
}

// The value lane SRC of the quad holds, in all four lanes of the quad.
template <int SRC>
__device__ __forceinline__ uint32_t ga_quad_bcast(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, SRC * 0x55, 0xf, 0xf, true);
}
// Byte c of the four dwords lane SRC of the quad holds, in their order (pick = the v_perm_b32 selector of byte c of a pair
// of dwords): two v_perm_b32 pick it from pairs of dwords, a third joins them.
template <int SRC>
__device__ __forceinline__ uint32_t ga_codes_from(const u32x4& q, uint32_t pick) {
    const uint32_t x = ga_quad_bcast<SRC>(q.x), y = ga_quad_bcast<SRC>(q.y), z = ga_quad_bcast<SRC>(q.z), w = ga_quad_bcast<SRC>(q.w);
    const uint32_t lo = __builtin_amdgcn_perm(y, x, pick);     // {x.byte c, y.byte c, 0, 0}
    const uint32_t hi = __builtin_amdgcn_perm(w, z, pick);     // {z.byte c, w.byte c, 0, 0}
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// The results of a tile leave through LDS so that a store instruction covers whole 128 B lines (a lane's own results are
// single floats 16 B apart per row: stored directly, an instruction touches 16 lines in 16 B pieces and the stores of a
// tile, 64 KB, cost 2.8 us of its 18).  One float into LDS ...
__device__ __forceinline__ void ga_lds_put(uint32_t addr, float v) {
    asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
// ... N 16-byte pieces back (STEP bytes apart), waited for, ...
template <int N, int STEP>
__device__ __forceinline__ void ga_lds_get(u32x4 (&q)[N], uint32_t addr) {
    static_assert(N == 1 || N == 2, "one or two reads");
    if constexpr (N == 2)
        asm volatile("ds_read_b128 %0, %2\n ds_read_b128 %1, %2 offset:%3\n s_waitcnt lgkmcnt(0)"
                     : "=&v"(q[0]), "=&v"(q[1]) : "v"(addr), "n"(STEP) : "memory");
    else
        asm volatile("ds_read_b128 %0, %1\n s_waitcnt lgkmcnt(0)" : "=&v"(q[0]) : "v"(addr) : "memory");
}
// ... and to memory, not waited for.  (A store of more than 64 bits still reads its data registers for two cycles after
// it is issued; the compiler keeps its own stores apart from a following write to those registers but does not look into
// assembly blocks, so the two idle cycles are part of the block.)
__device__ __forceinline__ void ga_store16(float* p, const u32x4& q) {
    asm volatile("global_store_dwordx4 %0, %1, off\n s_nop 1" : : "v"(p), "v"(q) : "memory");
}

// grid: 8 * (workgroups per XCD, at most one per CU) workgroups of 1024 threads; every workgroup walks several tiles
// (512 rows x KT k) one after the other.  Requires N % 32 == 0, K % KT == 0, M >= 32, M*K < 2^31, gC 16-byte aligned.
// rows_per_image = 0: gA row-major [M,K]; L > 0: image-major transposed gA[m / L][k][m % L].
// F32: S holds float32 entries, 16 columns per tile (a 64 B window is 16 floats, a 128-bit read feeds four v_fma_f32 instead
// of eight v_fma_mix_f32); no offset.
//
// CONV (input gradient of a 3x3 convolution of stride 1 and padding 1, as one implicit GEMM): the rows are the B*H*W INPUT
// pixels, A holds their pixel-major codes [M][C] (K = C here), S the expanded table of the kh*kw*C rows of B in tap-major
// order, and a tile (512 pixels x KT channels) adds, tap after tap, the products with the rows of gC of the output
// positions that tap connects the pixel to: row m + (1 - ti) * W + (1 - tj), or a line of zeros where that position lies
// outside the image.  The sums over taps and columns stay in the accumulators, so neither the [M][9C] gradient matrix
// nor its col2im pass exists; gA receives [B][C][H*W] (rows_per_image = H*W).  A tile lasts nine times as many chunk steps.
// CONV only: what the store needs to finish the input gradient of the quantised layer on the spot,
//   gx = inside ? (tap sums + *zw * zt[pixel]) / *scale : 0     (zt == nullptr: the tap sums are stored as they are)
struct GaFinish {
    const float* zt;          // [B*H*W] window sums of the output gradient's row sums
    const float* zw;          // device scalars
    const float* scale;
    const uint8_t* inside;    // [B][C][H*W]
};

template <int kGaKT, int FMT, bool CONV = false>
__global__ __launch_bounds__(kGaWaves * 64) void lutgemm_gradA_slab_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const u32x4* __restrict__ S, float* __restrict__ gA,
    uint32_t* __restrict__ flags, int M, int K, int N, float scale, int rows_per_image, int row_blocks, int band_rows_max,
    int conv_h, int conv_w, const float* __restrict__ zero_line, GaFinish fin) {
    __shared__ __align__(16) unsigned char smem[kGaStageBase + kGaStageBytes];
    constexpr bool F32 = FMT == kGaFmtF32, I16 = FMT == kGaFmtI16, HALF = FMT == kGaFmtHalf, F32W = FMT == kGaFmtF32W;
    constexpr bool WIDE = !HALF;                           // 16 (8) columns per tile, four chunk buffers
    constexpr bool ROWS128 = I16 || F32W;                  // 8-bit tables: 256 code rows of 128 B per chunk
    constexpr int CH = kGaKT / kGaChunkK;                  // chunks per column tile
    // Chunk buffers: three, requested two chunks ahead; with float32 entries the staging area is half the size and a fourth
    // buffer fits: three chunks ahead (the loop is bound by the delivery of the chunks, 36 KB per 32 K multiply-adds).
    constexpr int BUFS = WIDE ? 4 : kGaBufs;
    constexpr int DIST = BUFS - 1;                         // chunks between a request and its use
    constexpr int OUT = 2 * (DIST - 1);                    // chunk operations issued after the request of the chunk a step needs
    constexpr int STAGE_BASE = BUFS * kGaChunkBytes;
    static_assert(STAGE_BASE + kGaRows * (F32W ? kGaColsF32W : WIDE ? kGaColsF32 : kGaCols) * 4 <= kGaStageBase + kGaStageBytes, "LDS budget");
    constexpr int NTU = (CH % BUFS) == 0 ? 1 : BUFS;       // column tiles per unrolled pass: the buffer of a chunk is then static
    static_assert(NTU == 1 || NTU == 3, "the tile loop below unrolls one or three column tiles");
    constexpr int NST = CH / 2;                            // 16-byte stores per lane at the end of a tile
    constexpr int COLS = F32W ? kGaColsF32W : WIDE ? kGaColsF32 : kGaCols;      // columns per tile
    constexpr int STAGE_WAVE = kGaRowsPerWave * COLS * 4;  // bytes of gC rows a wave stages per column tile (4 KB / 2 KB)
    constexpr int ROWOPS = STAGE_WAVE / 1024;              // wave-wide 16-byte loads of a row request (4 / 2)
    static_assert(CH >= 4, "the bookkeeping of outstanding loads assumes at least four chunks per column tile");
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int quad = lane >> 2, c = lane & 3;

    // Tile order: a band of row blocks, then all k groups, then the next band, so that the tiles in flight at one
    // time share their chunks (same k group) and their rows of gC (same row block) in the caches.  The hardware deals
    // workgroups to the 8 XCDs round-robin by index; the workgroups of one XCD (same index mod 8) walk ONE eighth of
    // that order together, so that they meet in one L2.  A workgroup keeps its CU for all its tiles: the loads of
    // the next tile are under way while the current one is finished (a fresh workgroup per tile spent 7 us, a third
    // of a tile of two column tiles, on start-up, first loads and drain).
    const int k_groups = K / kGaKT;
    const int total_tiles = row_blocks * k_groups;
    const int per_xcd = (total_tiles + 7) / 8;
    const int xcd = (int)(blockIdx.x % 8), pos_stride = (int)(gridDim.x / 8);
    // column tiles of a tile; CONV: (column tile of gC, tap) pairs, the nine taps of a column tile one after the other (their rows
    // of gC are the same lines of memory shifted by a pixel or an image row)
    constexpr int TAPS = CONV ? 9 : 1;
    const int n_tiles = (N / COLS) * TAPS;
    const int total = n_tiles * CH;                          // chunks of a tile: (column tile, four k)
    static_assert(!CONV || FMT == kGaFmtHalf, "the convolution-shaped walk is written for the half tables");
    if (HALF && flags[5] != 0u) return;                      // (set before this launch and never changed during it: every wave sees the same)
    const float offset = HALF ? (float)(int)flags[3] : 0.f;
    // 16-byte stores need gA aligned and, image-major, four consecutive rows in one image (same for every wave)
    const bool wide_stores = ((uintptr_t)gA & 15) == 0 && (rows_per_image & 3) == 0;
    struct Tile { int k0, m_wave; bool valid; };
    auto decode = [&](int pos) {
        Tile t;
        const int logical = xcd * per_xcd + pos;
        t.valid = pos < per_xcd && logical < total_tiles;
        const int lg = t.valid ? logical : 0;
        const int band = lg / (band_rows_max * k_groups);
        const int band_rows = min(band_rows_max, row_blocks - band_rows_max * band);
        const int in_band = lg - band * band_rows_max * k_groups;
        const int k_group = in_band / band_rows;
        const int row_block = band_rows_max * band + (in_band - k_group * band_rows);
        t.k0 = k_group * kGaKT;
        t.m_wave = row_block * kGaRows + wave * kGaRowsPerWave;
        return t;
    };
    int pos = (int)(blockIdx.x / 8);
    Tile cur = decode(pos);
    if (!cur.valid) return;
    Tile nxt = decode(pos + pos_stride);

    // per-lane address constants: window c, piece (quad + s) % 4 at step s; byte 3 = 1 (see ga_read)
    // (int16 entries: a code's row is 128 B, window c 32 B, two pieces; the constant holds TWICE the offset, the bytes 1, 2, 3
    // for the buffer number, and ga_read_i16 halves the assembled address)
    uint32_t lane_const[4];
#pragma unroll
    for (int s = 0; s < 4; ++s)
        lane_const[s] = ROWS128 ? ((uint32_t)(c << 6) | (uint32_t)(((quad + s) & 1) << 5) | 0x03020100u)
                            : ((uint32_t)(c << 6) | (uint32_t)(((quad + s) & 3) << 4) | 0x01000000u);

    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // A wave whose rows would stick out of M is shifted up so that all its rows exist; the rows it then shares with
    // the wave above are not stored twice (a wave entirely beyond M stores nothing but still takes part in the copies
    // and barriers).  Rows of a lane: m_base + 16 r + quad.
    auto m_base_of = [&](const Tile& t) { return min(t.m_wave, M - kGaRowsPerWave); };
    // chunk q of the current tile: 32 KB = 32 wave-wide 16-byte loads, two per wave; beyond the end: the first chunks
    // of the next tile (the last chunk again when there is none, into a buffer nobody reads any more), so that every
    // step issues the same number of operations
    auto request_chunk = [&](int q, int buf) {
        int k0 = cur.k0;
        if (q >= total) {
            if (nxt.valid) { q -= total; k0 = nxt.k0; } else q = total - 1;
        }
        int nt = q / CH;
        const int kc = q - nt * CH;
        int k_quads = K / kGaChunkK;
        if constexpr (CONV) {       // S covers the 9 C rows of B: tap-major, channel k0 of tap t is row t * C + k0
            const int ct = nt;
            nt = ct / TAPS;
            k0 += (ct - nt * TAPS) * K;
            k_quads *= TAPS;
        }
        const u32x4* src = S + ((size_t)nt * k_quads + k0 / kGaChunkK + kc) * (kGaChunkBytes / 16);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(src + (wave + kGaWaves * i) * 64 + lane),
                                             (lptr_t)(smem + buf * kGaChunkBytes + (wave + kGaWaves * i) * 1024), 16, 0, 0);
    };
    // the 32 rows of this wave, 128 B (32 columns of tile nt) each: four wave-wide loads, lane = (row % 8, 16 B piece)
    // (float32 entries: 64 B of 16 columns, two loads, lane = (row % 16, piece));
    // beyond the last column tile: the first one of the next tile
    constexpr int RPO = 64 * 16 / (COLS * 4);                // rows per wave-wide load (8 / 16)
    const uint32_t glane = (uint32_t)(lane / (64 / RPO)) * (uint32_t)N + 4u * (uint32_t)(lane % (64 / RPO));
    // CONV: which neighbours of a pixel exist, for the four rows this lane requests (row 8 i + lane / 8 of the wave): bits
    // 4 i .. 4 i + 3 = (row below exists, row above exists, pixel to the right exists, pixel to the left exists)
    auto conv_neighbours = [&](int m_base) {
        uint32_t vm = 0;
        if constexpr (CONV) {
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const float inv_l = 1.0f / (float)rows_per_image, inv_w = 1.0f / (float)conv_w;
#pragma unroll
            for (int i = 0; i < ROWOPS; ++i) {
                const int m = m_base + RPO * i + (ln >> 3);
                const int pix = m - div_small(m, rows_per_image, inv_l) * rows_per_image;
                const int y = div_small(pix, conv_w, inv_w), x = pix - y * conv_w;
                vm |= (uint32_t)((y + 1 < conv_h) | ((y >= 1) << 1) | ((x + 1 < conv_w) << 2) | ((x >= 1) << 3)) << (4 * i);
            }
        }
        return vm;
    };
    uint32_t neighbours = conv_neighbours(m_base_of(cur));
    auto request_rows = [&](int nt) {
        int m_base = m_base_of(cur);
        bool of_next = false;
        if (nt >= n_tiles) {
            if (nxt.valid) { nt = 0; m_base = m_base_of(nxt); of_next = true; } else nt = n_tiles - 1;
        }
        if constexpr (CONV) {
            const int ct = nt;
            nt = ct / TAPS;
            const int tap = ct - nt * TAPS;
            const int ti = tap / 3, tj = tap - 3 * ti;
            // the output position tap (ti, tj) connects pixel (y, x) to is (y + 1 - ti, x + 1 - tj)
            const int shift = (1 - ti) * conv_w + (1 - tj);
            const uint32_t need = (ti == 0 ? 1u : 0u) | (ti == 2 ? 2u : 0u) | (tj == 0 ? 4u : 0u) | (tj == 2 ? 8u : 0u);
            // (the first rows of the next tile: its neighbour bits are worked out here, once, and again when it becomes current)
            const uint32_t vm = of_next ? conv_neighbours(m_base) : neighbours;
            const float* base = gC + ((size_t)m_base + shift) * N + nt * COLS;     // (shift < 0 never reaches below the rows that exist: see `need`)
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const float* zero = zero_line + 4 * (ln & 7);
#pragma unroll
            for (int i = 0; i < ROWOPS; ++i) {
                const bool ok = ((vm >> (4 * i)) & need) == need;
                const float* p = ok ? base + (size_t)(RPO * i) * N + glane : zero;
                __builtin_amdgcn_global_load_lds((gptr_t)p, (lptr_t)(smem + STAGE_BASE + wave * STAGE_WAVE + i * 1024), 16, 0, 0);
            }
            return;
        }
        const float* base = gC + (size_t)m_base * N + nt * COLS;
#pragma unroll
        for (int i = 0; i < ROWOPS; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(base + (size_t)(RPO * i) * N + glane),
                                             (lptr_t)(smem + STAGE_BASE + wave * STAGE_WAVE + i * 1024), 16, 0, 0);
    };
    // The codes of a tile: A[m][k0 + 4 j + c], one byte per chunk and row, packed four to a register.  The 2 x kGaKT bytes of
    // the two rows of a quad are fetched once, 16 bytes per lane (lane c: 32 k per tile: row c / 2, codes 16 (c % 2) ...;
    // 16 k per tile: row c % 2), and dealt out inside the quad.  Assembly load: the waiting is explicit (the compiler would
    // wait for everything in flight).  The codes of the NEXT tile are asked for in the second step of the last column tile,
    // in front of the other requests of that step, and have landed at the wait of the third step (which lets only those
    // other requests be outstanding): their way from memory is hidden behind a step of arithmetic.
    uint32_t codes[2][CH / 4], codes_next[2][CH / 4];
    static_assert(CH == 4 || CH == 8, "one or two 16-byte pieces of codes per row");
    u32x4 craw = {0, 0, 0, 0};
    // (both derive what they need from the lane number afresh: kept from the start of the kernel, as the compiler would,
    // these values take registers the main loop does not have)
    auto request_codes = [&](const Tile& t) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int r = CH == 8 ? ((ln >> 1) & 1) : (ln & 1), h = CH == 8 ? (ln & 1) : 0;
        const uint8_t* p = A + (size_t)(m_base_of(t) + 16 * r + (ln >> 2)) * K + t.k0 + 16 * h;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(craw) : "v"(p) : "memory");
    };
    auto unpack_codes = [&]() {
        int ln = lane;
        asm volatile("" : "+v"(craw), "+v"(ln));
        const uint32_t pick = 0x0c0c0000u | (uint32_t)(ln & 3) | ((uint32_t)(4 + (ln & 3)) << 8);
        if constexpr (CH == 8) {
            codes_next[0][0] = ga_codes_from<0>(craw, pick);
            codes_next[0][1] = ga_codes_from<1>(craw, pick);
            codes_next[1][0] = ga_codes_from<2>(craw, pick);
            codes_next[1][1] = ga_codes_from<3>(craw, pick);
        } else {
            codes_next[0][0] = ga_codes_from<0>(craw, pick);
            codes_next[1][0] = ga_codes_from<1>(craw, pick);
        }
        uint32_t high_bits = 0;
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int w = 0; w < CH / 4; ++w) high_bits |= codes_next[r][w];
        // (a masked code 128 of a 7-bit operand; an 8-bit table has a row for every value of a byte)
        if (!ROWS128 && __builtin_amdgcn_ballot_w64((high_bits & 0x80808080u) != 0) != 0) {
            if (lane == 0) atomicOr(&flags[2], 1u);
        }
    };
    auto take_codes = [&]() {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int w = 0; w < CH / 4; ++w) codes[r][w] = codes_next[r][w];
    };

    float acc[2][CH];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < CH; ++j) acc[r][j] = 0.f;
    float g[2][COLS];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int i = 0; i < COLS; ++i) g[r][i] = 0.f;
    // sums of the lane's rows of gC over all columns (to undo a non-zero offset): formed during the first tile a workgroup
    // walks on a block of rows and kept while its next tiles stay on the same rows (with the order above, every other k group)
    float row_sum[2] = {0.f, 0.f};
    bool sum_rows = offset != 0.f;
    u32x4 d[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    u32x4 e[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};      // float32 entries: the second half of a chunk's reads

    // Operations of a wave towards memory, in issue order (vmcnt counts them in this order):
    //   rows(0) chunk(0) .. chunk(DIST - 1) codes | step q: chunk(q + DIST); second step of column tile nt:
    //   [last column tile: codes(next tile)] chunk(q + DIST) rows(nt + 1) | end of a tile: NST stores | ...
    // (a chunk request is two operations, a row request ROWOPS = four, two with float32 entries, the codes one).  At the top
    // of step q, chunk q (requested DIST steps earlier) must have landed: all but the requests of the steps in between may be
    // outstanding; in the first two steps of a tile the stores of the previous one as well.
    request_rows(0);
#pragma unroll
    for (int i = 0; i < DIST; ++i) request_chunk(i, i);
    request_codes(cur);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unpack_codes();
    take_codes();
    bool after_stores = false;     // the previous tile's stores may still be on their way (this wave issued all NST of them)

    // Read i of a chunk (i = 0..7): step s = i / 2, row r = i % 2; data in d[i % 4].  Two pairs of reads are in flight;
    // the last pair of a chunk is consumed after the barrier of the next one, while its first reads travel.  The two
    // rows of a pair have independent sums: their multiply-adds alternate, a dependent v_fma_mix_f32 issues only
    // every 9 clocks.
    auto pair_fma = [&](auto kc_tag, auto s_tag, const u32x4& d0, const u32x4& d1) {
        constexpr int KC = decltype(kc_tag)::value;
        float s0 = acc[0][KC], s1 = acc[1][KC];
        if constexpr (F32 || F32W) {
            constexpr int S4 = 4 * decltype(s_tag)::value;
            const f32x4 f0 = __builtin_bit_cast(f32x4, d0), f1 = __builtin_bit_cast(f32x4, d1);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s0 = __builtin_fmaf(g[0][S4 + e], f0[e], s0);
                s1 = __builtin_fmaf(g[1][S4 + e], f1[e], s1);
            }
        } else if constexpr (I16) {
            // (entries 2 q and 2 q + 1 are the halves of dword q; the conversion sign-extends the half it selects)
            constexpr int S8 = 8 * decltype(s_tag)::value;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                s0 = __builtin_fmaf(g[0][S8 + 2 * q], (float)(int16_t)(d0[q] & 0xffffu), s0);
                s1 = __builtin_fmaf(g[1][S8 + 2 * q], (float)(int16_t)(d1[q] & 0xffffu), s1);
                s0 = __builtin_fmaf(g[0][S8 + 2 * q + 1], (float)((int32_t)d0[q] >> 16), s0);
                s1 = __builtin_fmaf(g[1][S8 + 2 * q + 1], (float)((int32_t)d1[q] >> 16), s1);
            }
        } else {
            constexpr int S8 = 8 * decltype(s_tag)::value;
            const f16x8 h0 = __builtin_bit_cast(f16x8, d0), h1 = __builtin_bit_cast(f16x8, d1);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                s0 = __builtin_fmaf(g[0][S8 + e], (float)h0[e], s0);
                s1 = __builtin_fmaf(g[1][S8 + e], (float)h1[e], s1);
            }
        }
        // pin: the sums are finished before the next volatile read is issued (otherwise the compiler keeps the
        // results of several reads live and runs out of registers)
        asm volatile("" : "+v"(s0), "+v"(s1));
        acc[0][KC] = s0;
        acc[1][KC] = s1;
    };
    auto chunk_step = [&](int nt, auto kc_tag, auto buf_tag) __attribute__((always_inline)) {
        constexpr int KC = decltype(kc_tag)::value;
        constexpr int BUF = decltype(buf_tag)::value;
        constexpr int KP = (KC + CH - 1) % CH;            // the previous chunk's k quad (its last pair of reads is consumed here)
        const int q = nt * CH + KC;
        // the last pair of the previous chunk has landed (nobody reads its buffer any more), chunk q has landed for
        // this wave; behind the barrier: for every wave
        // (the wait for the reads in flight stands alone, ahead of the branch: where the blocks below tie the registers
        // of those reads as operands, the register allocator may copy them, i.e. read them, in front of the block)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (KC < 2 && nt == 0 && after_stores) {
            asm volatile("s_waitcnt vmcnt(%2)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : "n"(OUT + NST) : "memory");
        } else if (KC == 2) {
            // the youngest operations are the row request and the chunk request of step 1: codes asked for in front of
            // them have landed
            asm volatile("s_waitcnt vmcnt(%2)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : "n"(2 + ROWOPS) : "memory");
        } else if (KC >= 2 && KC <= DIST + 1) {
            // the row request of step 1 was issued after the request of the chunk this step needs
            asm volatile("s_waitcnt vmcnt(%2)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : "n"(OUT + ROWOPS) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(%2)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : "n"(OUT) : "memory");
        }
        if (KC == 1) {
            if (nt == n_tiles - 1) request_codes(nxt.valid ? nxt : cur);
            else asm volatile("" : "=v"(craw));      // (no value to keep: the registers are free in the other column tiles)
        }
        request_chunk(q + DIST, (BUF + DIST) % BUFS);
        if (KC == 1) request_rows(nt + 1);
        if constexpr (WIDE) {
            // float32 entries: a read feeds four multiply-adds only, so the loop is bound by the latency of the LDS, not by
            // arithmetic: all eight reads of the chunk are issued at once (the registers are there: 16 values of gC per row
            // instead of 32) and consumed in order; nothing is carried over the barrier.  int16 entries: four reads.
            if (KC == 0) {
                const uint32_t gbase = (uint32_t)(STAGE_BASE + wave * STAGE_WAVE + quad * (COLS * 4));
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    constexpr int NP = COLS / 4;             // 16-byte pieces of a row of the tile
                    u32x4 t[NP];
#pragma unroll
                    for (int s4 = 0; s4 < NP; ++s4) {
                        // the rows of gC in the order the entries are read in: 16-byte pieces (quad + s) % 4 of the window
                        // (int16 entries: 32-byte pieces (quad + s) % 2, i.e. floats 8 ((quad + s4 / 2) % 2) + 4 (s4 % 2) ...;
                        // float32 entries of an 8-bit table: 16-byte pieces (quad + s) % 2)
                        const uint32_t ga = gbase + (I16 ? (uint32_t)((((quad + (s4 >> 1)) & 1) << 5) | ((s4 & 1) << 4))
                                                         : (uint32_t)(((quad + s4) & (NP - 1)) << 4));
                        // (the second row of the lane is 16 rows further on)
                        if (r == 0) asm volatile("ds_read_b128 %0, %1" : "=&v"(t[s4]) : "v"(ga) : "memory");
                        else asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(t[s4]) : "v"(ga), "n"(16 * COLS * 4) : "memory");
                    }
                    if constexpr (NP == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]) : : "memory");
                    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(t[0]), "+v"(t[1]) : : "memory");
#pragma unroll
                    for (int i = 0; i < NP; ++i) {
                        const f32x4 v = __builtin_bit_cast(f32x4, t[i]);
                        g[r][4 * i] = v.x; g[r][4 * i + 1] = v.y; g[r][4 * i + 2] = v.z; g[r][4 * i + 3] = v.w;
                    }
                }
            }
            if constexpr (ROWS128) {
                ga_read_i16<KC & 3, BUF>(d[0], codes[0][KC >> 2], lane_const[0]);
                ga_read_i16<KC & 3, BUF>(d[1], codes[1][KC >> 2], lane_const[0]);
                ga_read_i16<KC & 3, BUF>(d[2], codes[0][KC >> 2], lane_const[1]);
                ga_read_i16<KC & 3, BUF>(d[3], codes[1][KC >> 2], lane_const[1]);
                asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(d[0]), "+v"(d[1]) : : "memory");
                pair_fma(kc_tag, std::integral_constant<int, 0>{}, d[0], d[1]);
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(d[2]), "+v"(d[3]) : : "memory");
                pair_fma(kc_tag, std::integral_constant<int, 1>{}, d[2], d[3]);
                return;
            }
            ga_read<KC & 3, BUF>(d[0], codes[0][KC >> 2], lane_const[0]);
            ga_read<KC & 3, BUF>(d[1], codes[1][KC >> 2], lane_const[0]);
            ga_read<KC & 3, BUF>(d[2], codes[0][KC >> 2], lane_const[1]);
            ga_read<KC & 3, BUF>(d[3], codes[1][KC >> 2], lane_const[1]);
            ga_read<KC & 3, BUF>(e[0], codes[0][KC >> 2], lane_const[2]);
            ga_read<KC & 3, BUF>(e[1], codes[1][KC >> 2], lane_const[2]);
            ga_read<KC & 3, BUF>(e[2], codes[0][KC >> 2], lane_const[3]);
            ga_read<KC & 3, BUF>(e[3], codes[1][KC >> 2], lane_const[3]);
            asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(d[0]), "+v"(d[1]) : : "memory");
            pair_fma(kc_tag, std::integral_constant<int, 0>{}, d[0], d[1]);
            asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(d[2]), "+v"(d[3]) : : "memory");
            pair_fma(kc_tag, std::integral_constant<int, 1>{}, d[2], d[3]);
            asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(e[0]), "+v"(e[1]) : : "memory");
            pair_fma(kc_tag, std::integral_constant<int, 2>{}, e[0], e[1]);
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(e[2]), "+v"(e[3]) : : "memory");
            pair_fma(kc_tag, std::integral_constant<int, 3>{}, e[2], e[3]);
            return;
        }
        __builtin_amdgcn_s_setprio(3);
        ga_read<KC & 3, BUF>(d[0], codes[0][KC >> 2], lane_const[0]);
        ga_read<KC & 3, BUF>(d[1], codes[1][KC >> 2], lane_const[0]);
        if (KC != 0 || nt != 0) pair_fma(std::integral_constant<int, KP>{}, std::integral_constant<int, 3>{}, d[2], d[3]);
        ga_read<KC & 3, BUF>(d[2], codes[0][KC >> 2], lane_const[1]);
        ga_read<KC & 3, BUF>(d[3], codes[1][KC >> 2], lane_const[1]);
        if constexpr (HALF && KC == 0) {
            // New column tile: the rows of gC come from the staging area, piece by piece in this lane's rotated order (piece
            // s = eight floats of both rows = four reads).  Only the first piece is waited for on the spot; the reads of
            // piece s + 1 travel while the multiply-adds of step s run.
            // (addresses from the lane number afresh, not kept in registers over the other steps)
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int quad = ln >> 2;
            const uint32_t gbase = (uint32_t)(STAGE_BASE + wave * STAGE_WAVE + quad * (COLS * 4));
            u32x4 t[4];
            ga_issue_piece(t, gbase + (uint32_t)(((quad + 0) & 3) << 5));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]) : : "memory");
            ga_take_piece<0>(g[0], g[1], t);
            ga_issue_piece(t, gbase + (uint32_t)(((quad + 1) & 3) << 5));
            __builtin_amdgcn_s_setprio(2);
            pair_fma(kc_tag, std::integral_constant<int, 0>{}, d[0], d[1]);
            ga_read<KC & 3, BUF>(d[0], codes[0][KC >> 2], lane_const[2]);
            ga_read<KC & 3, BUF>(d[1], codes[1][KC >> 2], lane_const[2]);
            asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]) : : "memory");
            ga_take_piece<1>(g[0], g[1], t);
            ga_issue_piece(t, gbase + (uint32_t)(((quad + 2) & 3) << 5));
            __builtin_amdgcn_s_setprio(1);
            pair_fma(kc_tag, std::integral_constant<int, 1>{}, d[2], d[3]);
            ga_read<KC & 3, BUF>(d[2], codes[0][KC >> 2], lane_const[3]);
            ga_read<KC & 3, BUF>(d[3], codes[1][KC >> 2], lane_const[3]);
            asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(d[0]), "+v"(d[1]) : : "memory");
            ga_take_piece<2>(g[0], g[1], t);
            ga_issue_piece(t, gbase + (uint32_t)(((quad + 3) & 3) << 5));
            __builtin_amdgcn_s_setprio(0);
            pair_fma(kc_tag, std::integral_constant<int, 2>{}, d[0], d[1]);
            // (the last pair of table reads of this chunk is consumed behind the next barrier, as in every step; here its
            // landing is waited for together with the last piece)
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(d[2]), "+v"(d[3]) : : "memory");
            ga_take_piece<3>(g[0], g[1], t);
            if (sum_rows) {
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    float sr = row_sum[r];
#pragma unroll
                    for (int i = 0; i < COLS; ++i) sr += g[r][i];
                    row_sum[r] = sr;
                }
            }
            return;
        }
        __builtin_amdgcn_s_setprio(2);
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(d[0]), "+v"(d[1]) : : "memory");
        pair_fma(kc_tag, std::integral_constant<int, 0>{}, d[0], d[1]);
        ga_read<KC & 3, BUF>(d[0], codes[0][KC >> 2], lane_const[2]);
        ga_read<KC & 3, BUF>(d[1], codes[1][KC >> 2], lane_const[2]);
        __builtin_amdgcn_s_setprio(1);
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(d[2]), "+v"(d[3]) : : "memory");
        pair_fma(kc_tag, std::integral_constant<int, 1>{}, d[2], d[3]);
        ga_read<KC & 3, BUF>(d[2], codes[0][KC >> 2], lane_const[3]);
        ga_read<KC & 3, BUF>(d[3], codes[1][KC >> 2], lane_const[3]);
        __builtin_amdgcn_s_setprio(0);
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(d[0]), "+v"(d[1]) : : "memory");
        pair_fma(kc_tag, std::integral_constant<int, 2>{}, d[0], d[1]);
    };
    // End of a tile: last multiply-adds, gA of the tile is stored; none of it is waited for.
    // FREE = the buffer of the tile's last chunk: once every wave has read it, it is free until the request of the next
    // step (issued behind that step's barrier); each wave turns its results round in 2 KB of it.
    // Returns false when the workgroup has no further tile.
    auto finish_tile = [&](auto free_tag) __attribute__((always_inline)) {
        constexpr int FREE = decltype(free_tag)::value;
        if constexpr (HALF) {
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(d[2]), "+v"(d[3]) : : "memory");
            pair_fma(std::integral_constant<int, CH - 1>{}, std::integral_constant<int, 3>{}, d[2], d[3]);
        }
        if (wide_stores) asm volatile("s_barrier" ::: "memory");   // (the reads of the last chunk have landed in every wave)
        const int m_base = m_base_of(cur);
        const bool whole = m_base == cur.m_wave;             // every lane of the wave stores
        const bool fast = whole && wide_stores;              // NST store instructions, no more, no less
        float corr[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) corr[r] = offset * row_sum[r];
        if (fast) {
            // (everything below is derived from the lane number afresh: computed ahead of the tile loop, as the compiler
            // would, these addresses take registers the main loop does not have)
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int quad = ln >> 2, c = ln & 3;
            const uint32_t tbase = (uint32_t)(FREE * kGaChunkBytes + wave * 2048);
            if (rows_per_image == 0) {
                // row-major: the 16 rows r of the quads at a time, [row][kGaKT k] floats; the 16 B group j of a row sits at
                // j ^ (row % CH) (the rows are a multiple of 64 B apart).  Back: lane = (row % (64 / CH), group): whole rows.
                constexpr int PITCH = kGaKT * 4, RPI = 64 / CH;       // bytes per row; rows per read instruction
                const uint32_t wr = tbase + (uint32_t)(quad * PITCH + c * 4);
                const int row = ln / CH, grp = ln % CH;
                const uint32_t rd = tbase + (uint32_t)(row * PITCH + ((grp ^ (row & (CH - 1))) << 4));
                // (row + RPI has the same low bits as row when RPI is a multiple of CH; with CH = 8, RPI = 8)
                static_assert(RPI % CH == 0 || CH / 4 == 1, "the second read of a lane keeps its group position");
                float* out = gA + (size_t)(m_base + row) * K + cur.k0 + 4 * grp;
#pragma unroll
                for (int r = 0; r < 2; ++r) {
#pragma unroll
                    for (int j = 0; j < CH; ++j)
                        ga_lds_put(wr + (uint32_t)((j ^ (quad & (CH - 1))) << 4), (acc[r][j] + corr[r]) * scale);
                    u32x4 q[CH / 4];
                    ga_lds_get<CH / 4, RPI * PITCH>(q, rd);
#pragma unroll
                    for (int i = 0; i < CH / 4; ++i) ga_store16(out + (size_t)(16 * r + RPI * i) * K, q[i]);
                }
            } else {
                // image-major: half of the k at a time, [k][32 rows] floats; the rows of k with k % 4 >= 2 swap their halves
                // (k and k + 2 are 256 B apart).  Back: lane = (k % 8, four consecutive rows): whole lines of gA[img][k][:].
                constexpr int KH = kGaKT / 2;
                const int kl0 = ln >> 3, pp = ln & 7;
                const uint32_t rd = tbase + (uint32_t)(kl0 * 128 + (((4 * pp) ^ (16 * ((kl0 >> 1) & 1))) << 2));
                const int m4 = m_base + 4 * pp;
                const int img = m4 / rows_per_image, l = m4 - img * rows_per_image;
                const size_t out_off = ((size_t)img * K + cur.k0 + kl0) * rows_per_image + l;
                float* out = gA + out_off;
                // (CONV with a finishing store: the host only asks for it where every wave takes this branch)
                const bool finish = CONV && fin.zt != nullptr;
                f32x4 zt4 = {0.f, 0.f, 0.f, 0.f};
                float inv_den = 1.f;
                if (finish) {
                    zt4 = *reinterpret_cast<const f32x4*>(fin.zt + m4);
                    const float zw = *fin.zw;
                    zt4 = zt4 * zw;
                    inv_den = *fin.scale;
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int r = 0; r < 2; ++r)
#pragma unroll
                        for (int jj = 0; jj < CH / 2; ++jj)
                            ga_lds_put(tbase + (uint32_t)((4 * jj + c) * 128 + (((16 * r + quad) ^ (16 * (c >> 1))) << 2)),
                                       (acc[r][h * (CH / 2) + jj] + corr[r]) * scale);
                    u32x4 q[CH / 4];
                    ga_lds_get<CH / 4, 8 * 128>(q, rd);
#pragma unroll
                    for (int i = 0; i < CH / 4; ++i) {
                        const size_t ko = (size_t)(h * KH + 8 * i) * rows_per_image;
                        if (finish) {
                            const uint32_t in4 = *reinterpret_cast<const uint32_t*>(fin.inside + out_off + ko);
                            f32x4 v = __builtin_bit_cast(f32x4, q[i]);
                            v = v + zt4;
                            v.x = (in4 & 0xffu) ? v.x / inv_den : 0.f;
                            v.y = (in4 & 0xff00u) ? v.y / inv_den : 0.f;
                            v.z = (in4 & 0xff0000u) ? v.z / inv_den : 0.f;
                            v.w = (in4 & 0xff000000u) ? v.w / inv_den : 0.f;
                            q[i] = __builtin_bit_cast(u32x4, v);
                        }
                        ga_store16(out + ko, q[i]);
                    }
                }
            }
        } else {
            // (k outside, row inside: the two stores of a k then fill the same 128 B lines of the image-major layout)
            float* o[2];
            size_t k_stride = 4;
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int m = m_base + 16 * r + quad;
                if (m < cur.m_wave) {
                    o[r] = nullptr;          // row stored by the wave above
                } else if (rows_per_image > 0) {
                    const int img = m / rows_per_image, l = m - img * rows_per_image;
                    o[r] = gA + ((size_t)img * K + cur.k0 + c) * rows_per_image + l;
                    k_stride = (size_t)4 * rows_per_image;
                } else {
                    o[r] = gA + (size_t)m * K + cur.k0 + c;
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < CH; ++j)
#pragma unroll
                for (int r = 0; r < 2; ++r)
                    if (o[r]) o[r][j * k_stride] = (acc[r][j] + corr[r]) * scale;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        if (!nxt.valid) return false;
        unpack_codes();            // (they arrived during the last column tile)
        take_codes();
        after_stores = fast;
        const bool same_rows = nxt.m_wave == cur.m_wave;
        sum_rows = offset != 0.f && !same_rows;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            if (!same_rows) row_sum[r] = 0.f;
#pragma unroll
            for (int j = 0; j < CH; ++j) acc[r][j] = 0.f;
        }
        cur = nxt;
        pos += pos_stride;
        nxt = decode(pos + pos_stride);
        if constexpr (CONV) neighbours = conv_neighbours(m_base_of(cur));
        return true;
    };
    int nt = 0;
    // one column tile; J = its position in the unrolled pass (the buffers rotate with period three across tiles)
    auto tile_step = [&](auto j_tag) __attribute__((always_inline)) {
        constexpr int J = decltype(j_tag)::value;
        [&]<int... KC>(std::integer_sequence<int, KC...>) {
            (chunk_step(nt, std::integral_constant<int, KC>{}, std::integral_constant<int, (J * CH + KC) % BUFS>{}), ...);
        }(std::make_integer_sequence<int, CH>{});
        if (++nt < n_tiles) return true;
        nt = 0;
        return finish_tile(std::integral_constant<int, (J * CH + CH - 1) % BUFS>{});
    };
    for (;;) {
        if (!tile_step(std::integral_constant<int, 0>{})) break;
        if (NTU > 1) {
            if (!tile_step(std::integral_constant<int, 1 % NTU>{})) break;
            if (!tile_step(std::integral_constant<int, 2 % NTU>{})) break;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing is left in flight towards LDS when the workgroup ends
}

// ------------------------------------------------------------------------------------------ host
hipError_t launch_gradA(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                        const LutGeom& g, int M, int K, int N, float scale, int n_cu, hipStream_t stream,
                        const uint32_t* gate, int rows_per_image);

// Bytes of the expanded table S, or 0 when the expanded-table gradA does not apply.
size_t gradA_slab_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    // (below the thresholds the expansion, 2^b / M of the work but all of it HBM writes plus two more launches, costs
    // more than it saves: measured cross-over on MI355X at about 1000 rows and 1e8 multiply-adds; with `force` only
    // what the kernel cannot do is excluded)
    if (!force && (M < 1024 || (double)M * K * N < 1e8)) return 0;
    if (g.bits > 7 || M < 512 || (N % kGaCols) != 0 || (K % 16) != 0 || (size_t)M * K >= (1ull << 31)) return 0;
    return (size_t)(N / kGaCols) * (K / kGaChunkK) * kGaChunkBytes;
}

hipError_t launch_gradA_slab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                             const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                             int rows_per_image, hipStream_t stream) {
    const int lut_dwords = g.rows * g.cols / 2;
    // 16 k per workgroup (measured: 8 k is 15 % slower for long K, 64 k 20 % slower); 4 k where that would leave most CUs idle
    const int qpw = (long)(N / kGaCols) * ((K / 4 + 3) / 4) >= n_cu ? 4 : 1;
    hipLaunchKernelGGL(expand_gradA_kernel, dim3(N / kGaCols, (K / 4 + qpw - 1) / qpw), dim3(256), (size_t)lut_dwords * 4, stream, B,
                       reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols, 1 << g.bits, reinterpret_cast<uint32_t*>(S),
                       flags, K, N, qpw);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (((uintptr_t)gC & 15) != 0) return hipErrorInvalidValue;   // callers check: rows of gC are fetched 16 bytes at a time
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const int row_blocks = (M + kGaRows - 1) / kGaRows;
    // 16 row blocks x 2 k groups are in flight on an XCD at a time (measured: 8 to 32 row blocks make no difference)
    const int band_rows = 16;
    // (48 k per workgroup would need more registers than a wave of a 1024-thread workgroup has)
    // (fewer tiles than CUs: 16 k per tile, twice the tiles)
    const int kt = ((K % 32) == 0 && row_blocks * (K / 32) >= n_cu) ? 32 : 16;
    const int tiles = row_blocks * (K / kt);
    const int per_xcd = (tiles + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    const dim3 grid(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd));
    if (kt == 32)
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<32, kGaFmtHalf>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    else
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<16, kGaFmtHalf>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // masked codes in A or table entries a half cannot hold: the gated direct kernel recomputes gA
    return launch_gradA(gC, A, B, gA, lut, g, M, K, N, scale, n_cu, stream, flags + 2, rows_per_image);
}

// ------------------------------------------------------------------------------------------ convolution-shaped gradA
// Input gradient of a 3x3 / stride 1 / padding 1 convolution as one implicit GEMM over the B*H*W input pixels (see CONV
// above).  codes [B*H*W][C] pixel-major, Bt [9*C][N] tap-major, g_in [B][C][H*W].  Same conditions on the table as the
// GEMM-shaped kernel (flags[5] set by bwd_header_kernel: the kernel returns at once; a masked code or an entry a half
// cannot hold raises flags[2]); what the caller queues behind for those cases is its business.
bool gradA_slab_conv_applies(const LutGeom& g, long M, int C, int N, const float* gC, bool force) {
    if (!force && (M < 1024 || (double)M * C * 9 * N < 1e8)) return false;
    return g.bits <= 7 && M >= 512 && (N % kGaCols) == 0 && (C % 16) == 0 && (size_t)M * C < (1ull << 31) && M < (1L << 23) &&
           ((uintptr_t)gC & 15) == 0;
}
size_t gradA_slab_conv_workspace_bytes(int C, int N) { return (size_t)(N / kGaCols) * (9 * C / kGaChunkK) * kGaChunkBytes; }

// Whether the kernel's store can finish the gradient (mask, zero-point term, quantiser scale) for this geometry: every
// wave must take the branch of 16-byte image-major stores.
bool gradA_slab_conv_can_finish(int Bn, int H, int W, const float* g_in) {
    return ((long)Bn * H * W) % kGaRowsPerWave == 0 && ((H * W) & 3) == 0 && ((uintptr_t)g_in & 15) == 0;
}

hipError_t launch_gradA_slab_conv(const float* gC, const uint8_t* codes, const uint8_t* Bt, float* g_in, const int16_t* lut,
                                  const LutGeom& g, int Bn, int C, int H, int W, int N, float scale, int n_cu, uint32_t* flags,
                                  void* S, const float* zero_line, hipStream_t stream, const float* zt, const float* zw,
                                  const float* qscale, const uint8_t* inside, int expanded) {
    const GaFinish fin{zt, zw, qscale, inside};
    const int lut_dwords = g.rows * g.cols / 2;
    const int K = 9 * C, M = Bn * H * W;
    const int qpw = (long)(N / kGaCols) * ((K / 4 + 3) / 4) >= n_cu ? 4 : 1;
    // (expanded: S already holds the expansion of this Bt and table -- a caller's cache; the offset in flags[3] is a function of
    // the table alone, so the header of this call agrees with what the cached entries were built with)
    if (!expanded)
        hipLaunchKernelGGL(expand_gradA_kernel, dim3(N / kGaCols, (K / 4 + qpw - 1) / qpw), dim3(256), (size_t)lut_dwords * 4, stream, Bt,
                           reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols, 1 << g.bits, reinterpret_cast<uint32_t*>(S),
                           flags, K, N, qpw);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const int row_blocks = (M + kGaRows - 1) / kGaRows;
    const int band_rows = 16;
    const int kt = ((C % 32) == 0 && row_blocks * (C / 32) >= n_cu) ? 32 : 16;
    const int tiles = row_blocks * (C / kt);
    const int per_xcd = (tiles + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    const dim3 grid(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd));
    if (kt == 32)
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<32, kGaFmtHalf, true>), grid, block, 0, stream, gC, codes, S4, g_in, flags, M, C, N,
                           scale, H * W, row_blocks, band_rows, H, W, zero_line, fin);
    else
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<16, kGaFmtHalf, true>), grid, block, 0, stream, gC, codes, S4, g_in, flags, M, C, N,
                           scale, H * W, row_blocks, band_rows, H, W, zero_line, fin);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ 8-bit tables
// Bytes of the int16 expanded table of an 8-bit gradient table, or 0 when that kernel does not apply.  It is twice the size
// of the half one of a 7-bit table (256 code rows); every block of 512 rows streams all of it.
// (measured on MI355X against the direct kernel: 1.6-1.9 x faster from 8192 rows on, 1.3 x at 2048 rows, 0.65 x at 512)
size_t gradA_slab_i16_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    if (!force && (M < 2048 || (double)M * K * N < 2e8)) return 0;
    if (g.bits != 8 || M < 512 || (N % kGaColsF32) != 0 || (K % 16) != 0 || (size_t)M * K >= (1ull << 31)) return 0;
    return (size_t)(N / kGaColsF32) * (K / kGaChunkK) * kGaChunkBytes;
}

// No flag is read or written: 8-bit operands have no masked code and every int16 entry is held exactly.
hipError_t launch_gradA_slab_i16(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                                 const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                                 int rows_per_image, hipStream_t stream) {
    if (((uintptr_t)gC & 15) != 0) return hipErrorInvalidValue;   // callers check: rows of gC are fetched 16 bytes at a time
    const int lut_dwords = g.rows * g.cols / 2;
    static std::atomic<uint64_t> attr_done{0};
    if (hipError_t ea = allow_full_lds(reinterpret_cast<const void*>(expand_gradA_i16_kernel), attr_done); ea != hipSuccess) return ea;
    // every workgroup copies the table (130 KB) into its LDS: as many chunks per workgroup as still leave one workgroup per CU
    const long chunks = (long)(N / kGaColsF32) * (K / 4);
    long qpw = chunks / (n_cu > 0 ? n_cu : 1);
    qpw = qpw < 1 ? 1 : (qpw > kGaI16MaxQuads ? kGaI16MaxQuads : qpw);
    hipLaunchKernelGGL(expand_gradA_i16_kernel, dim3(N / kGaColsF32, (unsigned)((K / 4 + qpw - 1) / qpw)), dim3(256),
                       (size_t)lut_dwords * 4, stream, B, reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols,
                       reinterpret_cast<uint32_t*>(S), K, N, (int)qpw);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const int row_blocks = (M + kGaRows - 1) / kGaRows;
    const int band_rows = 16;
    const int kt = ((K % 32) == 0 && row_blocks * (K / 32) >= n_cu) ? 32 : 16;
    const int tiles = row_blocks * (K / kt);
    const int per_xcd = (tiles + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    const dim3 grid(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd));
    if (kt == 32)
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<32, kGaFmtI16>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    else
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<16, kGaFmtI16>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ 8-bit float32 tables
// Bytes of the float32 expanded table of an 8-bit float table, or 0 when that kernel does not apply: K*N*1 KB, four times the
// half table of a 7-bit one, and every block of 512 rows streams all of it: from 16384 rows on (measured on MI355X:
// 3 x the two-band direct kernel at 32768 rows; up to 8192 rows the kernel that expands the table in LDS is faster).
size_t gradA_slab_f32w_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    if (!force && (M < 16384 || (double)M * K * N < 2e8)) return 0;
    if (g.bits != 8 || M < 512 || (N % kGaColsF32W) != 0 || (K % 16) != 0 || (size_t)M * K >= (1ull << 31)) return 0;
    return (size_t)(N / kGaColsF32W) * (K / kGaChunkK) * kGaChunkBytes;
}

// No flag is read or written (8-bit operands have no masked code).
hipError_t launch_gradA_slab_f32w(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                                  const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                                  int rows_per_image, hipStream_t stream) {
    if (((uintptr_t)gC & 15) != 0) return hipErrorInvalidValue;   // callers check: rows of gC are fetched 16 bytes at a time
    const int qpw = 4;
    hipLaunchKernelGGL(expand_gradA_f32w_kernel, dim3(N / kGaColsF32W, (K / 4 + qpw - 1) / qpw), dim3(256), 0, stream, B, lut, g.cols,
                       reinterpret_cast<float*>(S), K, N, qpw);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const int row_blocks = (M + kGaRows - 1) / kGaRows;
    const int band_rows = 16;
    const int kt = ((K % 32) == 0 && row_blocks * (K / 32) >= n_cu) ? 32 : 16;
    const int tiles = row_blocks * (K / kt);
    const int per_xcd = (tiles + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    const dim3 grid(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd));
    if (kt == 32)
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<32, kGaFmtF32W>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    else
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<16, kGaFmtF32W>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------ float32 tables
hipError_t launch_gradA_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut, const LutGeom& g,
                               int M, int K, int N, float scale, int n_cu, hipStream_t stream, const uint32_t* gate,
                               int rows_per_image);

// Bytes of the float32 expanded table, or 0 when that kernel does not apply.  It is twice the size of the half one and
// every block of 512 rows streams all of it, so it pays for fewer shapes: with 4096 rows and K*N = 4608 x 512 the
// table alone is 1.2 GB.
size_t gradA_slab_f32_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    if (!force && (M < 4096 || (double)M * K * N < 2e8)) return 0;
    if (g.bits > 7 || M < 512 || (N % kGaColsF32) != 0 || (K % 16) != 0 || (size_t)M * K >= (1ull << 31)) return 0;
    return (size_t)(N / kGaColsF32) * (K / kGaChunkK) * kGaChunkBytes;
}

// flags[2] must be zero on entry (masked codes in A raise it; the gated direct kernel then recomputes gA).
hipError_t launch_gradA_slab_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                                    const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                                    int rows_per_image, hipStream_t stream) {
    if (((uintptr_t)gC & 15) != 0) return hipErrorInvalidValue;   // callers check: rows of gC are fetched 16 bytes at a time
    const int lut_entries = g.rows * g.cols;
    static std::atomic<uint64_t> attr_done{0};
    if (hipError_t ea = allow_full_lds(reinterpret_cast<const void*>(expand_gradA_f32_kernel), attr_done); ea != hipSuccess) return ea;
    const int qpw = 4;
    hipLaunchKernelGGL(expand_gradA_f32_kernel, dim3(N / kGaColsF32, (K / 4 + qpw - 1) / qpw), dim3(256), (size_t)lut_entries * 4,
                       stream, B, lut, lut_entries, g.cols, 1 << g.bits, reinterpret_cast<uint32_t*>(S), K, N, qpw);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const int row_blocks = (M + kGaRows - 1) / kGaRows;
    const int band_rows = 16;
    const int kt = ((K % 32) == 0 && row_blocks * (K / 32) >= n_cu) ? 32 : 16;
    const int tiles = row_blocks * (K / kt);
    const int per_xcd = (tiles + 7) / 8, cus_per_xcd = n_cu >= 8 ? n_cu / 8 : 1;
    const dim3 grid(8 * (per_xcd < cus_per_xcd ? per_xcd : cus_per_xcd));
    if (kt == 32)
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<32, kGaFmtF32>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    else
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<16, kGaFmtF32>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, 0, 0, (const float*)nullptr, GaFinish{});
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_gradA_f32tab(gC, A, B, gA, lut, g, M, K, N, scale, n_cu, stream, flags + 2, rows_per_image);
}

}  // namespace amr
