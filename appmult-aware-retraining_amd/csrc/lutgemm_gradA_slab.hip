// Backward LUT-GEMM, gradient of A, for large M on gfx950: "expanded-table" kernel (7-bit tables and
// narrower).
//
// Same result (to fp32 summation order) as lutgemm_gradA_kernel and as the reference's
// ApproxGemmBackwardKernelForGA (self_ops/src/approx_gemm_backward.cu:44-267):
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
// entries in [-1024, 3072]; the expansion picks the offset from the extremes of the table and leaves it in
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
// all column tiles.  The chunks go from L2 to LDS by LDS-direct loads, three buffers, requested two chunks ahead
// by waves 0-7; the rows of gC take the same road (64 KB staging area, requested a column tile ahead by waves
// 8-15), so no load of the main loop has a register destination and all waiting is explicit.
// Measured on MI355X: no LDS bank-conflict cycles (4.0 LDS clocks per 128-bit read); about 1.0 us per chunk and
// CU against 0.5 us of v_fma_mix_f32 issue (72 VALU instructions per wave and chunk, 4.25 clocks each, four waves
// per SIMD); without the LDS-direct loads of the loop 0.8 us.
#include <type_traits>

#include "amr_common.h"

namespace amr {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kGaCols = 32;                               // columns per tile
constexpr int kGaChunkK = 4;
constexpr int kGaChunkBytes = 128 * kGaChunkK * 2 * kGaCols;   // 32 KB
constexpr int kGaBufs = 3;
constexpr int kGaWaves = 16;
constexpr int kGaRowsPerWave = 32;                        // 16 quads x 2 rows
constexpr int kGaRows = kGaWaves * kGaRowsPerWave;        // 512 rows per workgroup
constexpr int kGaStageBase = kGaBufs * kGaChunkBytes;     // 96 KB: the rows of gC of one column tile, 128 B per row
constexpr int kGaStageBytes = kGaRows * kGaCols * 4;      // 64 KB
static_assert(kGaStageBase + kGaStageBytes == 160 * 1024, "the workgroup uses the whole LDS of a CU");

// ------------------------------------------------------------------------------------------ expand
// grid (n_tiles, K / 8), 256 threads.  Requires N % 32 == 0 and K % 8 == 0.
constexpr int kGaExpandK = 8;

__global__ __launch_bounds__(256) void expand_gradA_kernel(const uint8_t* __restrict__ B, const uint32_t* __restrict__ lut32,
                                                           int lut_dwords, int lut_cols, int n_codes,
                                                           uint32_t* __restrict__ S, uint32_t* __restrict__ flags, int K, int N) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int extremes[2];
    uint32_t* s32 = reinterpret_cast<uint32_t*>(smem);
    if (threadIdx.x == 0) { extremes[0] = 0; extremes[1] = 0; }
    __syncthreads();
    int lo = 0, hi = 0;
    for (int i = threadIdx.x; i < lut_dwords; i += 256) {
        const uint32_t w = lut32[i];
        s32[i] = w;
        const int v0 = (int)(int16_t)(w & 0xffffu), v1 = (int)(int16_t)(w >> 16);
        lo = min(lo, min(v0, v1));
        hi = max(hi, max(v0, v1));
    }
    atomicMin(&extremes[0], lo);
    atomicMax(&extremes[1], hi);
    __syncthreads();
    // every workgroup finds the same offset; the consumer reads it from flags[3]
    const float offset = (extremes[0] >= -2048 && extremes[1] <= 2048) ? 0.f : 1024.f;
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) flags[3] = (uint32_t)offset;
    const int16_t* s16 = reinterpret_cast<const int16_t*>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // a wave writes the 256 B row of one code: lane = (k % 4, column pair), one dword (two columns) per lane
    const int ks = lane >> 4, cp = lane & 15;
    const int n = blockIdx.x * kGaCols + 2 * cp;
    bool inexact = false;
    for (int pp = 0; pp < kGaExpandK / 4; ++pp) {
        const int kq = blockIdx.y * (kGaExpandK / 4) + pp;
        const int k = 4 * kq + ks;
        const int b0 = (int)B[(size_t)k * N + n], b1 = (int)B[(size_t)k * N + n + 1];
        uint32_t* chunk = S + ((size_t)blockIdx.x * (K / 4) + kq) * (kGaChunkBytes / 4);
        for (int a = wave; a < 128; a += 4) {
            // codes beyond the table (only the pad code 2^b of a narrower table can occur) contribute zero
            const float v0 = (a < n_codes) ? (float)s16[a * lut_cols + b0] : 0.f;
            const float v1 = (a < n_codes) ? (float)s16[a * lut_cols + b1] : 0.f;
            const _Float16 h0 = (_Float16)(v0 - offset), h1 = (_Float16)(v1 - offset);
            inexact |= ((float)h0 != v0 - offset) | ((float)h1 != v1 - offset);
            const uint32_t w = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
            chunk[a * 64 + ks * 16 + cp] = w;
        }
    }
    if (__builtin_amdgcn_ballot_w64(inexact) != 0 && lane == 0) atomicOr(&flags[2], 1u);
}

// ------------------------------------------------------------------------------------------ consume
// One 128-bit LDS read of a chunk, issued and NOT waited for.  The address comes out of ONE v_perm_b32:
// byte 0 = the lane's constant (window and piece), byte 1 = the code (BYTE of codeword; < 128), byte 2 = 1 for
// the third buffer (byte 3 of the lane's constant holds that 1), the second buffer goes into the offset field.
// Inline assembly: the compiler must not make these reads wait for the LDS-direct loads that fill the other
// buffers (same LDS array to it).
template <int BYTE, int BUF>
__device__ __forceinline__ void ga_read(u32x4& d, uint32_t codeword, uint32_t lane_const) {
    constexpr uint32_t sel = (BUF == 2 ? 0x0c030000u : 0x0c020000u) | ((4u + BYTE) << 8);
    uint32_t addr;
    // (the address computation sits inside the volatile block so that it stays where it is used: computed ahead
    // of the loop, as the compiler would, the addresses of all reads of a workgroup occupy registers that do not exist)
    asm volatile("v_perm_b32 %1, %2, %3, %4\n ds_read_b128 %0, %1 offset:%5"
                 : "=v"(d), "=&v"(addr)
                 : "v"(codeword), "v"(lane_const), "s"(sel), "n"(BUF == 1 ? kGaChunkBytes : 0)
                 : "memory");
}

// grid: row_blocks * K / KT workgroups (rounded up to a multiple of 8), 1024 threads.  Requires N % 32 == 0,
// K % KT == 0, M*K < 2^31, gC 16-byte aligned.
// rows_per_image = 0: gA row-major [M,K]; L > 0: image-major transposed gA[m / L][k][m % L].
template <int kGaKT>
__global__ __launch_bounds__(kGaWaves * 64) void lutgemm_gradA_slab_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const u32x4* __restrict__ S, float* __restrict__ gA,
    uint32_t* __restrict__ flags, int M, int K, int N, float scale, int rows_per_image, int row_blocks, int band_rows_max,
    int xcd_order) {
    __shared__ __align__(16) unsigned char smem[kGaStageBase + kGaStageBytes];
    constexpr int CH = kGaKT / kGaChunkK;                  // chunks per column tile
    constexpr int NTU = (CH % kGaBufs) == 0 ? 1 : kGaBufs; // column tiles per unrolled pass: the buffer of a chunk is then static
    static_assert(CH >= 4, "the bookkeeping of outstanding loads assumes at least four chunks per column tile");
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int quad = lane >> 2, c = lane & 3;

    // Workgroup order: a band of row blocks, then all k groups, then the next band, so that the workgroups in
    // flight at one time share their chunks (same k group) and their rows of gC (same row block) in the caches.
    // The hardware deals workgroups to the 8 XCDs round-robin by index; with xcd_order the workgroups of one XCD
    // (same index mod 8) take consecutive positions of that order, so that they meet in ONE L2.
    const int k_groups = K / kGaKT;
    const int total_wgs = row_blocks * k_groups;
    const int per_xcd = (total_wgs + 7) / 8;
    const int logical = xcd_order ? (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8) : (int)blockIdx.x;
    if (logical >= total_wgs) return;
    const int band = logical / (band_rows_max * k_groups);
    const int band_rows = min(band_rows_max, row_blocks - band_rows_max * band);
    const int in_band = logical - band * band_rows_max * k_groups;
    const int k_group = in_band / band_rows;
    const int row_block = band_rows_max * band + (in_band - k_group * band_rows);
    const int m_wave = row_block * kGaRows + wave * kGaRowsPerWave;
    const int k0 = k_group * kGaKT;
    const int n_tiles = N / kGaCols;
    const int total = n_tiles * CH;                          // chunks this workgroup walks: (tile, four k)
    const float offset = (float)flags[3];

    // Rows of this lane: m_wave + 16 r + quad (clamped for the loads; rows beyond M are not stored).
    // per-lane address constants: window c, piece (quad + s) % 4 at step s; byte 3 = 1 (see ga_read)
    uint32_t lane_const[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) lane_const[s] = (uint32_t)(c << 6) | (uint32_t)(((quad + s) & 3) << 4) | 0x01000000u;

    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // The waves share the requests by kind, since vmcnt counts the operations of a wave in issue order and a slow one
    // holds up the count for every later one: waves 0-7 fetch the chunks (needed two steps later, from L2), waves
    // 8-15 the rows of gC (from HBM, needed a whole column tile later).
    const bool chunk_wave = wave < kGaWaves / 2;
    // chunk q = (tile, four k of the workgroup's range): 32 KB = 32 wave-wide 16-byte loads, four per wave.
    // Requests beyond the end repeat the last chunk (into a buffer nobody reads any more) so that every step
    // issues the same number of operations.
    const u32x4* Sgroup = S + (size_t)(k0 / kGaChunkK) * (kGaChunkBytes / 16);
    auto request_chunk = [&](int q, int buf) {
        if (!chunk_wave) return;
        q = min(q, total - 1);
        const int nt = q / CH, kc = q - nt * CH;
        const u32x4* src = Sgroup + ((size_t)nt * (K / kGaChunkK) + kc) * (kGaChunkBytes / 16);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(src + (wave + 8 * i) * 64 + lane),
                                             (lptr_t)(smem + buf * kGaChunkBytes + (wave + 8 * i) * 1024), 16, 0, 0);
    };
    // the 512 rows of the workgroup, 128 B (32 columns of tile nt) each: 64 wave-wide loads of 8 rows, eight per wave,
    // lane = (row % 8, 16 B piece); rows beyond M repeat the last one
    int grow = row_block * kGaRows + (wave & 7) * 64 + (lane >> 3);
    auto request_rows = [&](int nt) {
        if (chunk_wave) return;
        nt = min(nt, n_tiles - 1);
        // (opaque to the compiler: the eight offsets are computed here, once per column tile, not kept in registers)
        asm volatile("" : "+v"(grow));
        const float* base = gC + nt * kGaCols + 4 * (lane & 7);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(base + (size_t)((uint32_t)min(grow + 8 * i, M - 1) * (uint32_t)N)),
                                             (lptr_t)(smem + kGaStageBase + ((wave & 7) * 8 + i) * 1024), 16, 0, 0);
    };

    float acc[2][CH];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < CH; ++j) acc[r][j] = 0.f;
    float g[2][kGaCols];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int i = 0; i < kGaCols; ++i) g[r][i] = 0.f;
    float row_sum[2] = {0.f, 0.f};
    u32x4 d[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};

    // Operations of a thread towards LDS, in issue order (vmcnt counts them in this order):
    //   rows(0) chunk(0) chunk(1) | top of chunk q: chunk(q + 2); top of the second chunk of tile nt also: rows(nt + 1)
    // (a chunk request is two operations, a row request four).  At the top of chunk q, chunk q (requested two
    // chunks earlier) must have landed: all but the requests of the previous top may be outstanding.
    request_rows(0);
    request_chunk(0, 0);
    request_chunk(1, 1);
    // (the codes after the first requests: both then travel at the same time)
    uint32_t codes[2][(CH + 3) / 4];
    uint32_t high_bits = 0;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint8_t* arow = A + (size_t)min(m_wave + 16 * r + quad, M - 1) * K + k0;
#pragma unroll
        for (int w = 0; w < (CH + 3) / 4; ++w) codes[r][w] = 0;
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const uint32_t a = (load_u32_unaligned(arow + 4 * j) >> (8 * c)) & 0xffu;      // A[m][k0 + 4 j + c]
            high_bits |= a;
            codes[r][j >> 2] |= a << (8 * (j & 3));
        }
    }
    if (__builtin_amdgcn_ballot_w64((high_bits & 0x80u) != 0) != 0) {
        if (lane == 0) atomicOr(&flags[2], 1u);
    }


    // Read i of a chunk (i = 0..7): step s = i / 2, row r = i % 2; data in d[i % 4].  Two pairs of reads are in flight;
    // the last pair of a chunk is consumed after the barrier of the next one, while its first reads travel.  The two
    // rows of a pair have independent sums: their multiply-adds alternate, a dependent v_fma_mix_f32 issues only
    // every 9 clocks.
    auto pair_fma = [&](auto kc_tag, auto s_tag, const u32x4& d0, const u32x4& d1) {
        constexpr int KC = decltype(kc_tag)::value;
        constexpr int S8 = 8 * decltype(s_tag)::value;
        const f16x8 h0 = __builtin_bit_cast(f16x8, d0), h1 = __builtin_bit_cast(f16x8, d1);
        float s0 = acc[0][KC], s1 = acc[1][KC];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            s0 = __builtin_fmaf(g[0][S8 + e], (float)h0[e], s0);
            s1 = __builtin_fmaf(g[1][S8 + e], (float)h1[e], s1);
        }
        // pin: the sums are finished before the next volatile read is issued (otherwise the compiler keeps the
        // results of several reads live and runs out of registers)
        asm volatile("" : "+v"(s0), "+v"(s1));
        acc[0][KC] = s0;
        acc[1][KC] = s1;
    };
    auto chunk_step = [&](int nt, auto kc_tag, auto buf_tag) {
        constexpr int KC = decltype(kc_tag)::value;
        constexpr int BUF = decltype(buf_tag)::value;
        constexpr int KP = (KC + CH - 1) % CH;            // the previous chunk's k quad (its last pair of reads is consumed here)
        const int q = nt * CH + KC;
        // the last pair of the previous chunk has landed (nobody reads its buffer any more), chunk q has landed for
        // this wave; behind the barrier: for every wave
        if (chunk_wave)
            asm volatile("s_waitcnt lgkmcnt(0)\n s_waitcnt vmcnt(4)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : : "memory");
        else if (KC == 0)
            asm volatile("s_waitcnt lgkmcnt(0)\n s_waitcnt vmcnt(0)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : : "memory");
        else
            asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" : "+v"(d[2]), "+v"(d[3]) : : "memory");
        request_chunk(q + 2, (BUF + 2) % kGaBufs);
        if (KC == 1) request_rows(nt + 1);
        __builtin_amdgcn_s_setprio(3);
        ga_read<KC & 3, BUF>(d[0], codes[0][KC >> 2], lane_const[0]);
        ga_read<KC & 3, BUF>(d[1], codes[1][KC >> 2], lane_const[0]);
        pair_fma(std::integral_constant<int, KP>{}, std::integral_constant<int, 3>{}, d[2], d[3]);
        ga_read<KC & 3, BUF>(d[2], codes[0][KC >> 2], lane_const[1]);
        ga_read<KC & 3, BUF>(d[3], codes[1][KC >> 2], lane_const[1]);
        if (KC == 0) {
            // new column tile: the rows of gC from the staging area, pieces in this lane's rotated order
            const uint32_t gbase = (uint32_t)(kGaStageBase + wave * 4096 + quad * 128);
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                u32x4 t[8];
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint32_t ga = gbase + (uint32_t)(((quad + s) & 3) << 5);
                    if (r == 0) {
                        asm volatile("ds_read_b128 %0, %2\n ds_read_b128 %1, %2 offset:16" : "=&v"(t[2 * s]), "=&v"(t[2 * s + 1]) : "v"(ga) : "memory");
                    } else {
                        asm volatile("ds_read_b128 %0, %2 offset:2048\n ds_read_b128 %1, %2 offset:2064" : "=&v"(t[2 * s]), "=&v"(t[2 * s + 1]) : "v"(ga) : "memory");
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]), "+v"(d[0]),
                               "+v"(d[1]), "+v"(d[2]), "+v"(d[3])
                             :
                             : "memory");
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const f32x4 v = __builtin_bit_cast(f32x4, t[i]);
                    g[r][4 * i] = v.x; g[r][4 * i + 1] = v.y; g[r][4 * i + 2] = v.z; g[r][4 * i + 3] = v.w;
                }
                if (offset != 0.f) {
                    float s = row_sum[r];
#pragma unroll
                    for (int i = 0; i < kGaCols; ++i) s += g[r][i];
                    row_sum[r] = s;
                }
            }
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
    auto tile_steps = [&](int nt, auto j_tag) {
        constexpr int J = decltype(j_tag)::value;            // position of the tile in the unrolled pass
        [&]<int... KC>(std::integer_sequence<int, KC...>) {
            (chunk_step(nt, std::integral_constant<int, KC>{}, std::integral_constant<int, (J * CH + KC) % kGaBufs>{}), ...);
        }(std::make_integer_sequence<int, CH>{});
    };
    for (int nt0 = 0; nt0 < n_tiles; nt0 += NTU) {
        tile_steps(nt0, std::integral_constant<int, 0>{});
        if (NTU > 1) {
            if (nt0 + 1 < n_tiles) tile_steps(nt0 + 1, std::integral_constant<int, 1 % NTU>{});
            if (nt0 + 2 < n_tiles) tile_steps(nt0 + 2, std::integral_constant<int, 2 % NTU>{});
        }
    }
    // the last pair of reads of the last chunk
    asm volatile("s_waitcnt lgkmcnt(0)\n s_waitcnt vmcnt(0)" : "+v"(d[2]), "+v"(d[3]) : : "memory");
    pair_fma(std::integral_constant<int, CH - 1>{}, std::integral_constant<int, 3>{}, d[2], d[3]);

    // (k outside, row inside: the two stores of a k then fill the same 128 B lines of the image-major layout)
    float* o[2];
    float corr[2];
    size_t k_stride = 4;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int m = m_wave + 16 * r + quad;
        corr[r] = offset * row_sum[r];
        if (m >= M) {
            o[r] = nullptr;
        } else if (rows_per_image > 0) {
            const int img = m / rows_per_image, l = m - img * rows_per_image;
            o[r] = gA + ((size_t)img * K + k0 + c) * rows_per_image + l;
            k_stride = (size_t)4 * rows_per_image;
        } else {
            o[r] = gA + (size_t)m * K + k0 + c;
        }
    }
#pragma unroll
    for (int j = 0; j < CH; ++j)
#pragma unroll
        for (int r = 0; r < 2; ++r)
            if (o[r]) o[r][j * k_stride] = (acc[r][j] + corr[r]) * scale;
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
    if (g.bits > 7 || M < (force ? 2048 : 4096) || (N % kGaCols) != 0 || (K % 16) != 0 || (size_t)M * K >= (1ull << 31)) return 0;
    return (size_t)(N / kGaCols) * (K / kGaChunkK) * kGaChunkBytes;
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
    if (((uintptr_t)gC & 15) != 0) return hipErrorInvalidValue;   // callers check: rows of gC are fetched 16 bytes at a time
    const u32x4* S4 = reinterpret_cast<const u32x4*>(S);
    const dim3 block(kGaWaves * 64);
    const int row_blocks = (M + kGaRows - 1) / kGaRows;
    // 16 row blocks x 2 k groups are in flight on an XCD at a time (measured: 8 to 32 row blocks make no difference,
    // the XCD order gains 15 % where there are few row blocks)
    const int band_rows = 16, xcd_order = 1;
    auto launch = [&](auto kt_tag) {
        constexpr int KT = decltype(kt_tag)::value;
        const dim3 grid(8 * ((row_blocks * (K / KT) + 7) / 8));
        hipLaunchKernelGGL((lutgemm_gradA_slab_kernel<KT>), grid, block, 0, stream, gC, A, S4, gA, flags, M, K, N, scale,
                           rows_per_image, row_blocks, band_rows, xcd_order);
    };
    (void)n_cu;
    // (48 k per workgroup would need more registers than a wave of a 1024-thread workgroup has)
    const int kt = (K % 32) == 0 ? 32 : 16;
    if (kt == 32) launch(std::integral_constant<int, 32>{});
    else launch(std::integral_constant<int, 16>{});
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // masked codes in A or table entries a half cannot hold: the gated direct kernel recomputes gA
    return launch_gradA(gC, A, B, gA, lut, g, M, K, N, scale, n_cu, stream, flags + 2, rows_per_image);
}

}  // namespace amr
