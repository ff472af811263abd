// Forward LUT-GEMM for large M on gfx950: "expanded-table" formulation (7-bit tables and narrower; 8-bit tables: the
// variant at the end of the file).
//
// Same result as lutgemm_fwd_kernel (and as the reference's ApproxGemmForwardKernel,
// self_ops/src/approx_gemm_forward.cu:45-229), different work decomposition:
//
//   step 1  expand_fwd_kernel:  E[k][a][n] = lut[a][B[k,n]] for every code a      (K * 2^b * N gathers)
//   step 2  lutgemm_fwd_slab_kernel:  C[m, :] = sum_k E[k][A[m,k]][:]             (M * K row additions)
//
// Step 1 costs 2^b / M of the M*K*N gathers of the direct kernel.  Step 2 never gathers single
// entries: for one (m,k) a lane reads EIGHT adjacent uint16 entries of row a = A[m,k] with one
// ds_read_b128.  Wide LDS reads move 256 B/clk/CU on gfx950, twice the 32 lanes/clk of 16/32-bit
// gathers, and they are conflict-free by construction here, so the LDS no longer limits the kernel.
//
// Layout of E in HBM (uint16): E[n_tile][k_quad][a (128 rows)][kk (4 values of k)][32 columns]; one
// (n_tile, k_quad) block ("chunk") is 32 KB and a code owns one 256 B line in it.
// A workgroup (16 waves) owns 1024 rows of A and one 32-column tile and walks K chunk by chunk.
// Four chunk buffers live in LDS; chunk c+2 is requested (LDS-direct loads) when chunk c starts to be
// consumed, so a request has two chunk periods to arrive: with one period the L2 latency, not the
// arithmetic, set the pace.  Every chunk a workgroup fetches serves 1024 x 4 x 32 additions.
// Lane l of a wave: row slot rs = l/4 (16 rows per instruction), column group cg = l%4 (8 columns).
// Row slot rs visits the four k of a chunk starting at k = rs%4, so the four slots that the LDS serves
// together (16 lanes of a 128-bit read) read four different 64 B quarters of their 256 B lines: each
// quarter lives in its own 16 banks, which makes every read conflict-free.
// The LDS address (buffer pair<<16 | a<<8 | kk<<6 | cg<<4) is assembled from the code byte and a
// per-lane constant by ONE v_perm_b32 per eight entries.  That needs a < 128: a 7-bit operand holding
// the masked code 128 (zero contribution) is detected, flags[1] is raised and the direct kernel, queued
// behind this one and gated on that flag, recomputes C.
// Accumulation: the four k of a chunk are first added as packed uint16 pairs (plain 32-bit additions:
// no half overflows when 4 * max(lut) < 65536, true of every multiplier table of at most 7 bits) and
// widened to 32 bit once per chunk: 2.5 vector instructions per four entries (one address, two additions,
// two widening additions per pair of columns and four k), which is what bounds the kernel.  A table with
// larger entries (the expand kernel leaves the maximum in flags[0]) is left to the gated direct kernel.
#include <type_traits>

#include "amr_common.h"

namespace amr {

hipError_t launch_zero_u32(void* p, size_t n_dwords, hipStream_t stream);
hipError_t launch_u32_to_f32(void* p, size_t n_dwords, hipStream_t stream);

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // native 16-byte vector (stays in registers)

constexpr int kSlabRows = 128;                       // codes per chunk
constexpr int kSlabCols = 32;                        // columns per n tile
constexpr int kSlabChunkBytes = kSlabRows * 256;     // 32 KB: 128 codes x 4 k x 32 columns x uint16
constexpr int kSlabBuffers = 4;

// ------------------------------------------------------------------------------------------ expand
// grid: (n_tiles, ceil(k_quads / kExpandQuadsPerWg)); 256 threads.  Entries of k >= K or n >= N are
// written as zeros.  Block (0,0) also writes the scratch header: flags[0] = max over the table (used to pick the
// packed accumulation path), flags[1] = 0.
constexpr int kExpandQuadsPerWg = 4;

__global__ __launch_bounds__(256) void expand_fwd_kernel(const uint8_t* __restrict__ B,
                                                         const uint32_t* __restrict__ lut32, int lut_dwords,
                                                         int lut_cols, int n_codes, uint32_t* __restrict__ E,
                                                         uint32_t* __restrict__ flags, int K, int N, int k_quads, int chunk_rows) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* s32 = reinterpret_cast<uint32_t*>(smem);
    uint32_t mx = 0;
    // (eight loads of a thread in flight before the first is stored: a load-wait-store loop pays the memory latency 33 times)
    for (int base = 0; base < lut_dwords; base += 8 * 256) {
        uint32_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = lut32[min(base + u * 256 + (int)threadIdx.x, lut_dwords - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + u * 256 + (int)threadIdx.x;
            if (i < lut_dwords) {
                s32[i] = v[u];
                mx = max(mx, max(v[u] & 0xffffu, v[u] >> 16));
            }
        }
    }
    // Workgroup (0,0) leaves the scratch header for the kernels queued behind this launch: flags[0] = maximum of the table,
    // flags[1] = 0 (no fall-back requested yet); no separate launch clears them.
    uint32_t* wave_max = s32 + lut_dwords;         // four words behind the table (the launch asks for them)
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o));
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = mx;
    __syncthreads();
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        flags[0] = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
        flags[1] = 0u;
        flags[32] = flags[33] = flags[34] = flags[35] = 0u;      // the 16 zero codes the convolution-shaped kernel reads for padding
    }
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // a wave writes whole 256 B lines: lane = (kk, column pair), one dword (two columns) per lane.  Per entry: two
    // 16-bit LDS reads, one shift-or, the store (the kernel should run at the speed of its writes).  Positions
    // beyond K or N and codes beyond the table read the table's all-zero pad column / pad row.
    const int kk = lane >> 4, n = blockIdx.x * kSlabCols + 2 * (lane & 15);
    // the codes of B for all k quads of the workgroup first (one trip to memory instead of one per quad)
    int b0[kExpandQuadsPerWg], b1[kExpandQuadsPerWg];
#pragma unroll
    for (int qq = 0; qq < kExpandQuadsPerWg; ++qq) {
        const int k = 4 * (blockIdx.y * kExpandQuadsPerWg + qq) + kk;
        const bool live0 = (k < K) && (n < N), live1 = (k < K) && (n + 1 < N);
        b0[qq] = live0 ? (int)B[(size_t)k * N + n] : n_codes;
        b1[qq] = live1 ? (int)B[(size_t)k * N + n + 1] : n_codes;
    }
#pragma unroll
    for (int qq = 0; qq < kExpandQuadsPerWg; ++qq) {
        const int q = blockIdx.y * kExpandQuadsPerWg + qq;
        if (q >= k_quads) break;
        // (a chunk holds chunk_rows codes, 256 B each: 128 for tables of at most 7 bits, 256 for 8-bit tables)
        uint32_t* blk = E + ((size_t)blockIdx.x * k_quads + q) * (size_t)(chunk_rows * 64) + lane;
        const uint16_t* p0 = s16 + b0[qq];
        const uint16_t* p1 = s16 + b1[qq];
#pragma unroll 8
        for (int a = wave; a < chunk_rows; a += 4) {
            const int row = min(a, n_codes) * lut_cols;
            blk[a * 64] = (uint32_t)p0[row] | ((uint32_t)p1[row] << 16);
        }
    }
}

// Copies one 32 KB chunk of E from global memory straight into LDS (global_load_lds_dwordx4: the data
// of lane l lands at the wave-uniform LDS base + 16*l; no VGPRs are held while the load is in flight).
// Completion is tracked by vmcnt (two operations per thread and chunk with 1024 threads).
template <int THREADS, int BYTES = kSlabChunkBytes>
__device__ __forceinline__ void slab_copy_chunk(const u32x4* src, unsigned char* lds_dst, int tid, int wave) {
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    constexpr int CPT = BYTES / 16 / THREADS;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const u32x4* g = src + tid + THREADS * i;
        unsigned char* l = lds_dst + (size_t)(THREADS * i + wave * 64) * 16;
        __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)l, 16, 0, 0);
    }
}

// Four 128-bit LDS reads (one row group x four k) issued back to back, NOT waited for.  Inline
// assembly, for two reasons: the reads of the chunk being consumed must not wait for the LDS-direct
// loads of later chunks (the compiler cannot tell the two apart, same LDS array), and the reads of
// block b+1 are issued before block b is consumed (software pipelining with explicit counters).
// OFF is the part of the buffer offset that does not fit the v_perm-built address (odd buffers).
template <int OFF>
__device__ __forceinline__ void slab_issue4(u32x4 (&d)[4], const uint32_t (&addr)[4]) {
    asm volatile(
        "ds_read_b128 %0, %4 offset:%8\n ds_read_b128 %1, %5 offset:%8\n ds_read_b128 %2, %6 offset:%8\n"
        "ds_read_b128 %3, %7 offset:%8"
        : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3])
        : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3]), "n"(OFF)
        : "memory");
}

// Waits until at most PENDING LDS operations are outstanding.  The four results are passed through
// as in/out operands so that every use of them is ordered after the wait.
template <int PENDING>
__device__ __forceinline__ void slab_wait4(u32x4 (&d)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]) : "n"(PENDING) : "memory");
}

__device__ __forceinline__ void slab_addr4(uint32_t (&addr)[4], uint32_t codes4, const uint32_t (&base)[4],
                                           const uint32_t (&sel)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) addr[j] = __builtin_amdgcn_perm(codes4, base[j], sel[j]);
}

// One pair of columns (one dword of each of the four reads of a row group) into its two sums.
// PACKED (4 * max(lut) < 65536): even / odd are the sums of the even and of the odd column.
// Otherwise: even collects the whole dwords, i.e. sum(even entries) + 65536 * sum(odd entries) modulo 2^32, and odd the odd
// entries alone; slab_store_tile takes 65536 * odd off again (the sums are defined modulo 2^32 anyway).  That is six
// instructions per eight entries instead of eight (or twelve with masks and shifts).
template <bool PACKED>
__device__ __forceinline__ void slab_add_pair(uint32_t& even, uint32_t& odd, uint32_t x0, uint32_t x1, uint32_t x2, uint32_t x3) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    if (PACKED) {
        // (no 16-bit half of these sums overflows, so one 32-bit addition adds both halves and a three-operand
        // addition saves an instruction per pair of columns over packed 16-bit additions)
        const us2 s = __builtin_bit_cast(us2, (x0 + x1 + x2) + x3);
        even += s.x;
        odd += s.y;
    } else {
        even = (even + x0 + x1) + x2 + x3;
        const us2 hi = {0, 1};
        odd = __builtin_amdgcn_udot2(__builtin_bit_cast(us2, x0), hi, odd, false);
        odd = __builtin_amdgcn_udot2(__builtin_bit_cast(us2, x1), hi, odd, false);
        odd = __builtin_amdgcn_udot2(__builtin_bit_cast(us2, x2), hi, odd, false);
        odd = __builtin_amdgcn_udot2(__builtin_bit_cast(us2, x3), hi, odd, false);
    }
}

// One chunk (4 k) for all RG row groups of a lane; every code is < 128 (8-bit kernel: < 256).
template <int RG, bool PACKED, int OFF>
__device__ __forceinline__ void slab_chunk_fast(uint32_t (&acc)[RG][8], const uint32_t (&a_cur)[RG],
                                                const uint32_t (&base)[4], const uint32_t (&sel)[4]) {
    u32x4 d[2][4];
    {
        uint32_t addr[4];
        slab_addr4(addr, a_cur[0], base, sel);
        slab_issue4<OFF>(d[0], addr);
    }
#pragma unroll
    for (int b = 0; b < RG; ++b) {
        // waves that are behind go first: the four waves of a SIMD then move through a chunk in step instead of one
        // after the other (oldest first), and the last one does not run alone, latencies exposed, before the barrier
        if (b == 0) __builtin_amdgcn_s_setprio(3);
        else if (b == 1) __builtin_amdgcn_s_setprio(2);
        else if (b == 2) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
        if (b + 1 < RG) {
            uint32_t addr[4];
            slab_addr4(addr, a_cur[b + 1], base, sel);
            slab_issue4<OFF>(d[(b + 1) & 1], addr);
            slab_wait4<4>(d[b & 1]);
        } else {
            slab_wait4<0>(d[b & 1]);
        }
        const u32x4 x0 = d[b & 1][0], x1 = d[b & 1][1], x2 = d[b & 1][2], x3 = d[b & 1][3];
        slab_add_pair<PACKED>(acc[b][0], acc[b][1], x0.x, x1.x, x2.x, x3.x);
        slab_add_pair<PACKED>(acc[b][2], acc[b][3], x0.y, x1.y, x2.y, x3.y);
        slab_add_pair<PACKED>(acc[b][4], acc[b][5], x0.z, x1.z, x2.z, x3.z);
        slab_add_pair<PACKED>(acc[b][6], acc[b][7], x0.w, x1.w, x2.w, x3.w);
        // Pin the accumulation here: an empty volatile asm that "modifies" the eight accumulators cannot
        // be moved across the volatile read blocks, so the sums are not postponed until all reads of
        // the chunk are done (which would keep every result live and overflow the register file).
        asm volatile("" : "+v"(acc[b][0]), "+v"(acc[b][1]), "+v"(acc[b][2]), "+v"(acc[b][3]), "+v"(acc[b][4]),
                          "+v"(acc[b][5]), "+v"(acc[b][6]), "+v"(acc[b][7]));
    }
}

// ------------------------------------------------------------------------------------------ consume
// The codes of A take the same road as the chunks: LDS-direct loads into a small staging area, 16 bytes
// (the codes of four chunks) per row at a time, so that a cache line of A is asked for 8 times, not 32
// (1024 rows x 128 B per workgroup do not stay in the caches between two visits).  No load of the main loop
// has a register destination, so all waiting is explicit: the compiler forces vmcnt(0) in front of every
// s_barrier it knows of and in front of the first use of a loaded register once LDS-direct loads are
// pending, either of which would serialise the loop on the memory latency.  The barrier is therefore
// issued from inline assembly together with the one wait that is needed.
constexpr int kSlabCodeBytes = 16 * 64 * 16;   // staging of one group of four chunks: 16 waves x 64 rows x 16 codes

// Four dwords at a stride of 256 B (the codes of this lane's four rows for one chunk).
__device__ __forceinline__ void slab_read_codes(uint32_t (&a)[4], uint32_t addr) {
    asm volatile(
        "ds_read_b32 %0, %4\n ds_read_b32 %1, %4 offset:256\n ds_read_b32 %2, %4 offset:512\n ds_read_b32 %3, %4 offset:768\n"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(a[0]), "=&v"(a[1]), "=&v"(a[2]), "=&v"(a[3])
        : "v"(addr)
        : "memory");
}

// The sums of a wave (64 rows x 32 columns) leave through LDS, 8 KB per wave in the chunk buffers nobody reads any more,
// so that every store or atomic instruction of a wave covers two whole 128 B lines of C (straight from the accumulators an
// instruction would touch 16 rows and four dwords in each; a split K adds its sums with atomics, which pay per line).
// The caller has waited for its loads towards LDS and passed a workgroup barrier.
template <int RG, bool PACKED>
__device__ __forceinline__ void slab_store_tile(const uint32_t (&acc)[RG][8], unsigned char* wave_lds, int lane, int rs, int cg,
                                                uint32_t* __restrict__ C, int m_wave, int m_first, int n0, int N, int atomic_out,
                                                int out_f32) {
#pragma unroll
    for (int i = 0; i < RG; ++i) {
        u32x4* dst = reinterpret_cast<u32x4*>(wave_lds + (16 * i + rs) * 128 + cg * 32);
        u32x4 lo, hi;
        // (see slab_add_pair for what the even accumulators of the unpacked flavour hold)
        lo.x = PACKED ? acc[i][0] : acc[i][0] - (acc[i][1] << 16); lo.y = acc[i][1];
        lo.z = PACKED ? acc[i][2] : acc[i][2] - (acc[i][3] << 16); lo.w = acc[i][3];
        hi.x = PACKED ? acc[i][4] : acc[i][4] - (acc[i][5] << 16); hi.y = acc[i][5];
        hi.z = PACKED ? acc[i][6] : acc[i][6] - (acc[i][7] << 16); hi.w = acc[i][7];
        dst[0] = lo;
        dst[1] = hi;
    }
    const uint32_t* w32 = reinterpret_cast<const uint32_t*>(wave_lds);
    const int col = lane & 31, half = lane >> 5;
    const int n = n0 + col;
#pragma unroll 8
    for (int p = 0; p < 8 * RG; ++p) {
        const int row = 2 * p + half;
        const int m = m_wave + row;
        const uint32_t v = w32[row * 32 + col];
        if (m >= m_first && n < N) {
            if (atomic_out)
                atomicAdd(&C[(size_t)m * N + n], v);
            else if (out_f32)
                C[(size_t)m * N + n] = __float_as_uint((float)v);
            else
                C[(size_t)m * N + n] = v;
        }
    }
}

// The same tile, dequantised on its way out and stored as the NCHW activation:
//   out[b,n,pos] = (s_a*s_w) * ((float)sum + ((z_w*xs[m] + z_a*wr[n,pos]) + (z_a*z_w)*tp[pos])) + bias[n],   m = b*L + pos
// every operation rounded on its own in that order (the bits of dequant_rows_to_nchw_kernel on the float32 sums).  The sums
// go to LDS column-major ([32 columns][64 rows]); afterwards lane = row, so that a store instruction writes 64 consecutive
// positions of one output channel (256 B) and reads 64 different banks.
template <int RG, bool PACKED>
__device__ __forceinline__ void slab_store_tile_dequant(const uint32_t (&acc)[RG][8], unsigned char* wave_lds, int lane, int rs, int cg,
                                                        const SlabDequant& dq, int m_wave, int m_first, int n0, int N) {
    float* w = reinterpret_cast<float*>(wave_lds);
#pragma unroll
    for (int i = 0; i < RG; ++i) {
        const int row = 16 * i + rs;
#pragma unroll
        for (int c = 0; c < 8; c += 2) {
            const uint32_t even = PACKED ? acc[i][c] : acc[i][c] - (acc[i][c + 1] << 16);
            w[(cg * 8 + c) * 64 + row] = (float)even;
            w[(cg * 8 + c + 1) * 64 + row] = (float)acc[i][c + 1];
        }
    }
    const int m = m_wave + lane;
    const int L = dq.L;
    const int b = m / L, pos = m - b * L;
    const float za = *dq.za, zw = *dq.zw;
    const float s = __fmul_rn(*dq.sa, *dq.sw), zz = __fmul_rn(za, zw);
    const float x_term = __fmul_rn(zw, dq.xs[m]);
    const float t_term = __fmul_rn(zz, dq.tp[pos]);
    const float* wr = dq.wr + pos;
    float* out = dq.out + (size_t)b * N * L + pos;
    const bool live = m >= m_first;
#pragma unroll 8
    for (int col = 0; col < 32; ++col) {
        const int n = n0 + col;
        if (n < N && live) {
            const float terms = __fadd_rn(__fadd_rn(x_term, __fmul_rn(za, wr[(size_t)n * L])), t_term);
            float v = __fmul_rn(s, __fadd_rn(w[col * 64 + lane], terms));
            if (dq.bias != nullptr) v = __fadd_rn(v, dq.bias[n]);
            out[(size_t)n * L] = v;
        }
    }
}

// CONV: A holds pixel-major codes [M][cv.C] and K = 9 * cv.C: the 16 codes a lane fetches per group are 16 adjacent
// channels of ONE tap (cv.C % 16 == 0, no K split), i.e. 16 adjacent bytes of a neighbouring pixel, or of the zero line
// where that neighbour is padding -- no window matrix is read.
template <int RG, int WAVES, bool PACKED, bool DEQ = false, bool CONV = false>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_fwd_slab_kernel(
    const uint8_t* __restrict__ A, const u32x4* __restrict__ E, uint32_t* __restrict__ C,
    uint32_t* __restrict__ flags, int M, int K, int N, int k_quads, int chunks_per_split, int atomic_out, int out_f32,
    int n_tiles_grouped, int row_blocks, SlabDequant dq, SlabConv cv) {
    // static: lets the compiler fold the base address (chunk buffers first: their addresses come out of v_perm)
    __shared__ __align__(16) unsigned char smem[kSlabBuffers * kSlabChunkBytes + 2 * kSlabCodeBytes];
    constexpr int THREADS = WAVES * 64;
    constexpr int ROWS_PER_WAVE = 16 * RG;
    static_assert(RG == 4 && WAVES == 16, "staging layout and vmcnt bookkeeping are written for 16 waves of 64 rows");
    static_assert(kSlabChunkBytes / 16 / THREADS == 2, "two chunk-copy operations per thread and chunk");
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 2, cg = lane & 3, rot = rs & 3;
    // Workgroup -> (column tile, row block, K split).  Plain: the grid's three dimensions.  Grouped (n_tiles_grouped > 0,
    // 1-D grid, no K split): the hardware deals workgroups to the 8 XCDs round-robin by index; the column tiles of one
    // row block get consecutive slots of ONE XCD, so that they run at the same time behind the same L2 and fetch their
    // rows of A once between them (chosen by the host when A is larger than the expanded table).
    int tile_x = blockIdx.x, rb_y = blockIdx.y;
    const int split_z = blockIdx.z;
    if (n_tiles_grouped > 0) {
        const int xcd = (int)(blockIdx.x & 7), slot = (int)(blockIdx.x >> 3);
        tile_x = slot % n_tiles_grouped;
        rb_y = xcd + 8 * (slot / n_tiles_grouped);
        if (rb_y >= row_blocks) return;
    }
    // A wave whose rows would stick out of M is shifted up so that all its rows exist (the host only
    // takes this path for M >= 2048); the rows it then shares with the wave above are not stored twice.
    // (a wave entirely beyond M keeps running, it takes part in the chunk copies, and stores nothing)
    const int m_first = (rb_y * WAVES + wave) * ROWS_PER_WAVE;     // first row this wave must store
    const int m_wave = min(m_first, M - ROWS_PER_WAVE);
    const int c_begin = split_z * chunks_per_split;
    const int c_end = min(k_quads, c_begin + chunks_per_split);
    if (c_begin >= c_end) return;
    // 16-bit packed partial sums need 4 * max(lut) < 65536 (true of every multiplier table of at most 7 bits: 127 * 127 =
    // 16129; the expand kernel left the maximum in flags[0]).  A table with larger entries goes to the direct kernel,
    // which is queued behind this launch and gated on flags[1]; the other accumulation flavour serves 8-bit tables.
    if (PACKED && flags[0] >= 16384u) {
        if (tid == 0) atomicOr(&flags[1], 1u);
        return;
    }

    const u32x4* Eblk = E + ((size_t)tile_x * k_quads) * (kSlabChunkBytes / 16);

    // per-lane address pieces; instruction j of a chunk reads k = 4c + ((j + rot) & 3)
    uint32_t base_lo[4], base_hi[4], sel[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t kk = (uint32_t)((j + rot) & 3);
        base_lo[j] = (kk << 6) | (uint32_t)(cg << 4);
        base_hi[j] = base_lo[j] | 0x10000u;
        sel[j] = 0x0c020000u | ((4u + kk) << 8);
    }

    uint32_t acc[RG][8];
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0u;

    // Lane (rs, cg) consumes rows m_wave + 16 i + rs, i < 4.  Lane l fetches the codes of row m_wave + l,
    // which land at staging position l (16 B each): the four dword reads of a chunk are 256 B apart and the
    // eight row slots that one pass of a read serves are 16 B apart, in eight different banks.
    // 32-bit offsets: the host only takes this path when M*K < 2^31.
    const uint32_t code_off = (uint32_t)(m_wave + lane) * (uint32_t)(CONV ? cv.C : K);
    // CONV: which neighbours of this lane's pixel exist: bit 0 the row below, 1 the row above, 2 the pixel to the right, 3 the
    // pixel to the left
    uint32_t neighbours = 0;
    if constexpr (CONV) {
        const int m = m_wave + lane;
        const int pix = m % (cv.H * cv.W);
        const int y = pix / cv.W, x = pix - y * cv.W;
        neighbours = (uint32_t)((y + 1 < cv.H) | ((y >= 1) << 1) | ((x + 1 < cv.W) << 2) | ((x >= 1) << 3));
    }
    unsigned char* code_stage = smem + kSlabBuffers * kSlabChunkBytes + wave * 1024;      // + (group & 1) * kSlabCodeBytes
    const uint32_t code_read = (uint32_t)(kSlabBuffers * kSlabChunkBytes + wave * 1024 + rs * 16);

    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // Chunks / groups beyond the end repeat the last one (into buffers nobody reads any more) so that every
    // step issues the same number of operations.  K % 4 == 0 (host): a group starts at code 4 (c_begin + 4 g);
    // the last group is moved back so that its 16 bytes stay inside the row.
    const int g_last = (c_end - 1 - c_begin) >> 2;
    auto group_koff = [&](int g) { return min(4 * (c_begin + 4 * min(g, g_last)), K - 16); };
    auto request_codes = [&](int g) {
        if constexpr (CONV) {
            // tap (ti, tj) of output pixel (y, x) reads input pixel (y + ti - 1, x + tj - 1)
            const int koff = group_koff(g);
            const int tap = koff / cv.C, c0 = koff - tap * cv.C;
            const int ti = tap / 3, tj = tap - 3 * ti;
            const uint32_t need = (ti == 0 ? 2u : 0u) | (ti == 2 ? 1u : 0u) | (tj == 0 ? 8u : 0u) | (tj == 2 ? 4u : 0u);
            const int off = (int)code_off + ((ti - 1) * cv.W + (tj - 1)) * cv.C + c0;
            const uint8_t* p = (neighbours & need) == need ? A + off : cv.zero;
            __builtin_amdgcn_global_load_lds((gptr_t)p, (lptr_t)(code_stage + (g & 1) * kSlabCodeBytes), 16, 0, 0);
            return;
        }
        __builtin_amdgcn_global_load_lds((gptr_t)(A + (code_off + (uint32_t)group_koff(g))),
                                         (lptr_t)(code_stage + (g & 1) * kSlabCodeBytes), 16, 0, 0);
    };
    auto request_chunk = [&](int c, int buf) {
        slab_copy_chunk<THREADS>(Eblk + (size_t)min(c, c_end - 1) * (kSlabChunkBytes / 16), smem + (size_t)buf * kSlabChunkBytes, tid, wave);
    };

    uint32_t seen = 0;   // OR of every code dword this lane consumed

    // vmcnt counts the operations of a thread in issue order:
    //   codes(g0) chunk(c0) chunk(c0+1) | step 0 of group g: codes(g+1) chunk(c+2) | steps 1..3: chunk(c+2)
    // (a chunk request is two operations).  At the top of a step chunk(c), issued two steps earlier, and the
    // codes of its group must have landed: everything but the requests of the previous step.
    request_codes(0);
    request_chunk(c_begin, 0);
    request_chunk(c_begin + 1, 1);

    auto step = [&](int c, int g, auto buf_tag) {
        constexpr int BUF = decltype(buf_tag)::value;
        if (BUF == 1)
            asm volatile("s_waitcnt vmcnt(3)\n s_barrier" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(2)\n s_barrier" ::: "memory");
        if (BUF == 0) request_codes(g + 1);
        request_chunk(c + 2, (BUF + 2) & 3);
        uint32_t mine[RG];
        slab_read_codes(mine, code_read + (uint32_t)((g & 1) * kSlabCodeBytes + (4 * c - group_koff(g))));
#pragma unroll
        for (int i = 0; i < RG; ++i) seen |= mine[i];
        if (BUF & 2)
            slab_chunk_fast<RG, PACKED, (BUF & 1) * kSlabChunkBytes>(acc, mine, base_hi, sel);
        else
            slab_chunk_fast<RG, PACKED, (BUF & 1) * kSlabChunkBytes>(acc, mine, base_lo, sel);
    };
    for (int c = c_begin, g = 0; c < c_end; c += 4, ++g) {
        step(c, g, std::integral_constant<int, 0>{});
        if (c + 1 < c_end) step(c + 1, g, std::integral_constant<int, 1>{});
        if (c + 2 < c_end) step(c + 2, g, std::integral_constant<int, 2>{});
        if (c + 3 < c_end) step(c + 3, g, std::integral_constant<int, 3>{});
    }
    // nothing is left in flight towards LDS and every wave has read its last chunk: the buffers take the sums
    asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");

    // A code with bit 7 set (the masked code 128 of a 7-bit table) cannot be addressed by this kernel:
    // raise flags[1]; the host has queued the direct kernel behind this one, gated on that flag.
    if (__builtin_amdgcn_ballot_w64((seen & 0x80808080u) != 0) != 0) {
        if (lane == 0) atomicOr(&flags[1], 1u);
    }
    if constexpr (DEQ)
        slab_store_tile_dequant<RG, PACKED>(acc, smem + wave * 8192, lane, rs, cg, dq, m_wave, m_first, tile_x * kSlabCols, N);
    else
        slab_store_tile<RG, PACKED>(acc, smem + wave * 8192, lane, rs, cg, C, m_wave, m_first, tile_x * kSlabCols, N, atomic_out, out_f32);
}

// ------------------------------------------------------------------------------------------ 8-bit tables
// The same scheme for 256 codes: a chunk (four k, 32 columns) is 256 lines of 256 B = 64 KB, the code byte still
// lands in byte 1 of the LDS address through the one v_perm_b32, and the chunk buffer is picked by byte 2.  Two chunk
// buffers and the code staging fill the 160 KB of a CU exactly, so a chunk is requested one chunk period ahead only
// (chunk c+1 when chunk c starts): the kernel runs at the pace the chunks arrive (0.5 B per multiply-add, twice the
// volume of the 7-bit kernel).  Every code of a uint8 operand has its line: no masked code, no fall-back.
constexpr int kSlab8Rows = 256;
constexpr int kSlab8ChunkBytes = kSlab8Rows * 256;   // 64 KB

template <bool PACKED, bool DEQ = false>
__global__ __launch_bounds__(1024) void lutgemm_fwd_slab8_kernel(
    const uint8_t* __restrict__ A, const u32x4* __restrict__ E, uint32_t* __restrict__ C,
    const uint32_t* __restrict__ flags, int M, int K, int N, int k_quads, int chunks_per_split, int atomic_out, int out_f32,
    SlabDequant dq) {
    __shared__ __align__(16) unsigned char smem[2 * kSlab8ChunkBytes + 2 * kSlabCodeBytes];
    constexpr int RG = 4, WAVES = 16, THREADS = WAVES * 64, ROWS_PER_WAVE = 16 * RG;
    static_assert(2 * kSlab8ChunkBytes + 2 * kSlabCodeBytes == 160 * 1024, "the workgroup uses the whole LDS of a CU");
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 2, cg = lane & 3, rot = rs & 3;
    const int tile_x = blockIdx.x, rb_y = blockIdx.y, split_z = blockIdx.z;
    // (a wave whose rows would stick out of M is shifted up; the rows it shares with the wave above are stored once)
    const int m_first = (rb_y * WAVES + wave) * ROWS_PER_WAVE;
    const int m_wave = min(m_first, M - ROWS_PER_WAVE);
    const int c_begin = split_z * chunks_per_split;
    const int c_end = min(k_quads, c_begin + chunks_per_split);
    if (c_begin >= c_end) return;

    const u32x4* Eblk = E + ((size_t)tile_x * k_quads) * (kSlab8ChunkBytes / 16);
    // instruction j of a chunk reads k = 4c + ((j + rot) & 3); byte 2 of the address = chunk buffer
    uint32_t base0[4], base1[4], sel[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t kk = (uint32_t)((j + rot) & 3);
        base0[j] = (kk << 6) | (uint32_t)(cg << 4);
        base1[j] = base0[j] | 0x10000u;
        sel[j] = 0x0c020000u | ((4u + kk) << 8);
    }
    uint32_t acc[RG][8];
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0u;

    // codes: as in the 7-bit kernel (16 bytes = four chunks per row and request; row r of the wave at staging position r)
    const uint32_t code_off = (uint32_t)(m_wave + lane) * (uint32_t)K;
    unsigned char* code_stage = smem + 2 * kSlab8ChunkBytes + wave * 1024;
    const uint32_t code_read = (uint32_t)(2 * kSlab8ChunkBytes + wave * 1024 + rs * 16);
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    const int g_last = (c_end - 1 - c_begin) >> 2;
    auto group_koff = [&](int g) { return min(4 * (c_begin + 4 * min(g, g_last)), K - 16); };
    auto request_codes = [&](int g) {
        __builtin_amdgcn_global_load_lds((gptr_t)(A + (code_off + (uint32_t)group_koff(g))),
                                         (lptr_t)(code_stage + (g & 1) * kSlabCodeBytes), 16, 0, 0);
    };
    auto request_chunk = [&](int c, int buf) {
        slab_copy_chunk<THREADS, kSlab8ChunkBytes>(Eblk + (size_t)min(c, c_end - 1) * (kSlab8ChunkBytes / 16),
                                                   smem + (size_t)buf * kSlab8ChunkBytes, tid, wave);
    };
    // Operations of a thread towards memory, in issue order: codes(0) chunk(c0) | step c: [codes(g+1) in the first step of
    // a group] chunk(c+1).  At the top of a step everything issued so far must have landed (chunk c was the last request of
    // the previous step); behind the barrier every wave has finished reading the buffer the next request overwrites.
    request_codes(0);
    request_chunk(c_begin, 0);
    auto step = [&](int c, int g, auto buf_tag, bool first_of_group) {
        constexpr int BUF = decltype(buf_tag)::value;
        asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
        if (first_of_group) request_codes(g + 1);
        request_chunk(c + 1, BUF ^ 1);
        uint32_t mine[RG];
        slab_read_codes(mine, code_read + (uint32_t)((g & 1) * kSlabCodeBytes + (4 * c - group_koff(g))));
        if (BUF)
            slab_chunk_fast<RG, PACKED, 0>(acc, mine, base1, sel);
        else
            slab_chunk_fast<RG, PACKED, 0>(acc, mine, base0, sel);
    };
    // (chunk c of the split sits in buffer (c - c_begin) & 1; a group of codes covers four chunks)
    for (int c = c_begin, g = 0; c < c_end; c += 4, ++g) {
        step(c, g, std::integral_constant<int, 0>{}, true);
        if (c + 1 < c_end) step(c + 1, g, std::integral_constant<int, 1>{}, false);
        if (c + 2 < c_end) step(c + 2, g, std::integral_constant<int, 0>{}, false);
        if (c + 3 < c_end) step(c + 3, g, std::integral_constant<int, 1>{}, false);
    }
    // nothing is left in flight towards LDS and every wave has read its last chunk: the buffers take the sums
    asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
    if constexpr (DEQ)
        slab_store_tile_dequant<RG, PACKED>(acc, smem + wave * 8192, lane, rs, cg, dq, m_wave, m_first, tile_x * kSlabCols, N);
    else
        slab_store_tile<RG, PACKED>(acc, smem + wave * 8192, lane, rs, cg, C, m_wave, m_first, tile_x * kSlabCols, N, atomic_out, out_f32);
}

hipError_t launch_fwd_gated(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                            int M, int K, int N, const uint32_t* gate, hipStream_t stream, int out_f32);

// ------------------------------------------------------------------------------------------ host
// Workspace layout: [256 B flags][E].  Returns 0 when the expanded-table path does not apply.
size_t fwd_slab_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force) {
    // Worth it when the 2^b/M expansion overhead is small and there is enough work to amortise the extra launches.
    // (K % 4 == 0: the codes of A are fetched four and sixteen at a time)
    if (M < 2048 || K < (force ? 32 : 64) || (K & 3) != 0 || (size_t)M * K >= (1ull << 31)) return 0;
    if (g.bits == 8) {
        // 8-bit tables: 64 KB per (column tile, four k); every block of 1024 rows streams all of it, so the rows have to
        // outnumber the 256 codes well (measured against the direct kernel on MI355X: even at 2048 rows, 157 against 198 us
        // at 4096 x 1152 x 256)
        if (!force && (M < 4096 || (size_t)M * K * N < (3ull << 28))) return 0;
        return 256 + (size_t)((N + kSlabCols - 1) / kSlabCols) * (((size_t)K + 3) / 4) * kSlab8ChunkBytes;
    }
    // below about 4e8 multiply-adds the extra launches (expansion, gated fall-back) cost more than the
    // faster kernel gains (measured on MI355X: even at 3e8, 57 against 85 us at 5.4e8)
    if (!force && (size_t)M * K * N < (3ull << 27)) return 0;
    const size_t n_tiles = (N + kSlabCols - 1) / kSlabCols;
    const size_t k_quads = ((size_t)K + 3) / 4;
    return 256 + n_tiles * k_quads * kSlabChunkBytes;
}

hipError_t launch_dequant_gated(const float* c, const float* xs, const float* wr, const float* tp, const float* za, const float* zw,
                                const float* sa, const float* sw, const float* bias, float* out, int M, int N, int L,
                                const uint32_t* gate, hipStream_t stream);

// K splits of the expanded-table forward launch for this shape (1: every workgroup owns whole sums).
static int fwd_slab_ksplit(int M, int K, int N, int n_cu) {
    const int n_tiles = (N + kSlabCols - 1) / kSlabCols, k_quads = (K + 3) / 4;
    const long wgs = (long)n_tiles * ((M + 1023) / 1024);
    int ksplit = 1;
    if (wgs < n_cu) {
        ksplit = (int)((n_cu + wgs - 1) / wgs);
        const int max_split = k_quads / 8 > 0 ? k_quads / 8 : 1;     // at least 32 k per workgroup
        if (ksplit > max_split) ksplit = max_split;
    }
    const int cps = (k_quads + ksplit - 1) / ksplit;
    return (k_quads + cps - 1) / cps;
}

// The expanded-table forward pass can dequantise in its store when no K split adds partial sums in memory.
bool fwd_slab_can_dequant(const LutGeom& g, int M, int K, int N, int n_cu, bool force) {
    return fwd_slab_workspace_bytes(g, M, K, N, force) != 0 && fwd_slab_ksplit(M, K, N, n_cu) == 1;
}

// dq != nullptr (only with fwd_slab_can_dequant): the kernel stores the dequantised NCHW activation dq->out instead of C; C
// (float32 [M,N]) is then scratch that only the gated fall-back touches, followed by a dequantisation pass under the same gate.
// expanded != 0: `workspace` already holds the expansion of this B and table (a caller's cache); only the fall-back request
// in its header is cleared, by a one-word fill, in place of the expansion launch.
hipError_t launch_poison_if_raised(float* gx, size_t total, const uint32_t* gate, hipStream_t stream);

// Whether the convolution-shaped forward launch serves this geometry (then with a dequantising store and no K split).
bool fwd_slab_conv_applies(const LutGeom& g, long M, int C, int N, int n_cu, bool force) {
    if (g.bits > 7 || (C & 15) != 0 || M > (1L << 30) || 9L * C > (1L << 24)) return false;
    return fwd_slab_can_dequant(g, (int)M, 9 * C, N, n_cu, force);
}

// cv != nullptr (only with fwd_slab_conv_applies and dq): A holds the pixel-major codes of the layer's input, B the
// tap-major weight codes [9 C][N]; a_fallback (optional) the window matrix [M][9 C] for the gated direct kernel -- without
// it a masked code or a table that does not fit packed sums leaves NaN in dq->out.
hipError_t launch_fwd_slab(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                           int M, int K, int N, int n_cu, void* workspace, hipStream_t stream, int out_f32,
                           const SlabDequant* dq = nullptr, int expanded = 0, const SlabConv* cv = nullptr,
                           const uint8_t* a_fallback = nullptr) {
    const int n_tiles = (N + kSlabCols - 1) / kSlabCols;
    const int k_quads = (K + 3) / 4;
    const SlabDequant none{};
    const SlabConv no_conv{};
    if (cv && (!dq || g.bits == 8)) return hipErrorInvalidValue;
    uint32_t* flags = reinterpret_cast<uint32_t*>(workspace);
    uint32_t* E = reinterpret_cast<uint32_t*>(reinterpret_cast<unsigned char*>(workspace) + 256);
    hipError_t e;
    const int lut_dwords = g.rows * g.cols / 2;
    if (expanded && (e = launch_zero_u32(flags + 1, 1, stream)) != hipSuccess) return e;
    if (g.bits == 8) {
        static std::atomic<uint64_t> attr_done{0};
        if ((e = allow_full_lds(reinterpret_cast<const void*>(expand_fwd_kernel), attr_done)) != hipSuccess) return e;
        if (!expanded)
            hipLaunchKernelGGL(expand_fwd_kernel, dim3(n_tiles, (k_quads + kExpandQuadsPerWg - 1) / kExpandQuadsPerWg), dim3(256),
                               (size_t)lut_dwords * 4 + 16, stream, B, reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols,
                               1 << g.bits, E, flags, K, N, k_quads, kSlab8Rows);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        const int row_blocks8 = (M + 1023) / 1024;
        const long wgs8 = (long)n_tiles * row_blocks8;
        int ksplit8 = 1;
        if (wgs8 < n_cu) {
            ksplit8 = (int)((n_cu + wgs8 - 1) / wgs8);
            const int max_split = k_quads / 8 > 0 ? k_quads / 8 : 1;     // at least 32 k per workgroup
            if (ksplit8 > max_split) ksplit8 = max_split;
        }
        const int cps8 = (k_quads + ksplit8 - 1) / ksplit8;
        const int zs8 = (k_quads + cps8 - 1) / cps8;
        if (zs8 > 1 && (e = launch_zero_u32(C, (size_t)M * N, stream)) != hipSuccess) return e;
        const dim3 grid8(n_tiles, row_blocks8, zs8);
        if (dq) {
            if (zs8 != 1) return hipErrorInvalidValue;
            hipLaunchKernelGGL((lutgemm_fwd_slab8_kernel<false, true>), grid8, dim3(1024), 0, stream, A, reinterpret_cast<const u32x4*>(E), C,
                               flags, M, K, N, k_quads, cps8, 0, 1, *dq);
            return hipGetLastError();
        }
        hipLaunchKernelGGL((lutgemm_fwd_slab8_kernel<false>), grid8, dim3(1024), 0, stream, A, reinterpret_cast<const u32x4*>(E), C, flags,
                           M, K, N, k_quads, cps8, zs8 > 1 ? 1 : 0, out_f32, none);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if (zs8 > 1 && out_f32) return launch_u32_to_f32(C, (size_t)M * N, stream);
        return hipSuccess;
    }
    if (!expanded)
        hipLaunchKernelGGL(expand_fwd_kernel, dim3(n_tiles, (k_quads + kExpandQuadsPerWg - 1) / kExpandQuadsPerWg), dim3(256),
                           (size_t)lut_dwords * 4 + 16, stream, B, reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols,
                           1 << g.bits, E, flags, K, N, k_quads, kSlabRows);
    e = hipGetLastError();
    if (e != hipSuccess) return e;

    // 16 waves x 64 rows = 1024 rows per workgroup
    constexpr int RG = 4, WAVES = 16;
    const int m_tile = WAVES * 16 * RG;
    const long wgs = (long)n_tiles * ((M + m_tile - 1) / m_tile);
    int ksplit = 1;
    if (wgs < n_cu) {
        ksplit = (int)((n_cu + wgs - 1) / wgs);
        const int max_split = k_quads / 8 > 0 ? k_quads / 8 : 1;     // at least 32 k per workgroup
        if (ksplit > max_split) ksplit = max_split;
    }
    const int cps = (k_quads + ksplit - 1) / ksplit;
    const int zs = (k_quads + cps - 1) / cps;
    if (zs > 1) {
        e = launch_zero_u32(C, (size_t)M * N, stream);
        if (e != hipSuccess) return e;
    }
    const int row_blocks = (M + m_tile - 1) / m_tile;
    dim3 grid(n_tiles, row_blocks, zs);
    // A larger than the expanded table (M > 256 N) and several column tiles: the tiles of a row block share an XCD
    int grouped = 0;
    // (measured: conv2_x 0.40 -> 0.38 ms, conv3_x 0.395 -> 0.37 ms; with a split K the rows are few and A is small)
    if (zs == 1 && n_tiles > 1 && (size_t)M > (size_t)256 * N) {
        grouped = n_tiles;
        grid = dim3(8 * ((row_blocks + 7) / 8) * n_tiles);
    }
    if (cv) {
        if (zs != 1) return hipErrorInvalidValue;
        SlabConv c = *cv;
        c.zero = reinterpret_cast<const uint8_t*>(flags + 32);
        hipLaunchKernelGGL((lutgemm_fwd_slab_kernel<RG, WAVES, true, true, true>), grid, dim3(WAVES * 64), 0, stream, A,
                           reinterpret_cast<const u32x4*>(E), C, flags, M, K, N, k_quads, cps, 0, 1, grouped, row_blocks, *dq, c);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if (!a_fallback) return launch_poison_if_raised(dq->out, (size_t)M * N, flags + 1, stream);
        if ((e = launch_fwd_gated(a_fallback, B, C, lut, g, M, K, N, flags + 1, stream, 1)) != hipSuccess) return e;
        return launch_dequant_gated(reinterpret_cast<const float*>(C), dq->xs, dq->wr, dq->tp, dq->za, dq->zw, dq->sa, dq->sw, dq->bias,
                                    dq->out, M, N, dq->L, flags + 1, stream);
    }
    if (dq) {
        if (zs != 1) return hipErrorInvalidValue;
        hipLaunchKernelGGL((lutgemm_fwd_slab_kernel<RG, WAVES, true, true>), grid, dim3(WAVES * 64), 0, stream, A,
                           reinterpret_cast<const u32x4*>(E), C, flags, M, K, N, k_quads, cps, 0, 1, grouped, row_blocks, *dq, no_conv);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        // masked codes / entries too large for packed sums: the direct kernel recomputes the sums into C, a pass under the
        // same gate dequantises them
        if ((e = launch_fwd_gated(A, B, C, lut, g, M, K, N, flags + 1, stream, 1)) != hipSuccess) return e;
        return launch_dequant_gated(reinterpret_cast<const float*>(C), dq->xs, dq->wr, dq->tp, dq->za, dq->zw, dq->sa, dq->sw, dq->bias,
                                    dq->out, M, N, dq->L, flags + 1, stream);
    }
    hipLaunchKernelGGL((lutgemm_fwd_slab_kernel<RG, WAVES, true>), grid, dim3(WAVES * 64), 0, stream, A,
                       reinterpret_cast<const u32x4*>(E), C, flags, M, K, N, k_quads, cps, zs > 1 ? 1 : 0, out_f32, grouped, row_blocks, none,
                       no_conv);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // (partial sums over a split K met as integers: converted before the fall-back, which stores floats itself)
    if (zs > 1 && out_f32) {
        e = launch_u32_to_f32(C, (size_t)M * N, stream);
        if (e != hipSuccess) return e;
    }
    // (the fall-back for the masked code of a 7-bit operand and for tables whose entries do not fit packed sums)
    return launch_fwd_gated(A, B, C, lut, g, M, K, N, flags + 1, stream, out_f32);
}

}  // namespace amr
