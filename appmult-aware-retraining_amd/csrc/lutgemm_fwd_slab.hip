// Forward LUT-GEMM for large M on gfx950: "expanded-table" formulation (7-bit tables and narrower).
//
// Same result as lutgemm_fwd_kernel (and as the reference's ApproxGemmForwardKernel,
// self_ops/src/approx_gemm_forward.cu:45-229), different work decomposition:
//
//   step 1  expand_fwd_kernel:  E[k][a][n] = lut[a][B[k,n]] for every code a      (K * 2^b * N gathers)
//   step 2  lutgemm_fwd_slab_kernel:  C[m, :] = sum_k E[k][A[m,k]][:]             (M * K row additions)
//
// Step 1 costs 2^b / M of the M*K*N gathers of the direct kernel.  Step 2 never gathers single
// entries: for one (m,k) a lane reads FOUR adjacent uint16 entries of row a = A[m,k] with one
// ds_read_b64.  64-bit LDS reads move 256 B/clk/CU on gfx950, twice the 32 lanes/clk of 16/32-bit
// gathers, and they are conflict-free by construction here, so the LDS no longer limits the kernel.
//
// Layout of E in HBM (uint16): E[n_tile][k_pair][a (128 rows)][half (k parity)][64 columns]; one
// (n_tile, k_pair) block is 32 KB, a table row of one k is 128 B and the two k of a pair share a
// 256 B line.  A workgroup (16 waves) owns 512 rows of A and one 64-column tile, and walks K in
// chunks of 4 (two k-pairs = 64 KB) that are double buffered in LDS and filled by LDS-direct loads.
// Lane l of a wave: row slot rs = l/16 (4 rows per instruction), column group cg = l%16 (4 columns).
// Odd row slots visit the two k of a pair in swapped order, so that in every instruction two slots
// read the low 128 B half of their 256 B line and two the high half: each half lives in its own
// 32 banks, which makes every read conflict-free.
// The LDS address (buffer<<16 | a<<8 | half<<7 | cg<<3) is assembled from the code byte and a
// per-lane constant by ONE v_perm_b32.  That needs a < 128: a 7-bit operand holding the masked code
// 128 (zero contribution) is detected, flags[1] is raised and the direct kernel, queued behind this
// one and gated on that flag, recomputes C.
// Accumulation: when 4 * max(lut) < 65536 (flag written by the expand kernel) the four k of a chunk
// are first added as packed uint16 pairs (v_pk_add_u16) and widened to 32 bit once per chunk.
#include "amr_common.h"

namespace amr {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // native 16-byte vector (stays in registers)

constexpr int kSlabRows = 128;                       // rows per (n_tile, k_pair) block
constexpr int kSlabPairBytes = kSlabRows * 256;      // 32 KB
constexpr int kSlabChunkPairs = 2;                   // k-pairs per LDS buffer (4 k)
constexpr int kSlabChunkBytes = kSlabChunkPairs * kSlabPairBytes;   // 64 KB

// ------------------------------------------------------------------------------------------ expand
// grid: (n_tiles, ceil(k_pairs_padded / PAIRS_PER_WG)); 256 threads.  k_pairs_padded is a multiple of
// kSlabChunkPairs; pairs / columns beyond K / N are written as zeros.  Block (0,0) also writes
// flags[0] = max over the table (used to pick the packed accumulation path).
constexpr int kExpandPairsPerWg = 4;

__global__ __launch_bounds__(256) void expand_fwd_kernel(const uint8_t* __restrict__ B,
                                                         const uint32_t* __restrict__ lut32, int lut_dwords,
                                                         int lut_cols, int n_codes, uint16_t* __restrict__ E,
                                                         uint32_t* __restrict__ flags, int K, int N, int k_pairs_padded) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* s32 = reinterpret_cast<uint32_t*>(smem);
    uint32_t mx = 0;
    for (int i = threadIdx.x; i < lut_dwords; i += 256) {
        const uint32_t v = lut32[i];
        s32[i] = v;
        mx = max(mx, max(v & 0xffffu, v >> 16));
    }
    __syncthreads();
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        // wave-level max, then one atomicMax per wave (flags[0] is zeroed by the host before launch)
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o));
        if ((threadIdx.x & 63) == 0) atomicMax(&flags[0], mx);
    }
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = blockIdx.x * 64 + lane;
    for (int pp = 0; pp < kExpandPairsPerWg; ++pp) {
        const int kp = blockIdx.y * kExpandPairsPerWg + pp;
        if (kp >= k_pairs_padded) break;
        uint16_t* blk = E + ((size_t)blockIdx.x * k_pairs_padded + kp) * (kSlabPairBytes / 2);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = 2 * kp + h;
            const bool live = (k < K) && (n < N);
            const int b = live ? (int)B[(size_t)k * N + n] : 0;
            for (int a = wave; a < kSlabRows; a += 4) {
                uint16_t v = 0;
                if (live && a < n_codes) v = s16[a * lut_cols + b];
                blk[a * 128 + h * 64 + lane] = v;
            }
        }
    }
}

// Copies one 64 KB chunk of E from global memory straight into LDS (global_load_lds_dwordx4: the data
// of lane l lands at the wave-uniform LDS base + 16*l; no VGPRs are held while the load is in flight).
// Completion is tracked by vmcnt; the caller waits for vmcnt(0) before the barrier.
template <int THREADS>
__device__ __forceinline__ void slab_copy_chunk(const u32x4* src, unsigned char* lds_dst, int tid, int wave) {
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    constexpr int CPT = kSlabChunkBytes / 16 / THREADS;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const u32x4* g = src + tid + THREADS * i;
        unsigned char* l = lds_dst + (size_t)(THREADS * i + wave * 64) * 16;
        __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)l, 16, 0, 0);
    }
}

// Eight 64-bit LDS reads (two row groups x four k) issued back to back, NOT waited for.  Inline
// assembly, for two reasons: the reads of the chunk being consumed must not wait for the LDS-direct
// loads of the NEXT chunk (the compiler cannot tell the two apart, same LDS array), and the reads of
// block b+1 are issued before block b is consumed (software pipelining with explicit counters).
__device__ __forceinline__ void slab_issue8(uint64_t (&d)[8], const uint32_t (&addr)[8]) {
    asm volatile(
        "ds_read_b64 %0, %8\n ds_read_b64 %1, %9\n ds_read_b64 %2, %10 offset:32768\n ds_read_b64 %3, %11 offset:32768\n"
        "ds_read_b64 %4, %12\n ds_read_b64 %5, %13\n ds_read_b64 %6, %14 offset:32768\n ds_read_b64 %7, %15 offset:32768"
        : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3]), "=&v"(d[4]), "=&v"(d[5]), "=&v"(d[6]), "=&v"(d[7])
        : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3]), "v"(addr[4]), "v"(addr[5]), "v"(addr[6]), "v"(addr[7])
        : "memory");
}

// Waits until at most PENDING LDS operations are outstanding.  The eight results are passed through
// as in/out operands so that every use of them is ordered after the wait.
template <int PENDING>
__device__ __forceinline__ void slab_wait8(uint64_t (&d)[8]) {
    asm volatile("s_waitcnt lgkmcnt(%8)"
                 : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]), "+v"(d[4]), "+v"(d[5]), "+v"(d[6]), "+v"(d[7])
                 : "n"(PENDING)
                 : "memory");
}

template <int RG>
__device__ __forceinline__ void slab_addr8(uint32_t (&addr)[8], const uint32_t (&a_cur)[RG], int i, uint32_t b0,
                                           uint32_t b1, const uint32_t (&sel)[4]) {
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) addr[4 * g + j] = __builtin_amdgcn_perm(a_cur[i + g], (j & 1) ? b1 : b0, sel[j]);
}

// One chunk (4 k) for all RG row groups of a lane; every code is < 128.
template <int RG, bool PACKED>
__device__ __forceinline__ void slab_chunk_fast(uint32_t (&acc)[RG][4], const uint32_t (&a_cur)[RG], uint32_t b0,
                                                uint32_t b1, const uint32_t (&sel)[4]) {
    static_assert(RG % 2 == 0, "row groups are processed in pairs");
    constexpr int NB = RG / 2;
    uint64_t d[2][8];
    {
        uint32_t addr[8];
        slab_addr8<RG>(addr, a_cur, 0, b0, b1, sel);
        slab_issue8(d[0], addr);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int i = 2 * b;
        if (b + 1 < NB) {
            uint32_t addr[8];
            slab_addr8<RG>(addr, a_cur, i + 2, b0, b1, sel);
            slab_issue8(d[(b + 1) & 1], addr);
            slab_wait8<8>(d[b & 1]);
        } else {
            slab_wait8<0>(d[b & 1]);
        }
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lo[j] = (uint32_t)d[b & 1][4 * g + j];
                hi[j] = (uint32_t)(d[b & 1][4 * g + j] >> 32);
            }
            if (PACKED) {
                typedef unsigned short us2 __attribute__((ext_vector_type(2)));
                const us2 l = (__builtin_bit_cast(us2, lo[0]) + __builtin_bit_cast(us2, lo[1])) +
                              (__builtin_bit_cast(us2, lo[2]) + __builtin_bit_cast(us2, lo[3]));
                const us2 h = (__builtin_bit_cast(us2, hi[0]) + __builtin_bit_cast(us2, hi[1])) +
                              (__builtin_bit_cast(us2, hi[2]) + __builtin_bit_cast(us2, hi[3]));
                acc[i + g][0] += l.x;
                acc[i + g][1] += l.y;
                acc[i + g][2] += h.x;
                acc[i + g][3] += h.y;
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i + g][0] += lo[j] & 0xffffu;
                    acc[i + g][1] += lo[j] >> 16;
                    acc[i + g][2] += hi[j] & 0xffffu;
                    acc[i + g][3] += hi[j] >> 16;
                }
            }
        }
        // Pin the accumulation here: an empty volatile asm that "modifies" the eight accumulators cannot
        // be moved across the volatile read blocks, so the sums are not postponed until all reads of
        // the chunk are done (which would keep every result live and overflow the register file).
        asm volatile("" : "+v"(acc[i][0]), "+v"(acc[i][1]), "+v"(acc[i][2]), "+v"(acc[i][3]), "+v"(acc[i + 1][0]),
                          "+v"(acc[i + 1][1]), "+v"(acc[i + 1][2]), "+v"(acc[i + 1][3]));
    }
}

// ------------------------------------------------------------------------------------------ consume
template <int RG, int WAVES, bool PACKED>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_fwd_slab_kernel(
    const uint8_t* __restrict__ A, const u32x4* __restrict__ E, uint32_t* __restrict__ C,
    uint32_t* __restrict__ flags, int M, int K, int N, int k_pairs_padded, int chunks_per_split, int atomic_out) {
    __shared__ __align__(16) unsigned char smem[2 * kSlabChunkBytes];   // static: lets the compiler fold the base address
    constexpr int THREADS = WAVES * 64;
    constexpr int ROWS_PER_WAVE = 4 * RG;
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = tid & 63;
    const int rs = lane >> 4, cg = lane & 15, odd = rs & 1;
    // A wave whose rows would stick out of M is shifted up so that all its rows exist (the host only
    // takes this path for M >= 2048); the rows it then shares with the wave above are not stored twice.
    // (a wave entirely beyond M keeps running, it takes part in the chunk copies, and stores nothing)
    const int m_first = (blockIdx.y * WAVES + wave) * ROWS_PER_WAVE;     // first row this wave must store
    const int m_wave = min(m_first, M - ROWS_PER_WAVE);
    const int total_chunks = k_pairs_padded / kSlabChunkPairs;
    const int c_begin = blockIdx.z * chunks_per_split;
    const int c_end = min(total_chunks, c_begin + chunks_per_split);
    if (c_begin >= c_end) return;
    // Two instances of this kernel are queued for every GEMM; the table maximum (written by the
    // expand kernel) decides which one does the work: 16-bit packed partial sums need 4*max < 65536.
    if ((flags[0] < 16384u) != PACKED) return;

    const u32x4* Eblk = E + ((size_t)blockIdx.x * k_pairs_padded) * (kSlabPairBytes / 16);
    // chunk c_begin -> buffer 0
    slab_copy_chunk<THREADS>(Eblk + (size_t)c_begin * (kSlabChunkBytes / 16), smem, tid, wave);

    // per-lane address pieces; instruction j of a chunk: pair p = j>>1, t = j&1, half h = t ^ odd, k = 2p + h
    uint32_t base[2], sel[4];
#pragma unroll
    for (int t = 0; t < 2; ++t) base[t] = (uint32_t)(((t ^ odd) << 7) | (cg << 3));
#pragma unroll
    for (int j = 0; j < 4; ++j) sel[j] = 0x0c020000u | ((uint32_t)(4 + (j & 2) + ((j & 1) ^ odd)) << 8);

    uint32_t acc[RG][4];
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[i][c] = 0u;

    // Row group i of this lane is row m_wave + rs + 4 i: byte offset off0 + i * 4K, i.e. a per-lane
    // 32-bit offset plus a wave-uniform term (the host only takes this path when M*K < 2^31).
    const uint32_t off0 = (uint32_t)(m_wave + rs) * (uint32_t)K;
    const uint32_t row_step = 4u * (uint32_t)K;

    uint32_t seen = 0;   // OR of every code dword this lane consumed
    uint32_t a_cur[RG];
    {
        // The last chunk may stick out of K: read the last 4 codes of the row and shift, so the load
        // stays inside the row; the surplus positions become code 0 and meet all-zero rows of E.
        const int k0 = c_begin * 4;
        const int koff = min(k0, K - 4), sh = 8 * (k0 - koff);
#pragma unroll
        for (int i = 0; i < RG; ++i) a_cur[i] = load_u32_unaligned(A + ((uint32_t)koff + (uint32_t)i * row_step) + off0) >> sh;
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
    __syncthreads();

    for (int c = c_begin; c < c_end; ++c) {
        const int buf = (c - c_begin) & 1;
        const bool more = (c + 1 < c_end);
        uint32_t a_nxt[RG];
        int sh_nxt = 0;
        if (more) {
            // the next chunk streams into the other buffer while this one is consumed
            slab_copy_chunk<THREADS>(Eblk + (size_t)(c + 1) * (kSlabChunkBytes / 16), smem + (size_t)(buf ^ 1) * kSlabChunkBytes, tid, wave);
            const int k1 = (c + 1) * 4;
            const int koff = min(k1, K - 4);
            sh_nxt = 8 * (k1 - koff);
#pragma unroll
            for (int i = 0; i < RG; ++i) a_nxt[i] = load_u32_unaligned(A + ((uint32_t)koff + (uint32_t)i * row_step) + off0);
        }
        const uint32_t bsel = (uint32_t)buf << 16;
        const uint32_t b0 = base[0] | bsel, b1 = base[1] | bsel;
#pragma unroll
        for (int i = 0; i < RG; ++i) seen |= a_cur[i];
        slab_chunk_fast<RG, PACKED>(acc, a_cur, b0, b1, sel);
        if (more) {
#pragma unroll
            for (int i = 0; i < RG; ++i) a_cur[i] = a_nxt[i] >> sh_nxt;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): the LDS-direct loads of the next chunk have landed
        __syncthreads();
    }

    // A code with bit 7 set (the masked code 128 of a 7-bit table) cannot be addressed by this kernel:
    // raise flags[1]; the host has queued the direct kernel behind this one, gated on that flag.
    if (__builtin_amdgcn_ballot_w64((seen & 0x80808080u) != 0) != 0) {
        if (lane == 0) atomicOr(&flags[1], 1u);
    }
    const int n = blockIdx.x * 64 + 4 * cg;
#pragma unroll
    for (int i = 0; i < RG; ++i) {
        const int m = m_wave + 4 * i + rs;
        if (m >= m_first) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (n + c < N) {
                    if (atomic_out)
                        atomicAdd(&C[(size_t)m * N + n + c], acc[i][c]);
                    else
                        C[(size_t)m * N + n + c] = acc[i][c];
                }
            }
        }
    }
}

hipError_t launch_fwd_gated(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                            int M, int K, int N, const uint32_t* gate, hipStream_t stream);

// ------------------------------------------------------------------------------------------ host
// Workspace layout: [256 B flags][E].  Returns 0 when the expanded-table path does not apply.
size_t fwd_slab_workspace_bytes(const LutGeom& g, int M, int K, int N) {
    // Worth it when the 2^b/M expansion overhead is small and K is long enough to amortise the extra
    // launches (measured cross-over on MI355X: K around 512).
    if (g.bits > 7 || M < 2048 || K < 512 || (size_t)M * K >= (1ull << 31)) return 0;
    const size_t n_tiles = (N + 63) / 64;
    const size_t kpp = (((size_t)K + 1) / 2 + kSlabChunkPairs - 1) / kSlabChunkPairs * kSlabChunkPairs;
    return 256 + n_tiles * kpp * kSlabPairBytes;
}

hipError_t launch_fwd_slab(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                           int M, int K, int N, int n_cu, void* workspace, hipStream_t stream) {
    const int n_tiles = (N + 63) / 64;
    const int kpp = ((K + 1) / 2 + kSlabChunkPairs - 1) / kSlabChunkPairs * kSlabChunkPairs;
    uint32_t* flags = reinterpret_cast<uint32_t*>(workspace);
    uint16_t* E = reinterpret_cast<uint16_t*>(reinterpret_cast<unsigned char*>(workspace) + 256);
    hipError_t e = hipMemsetAsync(flags, 0, 256, stream);
    if (e != hipSuccess) return e;
    const int lut_dwords = g.rows * g.cols / 2;
    hipLaunchKernelGGL(expand_fwd_kernel, dim3(n_tiles, (kpp + kExpandPairsPerWg - 1) / kExpandPairsPerWg), dim3(256),
                       (size_t)lut_dwords * 4, stream, B, reinterpret_cast<const uint32_t*>(lut), lut_dwords, g.cols,
                       1 << g.bits, E, flags, K, N, kpp);
    e = hipGetLastError();
    if (e != hipSuccess) return e;

    // 512 rows per workgroup
    const int chunks = kpp / kSlabChunkPairs;
    // 16 waves x 32 rows = 512 rows per workgroup (measured best among 256/512/1024-row tilings)
    constexpr int RG = 8, WAVES = 16;
    const int m_tile = WAVES * 4 * RG;
    const long wgs = (long)n_tiles * ((M + m_tile - 1) / m_tile);
    int ksplit = 1;
    if (wgs < n_cu) {
        ksplit = (int)((n_cu + wgs - 1) / wgs);
        const int max_split = chunks / 8 > 0 ? chunks / 8 : 1;     // at least 32 k per workgroup
        if (ksplit > max_split) ksplit = max_split;
    }
    const int cps = (chunks + ksplit - 1) / ksplit;
    const int zs = (chunks + cps - 1) / cps;
    if (zs > 1) {
        e = hipMemsetAsync(C, 0, (size_t)M * N * sizeof(uint32_t), stream);
        if (e != hipSuccess) return e;
    }
    dim3 grid(n_tiles, (M + m_tile - 1) / m_tile, zs);
    // both accumulation flavours are queued; flags[0] (table maximum) decides on the device which one works
    hipLaunchKernelGGL((lutgemm_fwd_slab_kernel<RG, WAVES, true>), grid, dim3(WAVES * 64), 0, stream, A,
                       reinterpret_cast<const u32x4*>(E), C, flags, M, K, N, kpp, cps, zs > 1 ? 1 : 0);
    hipLaunchKernelGGL((lutgemm_fwd_slab_kernel<RG, WAVES, false>), grid, dim3(WAVES * 64), 0, stream, A,
                       reinterpret_cast<const u32x4*>(E), C, flags, M, K, N, kpp, cps, zs > 1 ? 1 : 0);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (g.bits == 7) return launch_fwd_gated(A, B, C, lut, g, M, K, N, flags + 1, stream);
    return hipGetLastError();
}

}  // namespace amr
