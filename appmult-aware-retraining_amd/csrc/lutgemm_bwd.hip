// Backward LUT-GEMM kernels for gfx950.
//
//   gA[m,k] = scale * sum_n gC[m,n] * (float)Gx[A[m,k]][B[k,n]]     (lutgemm_gradA_kernel)
//   gB[k,n] = scale * sum_m (float)Gy[A[m,k]][B[k,n]] * gC[m,n]     (lutgemm_gradB_kernel)
//
// They replace ApproxGemmBackwardKernelForGA / ...ForGB
// (self_ops/src/approx_gemm_backward.cu:21-258 and :269-492); scale is the reference's
// FACTOR = 1/16 (self_ops/src/approx_mult.h:41) applied once per output, which is exact in fp32.
//
// Both kernels use the same "uniform-row gather" as the forward kernel: one operand code is
// wave-uniform per gather, so the 64 lanes read inside one 256-byte (7-bit) table row and bank
// conflicts are at most 2-way for any data.
//   gradB: lanes own columns n (their code b is fixed per k), the uniform operand is a = A[m,k];
//          each wave owns KT values of k, keeps KT fp32 accumulators per lane and walks down a
//          chunk of rows m.  The M reduction is split over blockIdx.z; partial sums go to a
//          workspace and are added in a fixed order by reduce_partials_kernel (deterministic).
//   gradA: lanes own rows m (their code a is fixed per k), the uniform operand is b = B[k,n]; the
//          table is transposed while it is staged into LDS so that the uniform code again selects
//          the row.  Each lane keeps RM x KT accumulators and walks along n; no cross-lane
//          reduction is needed.
#include "amr_common.h"

namespace amr {

// ------------------------------------------------------------------------------------------ gradB
template <int KT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_gradB_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
    float* __restrict__ out, const uint32_t* __restrict__ lut32, int lut_dwords, int row_bytes, int M, int K, int N,
    int m_chunk, float scale, const uint32_t* __restrict__ gate) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (gate != nullptr && *gate == 0u) return;   // queued as a fallback that turned out not to be needed
    stage_table_dwords<WAVES * 64>(smem, lut32, lut_dwords);
    __syncthreads();

    const int wave = uniform(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int k0 = (blockIdx.y * WAVES + wave) * KT;
    if (k0 >= K) return;
    const int n = blockIdx.x * 64 + lane;
    const int nc = min(n, N - 1);
    const int mb = blockIdx.z * m_chunk;
    const int me = min(M, mb + m_chunk);

    constexpr int DW = KT / 4;        // code dwords per row in this k tile
    constexpr int RPL = 64 / DW;      // rows covered by one loader instruction
    // Loader lane -> (row lane / DW, dword lane % DW).  A k tile that sticks out of K is clamped to the
    // last full dword-aligned position inside the row; its surplus accumulators are never stored.
    const int ldw = lane % DW;
    const int lrow = lane / DW;

    uint32_t boff[KT];
#pragma unroll
    for (int kk = 0; kk < KT; ++kk) boff[kk] = 2u * (uint32_t)B[(size_t)min(k0 + kk, K - 1) * N + nc];
    float acc[KT];
#pragma unroll
    for (int kk = 0; kk < KT; ++kk) acc[kk] = 0.f;

    // The codes and gC values of the next RPL rows are loaded while the current ones are consumed (two register sets
    // alternate); without that every trip of a wave pays the memory latency before its first gather.
    auto load_rows = [&](int m, uint32_t& a4, float (&g)[RPL]) __attribute__((always_inline)) {
        const int r = min(m + lrow, me - 1);
        a4 = load_codes4_clamped(A + (size_t)r * K, k0 + 4 * ldw, K);
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            const float v = gC[(size_t)min(m + i, me - 1) * N + nc];
            g[i] = (m + i < me) ? v : 0.f;
        }
    };
    auto consume_rows = [&](uint32_t a4, const float (&g)[RPL]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            float t[KT];
#pragma unroll
            for (int d = 0; d < DW; ++d) {
                const uint32_t aw = __builtin_amdgcn_readlane(a4, i * DW + d);
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    const uint32_t ro = ((aw >> (8 * kk)) & 0xffu) * (uint32_t)row_bytes;
                    t[4 * d + kk] = (float)*reinterpret_cast<const int16_t*>(smem + ro + boff[4 * d + kk]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < KT; ++kk) acc[kk] = __builtin_fmaf(t[kk], g[i], acc[kk]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Sums of blocks of kBlockTrips * 2 * RPL rows are added to a second set of accumulators: a chunk of tens of thousands of
    // rows (the gated launch behind an expanded-table kernel has no M split) then loses no more digits than a split sum.
    constexpr int kBlockTrips = 8;
    float tot[KT];
#pragma unroll
    for (int kk = 0; kk < KT; ++kk) tot[kk] = 0.f;
    {
        uint32_t a4x, a4y;
        float gx[RPL], gy[RPL];
        int m = mb, trips = 0;
        if (m < me) load_rows(m, a4x, gx);
        while (m < me) {
            if (m + RPL < me) load_rows(m + RPL, a4y, gy);
            consume_rows(a4x, gx);
            m += RPL;
            if (m >= me) break;
            if (m + RPL < me) load_rows(m + RPL, a4x, gx);
            consume_rows(a4y, gy);
            m += RPL;
            if (++trips == kBlockTrips) {     // (wave-uniform)
                trips = 0;
#pragma unroll
                for (int kk = 0; kk < KT; ++kk) {
                    tot[kk] += acc[kk];
                    acc[kk] = 0.f;
                }
            }
        }
    }
    if (n < N) {
        float* o = out + (size_t)blockIdx.z * K * N;
#pragma unroll
        for (int kk = 0; kk < KT; ++kk)
            if (k0 + kk < K) o[(size_t)(k0 + kk) * N + n] = (tot[kk] + acc[kk]) * scale;
    }
}

// out[i] = sum_s partial[s][i], s ascending (fixed order -> deterministic).
__global__ void reduce_partials_kernel(const float* __restrict__ partial, float* __restrict__ out, size_t count, int splits) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float s = partial[i];
    int p = 1;
    for (; p + 8 <= splits; p += 8) {      // (eight loads in flight, added in the order of the splits)
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = partial[(size_t)(p + u) * count + i];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += t[u];
    }
    for (; p < splits; ++p) s += partial[(size_t)p * count + i];
    out[i] = s;
}

// ------------------------------------------------------------------------------------------ gradA
// VEC: N % 4 == 0 and gC 16-byte aligned, so the per-lane rows of gC are read 16 bytes at a time; vec_store: K % 4 == 0
// and gA 16-byte aligned, so the per-lane rows of gA are written 16 bytes at a time (a lane owns a row, so every scalar access would
// touch 64 different cache lines per instruction).
template <int KT, int RM, int WAVES, bool VEC>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_gradA_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
    float* __restrict__ gA, const uint16_t* __restrict__ lut, int rows, int cols, int M, int K, int N, float scale,
    const uint32_t* __restrict__ gate, int rows_per_image, int vec_store) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (gate != nullptr && *gate == 0u) return;   // queued as a fallback that turned out not to be needed
    // Transposed staging: entry (a,b) of the row-major table goes to T[b][a], T row stride = cols
    // entries (cols is even, so T rows stay dword aligned).  T needs cols rows of `rows` entries.
    {
        // a dword of the table holds the entries (a, b) and (a, b + 1) (cols is even); eight loads of a thread are in
        // flight before the first entry is stored
        uint16_t* t16 = reinterpret_cast<uint16_t*>(smem);
        const uint32_t* lut32 = reinterpret_cast<const uint32_t*>(lut);
        const int hc = cols >> 1, total = rows * hc;
        const float inv_hc = 1.0f / (float)hc;
        constexpr int U = 8, THREADS = WAVES * 64;
        for (int base = 0; base < total; base += U * THREADS) {
            uint32_t v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = lut32[min(base + u * THREADS + (int)threadIdx.x, total - 1)];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = base + u * THREADS + (int)threadIdx.x;
                if (j < total) {
                    const int a = div_small(j, hc, inv_hc);
                    const int b = 2 * (j - a * hc);
                    t16[b * cols + a] = (uint16_t)v[u];
                    t16[(b + 1) * cols + a] = (uint16_t)(v[u] >> 16);
                }
            }
        }
    }
    __syncthreads();
    const int trow_bytes = cols * 2;

    const int wave = uniform(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    int tile_k, tile_m;
    folded_tile_xy((K + KT - 1) / KT, &tile_k, &tile_m);
    const int k0 = tile_k * KT;
    const int m0 = (tile_m * WAVES + wave) * (64 * RM);
    if (m0 >= M) return;

    int mr[RM];
    uint32_t aoff[RM][KT];
    float acc[RM][KT];
#pragma unroll
    for (int r = 0; r < RM; ++r) {
        mr[r] = min(m0 + lane + 64 * r, M - 1);
        const uint8_t* arow = A + (size_t)mr[r] * K;
#pragma unroll
        for (int d = 0; d < KT / 4; ++d) {
            const uint32_t a4 = load_codes4_clamped(arow, k0 + 4 * d, K);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                aoff[r][4 * d + kk] = 2u * ((a4 >> (8 * kk)) & 0xffu);
                acc[r][4 * d + kk] = 0.f;
            }
        }
    }
    // Loader lane kk (< KT) carries four B codes of row k0+kk; rows beyond K are clamped (never stored).
    const uint8_t* brow = B + (size_t)min(k0 + (lane % KT), K - 1) * N;

    for (int n = 0; n < N; n += 4) {
        const uint32_t b4 = load_codes4_clamped(brow, n, N);
        float g[RM][4];
#pragma unroll
        for (int r = 0; r < RM; ++r) {
            if (VEC) {
                typedef float f32x4 __attribute__((ext_vector_type(4)));
                const f32x4 v = *reinterpret_cast<const f32x4*>(gC + (size_t)mr[r] * N + n);
                g[r][0] = v.x; g[r][1] = v.y; g[r][2] = v.z; g[r][3] = v.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) g[r][j] = (n + j < N) ? gC[(size_t)mr[r] * N + n + j] : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float t[RM][KT];
#pragma unroll
            for (int kk = 0; kk < KT; ++kk) {
                const uint32_t bw = __builtin_amdgcn_readlane(b4, kk);
                const uint32_t ro = ((bw >> (8 * j)) & 0xffu) * (uint32_t)trow_bytes;
#pragma unroll
                for (int r = 0; r < RM; ++r)
                    t[r][kk] = (float)*reinterpret_cast<const int16_t*>(smem + ro + aoff[r][kk]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < RM; ++r)
#pragma unroll
                for (int kk = 0; kk < KT; ++kk) acc[r][kk] = __builtin_fmaf(g[r][j], t[r][kk], acc[r][kk]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int r = 0; r < RM; ++r) {
        const int m = m0 + lane + 64 * r;
        if (m < M && rows_per_image > 0) {
            // image-major transposed output gA_T[m / L][k][m % L] (L = rows_per_image): consecutive lanes hold
            // consecutive rows, so every store instruction writes a contiguous run (the layout col2im wants)
            const int img = m / rows_per_image, l = m - img * rows_per_image;
            float* o = gA + ((size_t)img * K + k0) * rows_per_image + l;
#pragma unroll
            for (int kk = 0; kk < KT; ++kk)
                if (k0 + kk < K) o[(size_t)kk * rows_per_image] = acc[r][kk] * scale;
        } else if (m < M) {
            if (vec_store) {   // K % 4 == 0 and gA 16-byte aligned
                typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
                for (int d = 0; d < KT / 4; ++d) {
                    if (k0 + 4 * d < K) {   // K % 4 == 0: the whole group is inside the row
                        f32x4 v = {acc[r][4 * d] * scale, acc[r][4 * d + 1] * scale, acc[r][4 * d + 2] * scale, acc[r][4 * d + 3] * scale};
                        *reinterpret_cast<f32x4*>(gA + (size_t)m * K + k0 + 4 * d) = v;
                    }
                }
            } else {
#pragma unroll
                for (int kk = 0; kk < KT; ++kk)
                    if (k0 + kk < K) gA[(size_t)m * K + k0 + kk] = acc[r][kk] * scale;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------ host
// M splits of a direct gradB launch whose workgroups have `waves` waves (each owning 16 k) and of which `wgs_per_cu` fit a
// CU at a time.  The grid runs in rounds of n_cu * wgs_per_cu workgroups: the split count is the one whose
// (rounds x rows per workgroup) is smallest -- 290 workgroups on 256 CUs take as long as 512 -- with every split keeping
// at least 32 rows (two trips of a wave's row loop: a wave walks its rows one group of 16 after the other, about 4 us
// per group, so few long chunks leave a small problem latency-bound on a handful of CUs).
int gradB_direct_splits(int M, int K, int N, int n_cu, int waves, int wgs_per_cu) {
    constexpr int KT = 16;
    const long ktiles = (K + KT - 1) / KT;
    const long per_split = (long)((N + 63) / 64) * ((ktiles + waves - 1) / waves);
    const long slots = (long)n_cu * wgs_per_cu;
    long max_s = M / 32;
    if (max_s > 256) max_s = 256;
    if (max_s < 1) max_s = 1;
    long best_s = 1, best_cost = -1;
    for (long sp = 1; sp <= max_s; ++sp) {
        long chunk = (M + sp - 1) / sp;
        chunk = (chunk + 15) & ~15L;
        const long zs = (M + chunk - 1) / chunk;
        const long rounds = (per_split * zs + slots - 1) / slots;
        // (+16 rows: staging the table and the reduction pass over one more partial result)
        const long cost = rounds * (chunk + 16);
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_s = sp; }
    }
    return (int)best_s;
}

// Scratch for the partial sums of the direct gradB kernels: the largest split count any of their launch shapes picks
// (4 waves and four workgroups per CU: int16 tables of at most 7 bits; two per CU: float tables of at most 7 bits; 16 waves,
// one per CU: 8-bit tables).
size_t gradB_workspace_bytes(int M, int K, int N, int n_cu) {
    int s = gradB_direct_splits(M, K, N, n_cu, 4, 4);
    const int s2 = gradB_direct_splits(M, K, N, n_cu, 4, 2), s3 = gradB_direct_splits(M, K, N, n_cu, 16, 1);
    if (s2 > s) s = s2;
    if (s3 > s) s = s3;
    return s > 1 ? (size_t)s * K * N * sizeof(float) : 0;
}

// M splits the direct gradB launch of a table of this width picks (launch_gradB below).
int gradB_direct_splits_for(const LutGeom& g, int M, int K, int N, int n_cu) {
    const bool big = g.bits == 8;
    return gradB_direct_splits(M, K, N, n_cu, big ? 16 : 4, big ? 1 : 4);
}

// workspace: room for the partial sums (gradB_workspace_bytes), or nullptr: no split over M.
hipError_t launch_gradB(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                        const LutGeom& g, int M, int K, int N, float scale, void* workspace, int n_cu,
                        hipStream_t stream, const uint32_t* gate = nullptr, int split_cap = 0) {
    constexpr int KT = 16;
    const int lut_dwords = g.rows * g.cols / 2;
    const size_t lds = (size_t)lut_dwords * 4;
    const bool big = g.bits == 8;
    // split_cap > 0: the most M splits the caller's scratch has room for
    int splits = workspace ? gradB_direct_splits(M, K, N, n_cu, big ? 16 : 4, big ? 1 : 4) : 1;
    if (split_cap > 0 && splits > split_cap) splits = split_cap;
    int m_chunk = (M + splits - 1) / splits;
    m_chunk = (m_chunk + 15) & ~15;
    const int zs = (M + m_chunk - 1) / m_chunk;
    float* out = zs > 1 ? reinterpret_cast<float*>(workspace) : gB;
    const int ktiles = (K + KT - 1) / KT;
    hipError_t e;
    if (big) {
        auto kern = lutgemm_gradB_kernel<KT, 16>;
        static std::atomic<uint64_t> done{0};
        if ((e = allow_full_lds(reinterpret_cast<const void*>(kern), done)) != hipSuccess) return e;
        dim3 grid((N + 63) / 64, (ktiles + 15) / 16, zs);
        hipLaunchKernelGGL(kern, grid, dim3(1024), lds, stream, gC, A, B, out, reinterpret_cast<const uint32_t*>(lut),
                           lut_dwords, g.cols * 2, M, K, N, m_chunk, scale, gate);
    } else {
        auto kern = lutgemm_gradB_kernel<KT, 4>;
        static std::atomic<uint64_t> done{0};
        if ((e = allow_full_lds(reinterpret_cast<const void*>(kern), done)) != hipSuccess) return e;
        dim3 grid((N + 63) / 64, (ktiles + 3) / 4, zs);
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, gC, A, B, out, reinterpret_cast<const uint32_t*>(lut),
                           lut_dwords, g.cols * 2, M, K, N, m_chunk, scale, gate);
    }
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (zs > 1) {
        const size_t count = (size_t)K * N;
        hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream,
                           reinterpret_cast<const float*>(workspace), gB, count, zs);
        e = hipGetLastError();
    }
    return e;
}

template <int KT, int RM, int WAVES, bool VEC>
static hipError_t launch_gradA_t(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                                 const LutGeom& g, int M, int K, int N, float scale, hipStream_t stream, const uint32_t* gate,
                                 int rows_per_image) {
    const int vec_store = ((K & 3) == 0) && (((uintptr_t)gA & 15) == 0);
    auto kern = lutgemm_gradA_kernel<KT, RM, WAVES, VEC>;
    static std::atomic<uint64_t> done{0};
    if (hipError_t ea = allow_full_lds(reinterpret_cast<const void*>(kern), done); ea != hipSuccess) return ea;
    const int rows_per_wg = 64 * RM * WAVES;
    dim3 grid((unsigned)((K + KT - 1) / KT) * (unsigned)((M + rows_per_wg - 1) / rows_per_wg));   // k tiles x row blocks, folded into x
    hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), (size_t)g.cols * g.cols * 2, stream, gC, A, B, gA,
                       reinterpret_cast<const uint16_t*>(lut), g.rows, g.cols, M, K, N, scale, gate, rows_per_image, vec_store);
    return hipGetLastError();
}

hipError_t launch_gradA(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                        const LutGeom& g, int M, int K, int N, float scale, int n_cu, hipStream_t stream,
                        const uint32_t* gate = nullptr, int rows_per_image = 0) {
    constexpr int KT = 16;
    const bool vec = ((N & 3) == 0) && (((uintptr_t)gC & 15) == 0);   // rows of gC are read 16 bytes at a time
    const int ktiles = (K + KT - 1) / KT;
    if (g.bits == 8 && M <= 1024) {
        // One block of rows: the k tiles are the only workgroups, one per CU at a time, and a launch lasts (rounds of n_cu
        // workgroups) x (k per tile).  4608 k in tiles of 16 are 288 workgroups, two rounds on 256 CUs with the second one
        // nearly empty; in tiles of 20 they are 231 workgroups, one round (measured: 0.36 -> 0.2 ms at 512 x 4608 x 512).
        auto cost = [&](int kt) { return ((long)((K + kt - 1) / kt) + n_cu - 1) / n_cu * kt; };
        int kt = 16;
        if (cost(20) < cost(kt)) kt = 20;
        if (cost(24) < cost(kt)) kt = 24;
#define AMR_GA8_CASE(t)                                                                                                  \
    if (kt == t)                                                                                                         \
        return vec ? launch_gradA_t<t, 1, 16, true>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image)  \
                   : launch_gradA_t<t, 1, 16, false>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image);
        AMR_GA8_CASE(20)
        AMR_GA8_CASE(24)
        AMR_GA8_CASE(16)
#undef AMR_GA8_CASE
    }
    if (g.bits == 8) {
        // one 1024-thread workgroup per CU; two rows per lane (half the scalar work per gather) unless one row per lane
        // needs fewer (rounds of n_cu workgroups) x (rows per workgroup)
        const long cost2 = (((long)ktiles * ((M + 2047) / 2048) + n_cu - 1) / n_cu) * 2048;
        const long cost1 = (((long)ktiles * ((M + 1023) / 1024) + n_cu - 1) / n_cu) * 1024;
        if (cost2 <= cost1)
            return vec ? launch_gradA_t<KT, 2, 16, true>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image)
                       : launch_gradA_t<KT, 2, 16, false>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image);
        return vec ? launch_gradA_t<KT, 1, 16, true>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image)
                   : launch_gradA_t<KT, 1, 16, false>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image);
    }
    // Two rows per lane amortise the scalar work per gather; fall back to one when that would leave CUs idle.
    const long wg2 = (long)ktiles * ((M + 511) / 512);
    if (wg2 >= 2L * n_cu) {
        return vec ? launch_gradA_t<KT, 2, 4, true>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image)
                   : launch_gradA_t<KT, 2, 4, false>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image);
    }
    return vec ? launch_gradA_t<KT, 1, 4, true>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image)
               : launch_gradA_t<KT, 1, 4, false>(gC, A, B, gA, lut, g, M, K, N, scale, stream, gate, rows_per_image);
}

// Direct kernel queued behind the expanded-table kernel; it runs only when *gate != 0 (an operand
// held a masked code) and then overwrites the whole result (no M split: no scratch and no second launch; the kernel adds
// its rows in blocks, so the long sum keeps its digits).
hipError_t launch_gradB_gated(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                              const LutGeom& g, int M, int K, int N, float scale, const uint32_t* gate, hipStream_t stream) {
    return launch_gradB(gC, A, B, gB, lut, g, M, K, N, scale, nullptr, 0, stream, gate);
}

}  // namespace amr
