// Backward LUT-GEMM with float32 gradient tables, gfx950.
//
//   gA[m,k] = scale * sum_n gC[m,n] * Gx[A[m,k]][B[k,n]]     (lutgemm_gradA_f32tab_kernel)
//   gB[k,n] = scale * sum_m Gy[A[m,k]][B[k,n]] * gC[m,n]     (lutgemm_gradB_f32tab_kernel)
//
// The same sums as ApproxGemmBackwardKernelForGA / ...ForGB (self_ops/src/approx_gemm_backward.cu:21-258 and
// :269-492) with the table entries given as float32 (unrounded slopes) instead of int16 = round(16 x slope), and the
// caller's scale in place of FACTOR (self_ops/src/approx_mult.h:41).  Tables keep the reference's padded geometry
// (self_ops/src/approx_mult.h:12-40), four bytes per entry.
//
// Both kernels are the "uniform-row gather" of lutgemm_bwd.hip: one operand code is wave-uniform per gather and picks
// the table row, the lanes' own codes pick the entry inside the row.  What is new is the size of the table: a 7-bit
// float table (67 KB) fits the LDS of a workgroup, an 8-bit one (265 KB) does not fit the 160 KB of a CU.  It is
// split along the uniform operand into `passes` bands of `rows_pp` rows (8 bit: 2 x 129 rows = 133 KB): the workgroup
// stages band 0, walks its whole reduction, stages band 1 and walks it again; the accumulators stay in registers
// across the bands, the codes are read once per band.  A gather whose uniform code lies outside the staged band is
// not skipped by a branch (every conditional read would have to be waited for where its branch ends, one LDS latency
// per gather, and the band tests are a dozen scalar instructions per gather): its row index is clamped to a row of
// zeros staged behind the band (one s_min_u32), so that it adds 0 x gC -- the reads of a row stay in flight together.
// (For a non-finite gC value that product is NaN where the reference, which has the whole table, adds nothing.)
#include "amr_common.h"

namespace amr {

__global__ void reduce_partials_kernel(const float* __restrict__ partial, float* __restrict__ out, size_t count, int splits);

// ------------------------------------------------------------------------------------------ gradB
// Lanes own columns n, the uniform operand is a = A[m,k]; band p holds table rows a in [p*rows_pp, (p+1)*rows_pp).
template <int KT, int WAVES, bool SPLIT>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_gradB_f32tab_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ out,
    const float* __restrict__ lut, int n_rows, int cols, int rows_pp, int passes, int M, int K, int N, int m_chunk,
    float scale, const uint32_t* __restrict__ gate) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (gate != nullptr && *gate == 0u) return;   // queued as a fallback that turned out not to be needed
    const int wave = uniform(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int k0 = (blockIdx.y * WAVES + wave) * KT;
    const bool active = k0 < K;            // idle waves still take part in the barriers between bands
    const int n = blockIdx.x * 64 + lane;
    const int nc = min(n, N - 1);
    const int mb = blockIdx.z * m_chunk;
    const int me = min(M, mb + m_chunk);
    const uint32_t row_bytes = (uint32_t)cols * 4u;

    constexpr int DW = KT / 4;        // code dwords per row in this k tile
    constexpr int RPL = 64 / DW;      // rows covered by one loader instruction
    const int ldw = lane % DW;
    const int lrow = lane / DW;

    uint32_t boff[KT];
#pragma unroll
    for (int kk = 0; kk < KT; ++kk) boff[kk] = 4u * (uint32_t)B[(size_t)min(k0 + kk, K - 1) * N + nc];
    // Sums of blocks of kBlockTrips * RPL rows are added to a second set of accumulators: a chunk of tens of thousands of rows
    // (the gated launch behind an expanded-table kernel has no M split) then loses no more digits than a split sum.
    constexpr int kBlockTrips = 16;
    float acc[KT], tot[KT];
#pragma unroll
    for (int kk = 0; kk < KT; ++kk) acc[kk] = tot[kk] = 0.f;

    for (int p = 0; p < passes; ++p) {
        const int lo = p * rows_pp;
        const uint32_t nr = (uint32_t)min(rows_pp, n_rows - lo);
        if (p) __syncthreads();
        {
            float* s = reinterpret_cast<float*>(smem);
            const float* src = lut + (size_t)lo * cols;
            const int count = (int)nr * cols;
            stage_table_dwords<WAVES * 64>(s, src, count);
            if (SPLIT)
                for (int i = threadIdx.x; i < cols; i += WAVES * 64) s[count + i] = 0.f;      // the row of zeros behind the band
        }
        __syncthreads();
        if (!active) continue;
        int trips = 0;
        for (int m = mb; m < me; m += RPL) {
            const int r = min(m + lrow, me - 1);
            const uint32_t a4 = load_codes4_clamped(A + (size_t)r * K, k0 + 4 * ldw, K);
            float g[RPL];
#pragma unroll
            for (int i = 0; i < RPL; ++i) g[i] = (m + i < me) ? gC[(size_t)(m + i) * N + nc] : 0.f;
#pragma unroll
            for (int i = 0; i < RPL; ++i) {
                float t[KT];
#pragma unroll
                for (int d = 0; d < DW; ++d) {
                    const uint32_t aw = __builtin_amdgcn_readlane(a4, i * DW + d);
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) {
                        uint32_t rel = ((aw >> (8 * kk)) & 0xffu) - (uint32_t)lo;    // wave-uniform; below the band: wraps to a huge value
                        if (SPLIT) rel = min(rel, nr);                                // outside the band: the row of zeros
                        t[4 * d + kk] = *reinterpret_cast<const float*>(smem + rel * row_bytes + boff[4 * d + kk]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 0; kk < KT; ++kk) acc[kk] = __builtin_fmaf(t[kk], g[i], acc[kk]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (++trips == kBlockTrips) {     // (wave-uniform) a block of rows is done: its sums join the totals
                trips = 0;
#pragma unroll
                for (int kk = 0; kk < KT; ++kk) {
                    tot[kk] += acc[kk];
                    acc[kk] = 0.f;
                }
            }
        }
    }
    if (active && n < N) {
        float* o = out + (size_t)blockIdx.z * K * N;
#pragma unroll
        for (int kk = 0; kk < KT; ++kk)
            if (k0 + kk < K) o[(size_t)(k0 + kk) * N + n] = (tot[kk] + acc[kk]) * scale;
    }
}

// ------------------------------------------------------------------------------------------ gradA
// Lanes own rows m, the uniform operand is b = B[k,n]; the table is transposed while it is staged, T[b - lo][a], so that
// the uniform code again picks the row; band p holds b in [p*rows_pp, (p+1)*rows_pp).
template <int KT, int RM, int WAVES, bool VEC, bool SPLIT>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_gradA_f32tab_kernel(
    const float* __restrict__ gC, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ gA,
    const float* __restrict__ lut, int n_rows, int cols, int rows_pp, int passes, int M, int K, int N, float scale,
    const uint32_t* __restrict__ gate, int rows_per_image, int vec_store) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (gate != nullptr && *gate == 0u) return;
    const int wave = uniform(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    int tile_k, tile_m;
    folded_tile_xy((K + KT - 1) / KT, &tile_k, &tile_m);
    const int k0 = tile_k * KT;
    const int m0 = (tile_m * WAVES + wave) * (64 * RM);
    const bool active = m0 < M;
    const uint32_t trow_bytes = (uint32_t)cols * 4u;

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
                aoff[r][4 * d + kk] = 4u * ((a4 >> (8 * kk)) & 0xffu);
                acc[r][4 * d + kk] = 0.f;
            }
        }
    }
    // Loader lane kk (< KT) carries four B codes of row k0+kk; rows beyond K are clamped (never stored).
    const uint8_t* brow = B + (size_t)min(k0 + (lane % KT), K - 1) * N;

    for (int p = 0; p < passes; ++p) {
        const int lo = p * rows_pp;
        const uint32_t nr = (uint32_t)min(rows_pp, n_rows - lo);
        if (p) __syncthreads();
        {
            // entry (a, b) of the row-major table goes to T[b - lo][a], T row stride = cols entries
            float* t32 = reinterpret_cast<float*>(smem);
            const int total = n_rows * (int)nr;
            const float inv_nr = 1.0f / (float)nr;
            constexpr int U = 8, THREADS = WAVES * 64;
            for (int base = 0; base < total; base += U * THREADS) {      // eight loads of a thread in flight
                float v[U];
                int a[U], bb[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int i = min(base + u * THREADS + (int)threadIdx.x, total - 1);
                    a[u] = div_small(i, (int)nr, inv_nr);
                    bb[u] = i - a[u] * (int)nr;
                    v[u] = lut[(size_t)a[u] * cols + lo + bb[u]];
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (base + u * THREADS + (int)threadIdx.x < total) t32[bb[u] * cols + a[u]] = v[u];
            }
            if (SPLIT)
                for (int i = threadIdx.x; i < cols; i += WAVES * 64) t32[(int)nr * cols + i] = 0.f;      // the row of zeros behind the band
        }
        __syncthreads();
        if (!active) continue;
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
                    uint32_t rel = ((bw >> (8 * j)) & 0xffu) - (uint32_t)lo;    // wave-uniform; below the band: wraps to a huge value
                    if (SPLIT) rel = min(rel, nr);                               // outside the band: the row of zeros
#pragma unroll
                    for (int r = 0; r < RM; ++r) t[r][kk] = *reinterpret_cast<const float*>(smem + rel * trow_bytes + aoff[r][kk]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 0; kk < KT; ++kk)
#pragma unroll
                    for (int r = 0; r < RM; ++r) acc[r][kk] = __builtin_fmaf(g[r][j], t[r][kk], acc[r][kk]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    if (!active) return;
#pragma unroll
    for (int r = 0; r < RM; ++r) {
        const int m = m0 + lane + 64 * r;
        if (m < M && rows_per_image > 0) {
            // image-major transposed output gA_T[m / L][k][m % L] (L = rows_per_image)
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
                    if (k0 + 4 * d < K) {
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
constexpr size_t kF32TabLdsCap = 140 * 1024;   // table band per workgroup (the 8-bit band of 129 rows needs 133 128 bytes)

// Bands of the table along the uniform operand: all n_rows rows when they fit, else the fewest equal bands that do.
static void f32tab_bands(const LutGeom& g, int* rows_pp, int* passes) {
    const size_t row = (size_t)g.cols * 4;
    int p = 1;
    while ((size_t)((g.rows + p - 1) / p) * row > kF32TabLdsCap) ++p;
    *passes = p;
    *rows_pp = (g.rows + p - 1) / p;
}

template <typename Kern>
static hipError_t allow_big_lds(Kern kern, std::atomic<uint64_t>* done) {
    return allow_full_lds(reinterpret_cast<const void*>(kern), *done);
}

int gradB_direct_splits(int M, int K, int N, int n_cu, int waves, int wgs_per_cu);

// workspace: room for the partial sums (gradB_workspace_bytes), or nullptr: no split over M.
hipError_t launch_gradB_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut, const LutGeom& g,
                               int M, int K, int N, float scale, void* workspace, int n_cu, hipStream_t stream,
                               const uint32_t* gate) {
    constexpr int KT = 16;
    int rows_pp, passes;
    f32tab_bands(g, &rows_pp, &passes);
    const size_t lds = (size_t)(rows_pp + 1) * g.cols * 4;      // + the row of zeros
    const bool wide = passes > 1 || lds > 80 * 1024;            // one 1024-thread workgroup per CU
    const int splits = workspace ? gradB_direct_splits(M, K, N, n_cu, wide ? 16 : 4, wide ? 1 : 2) : 1;
    int m_chunk = (M + splits - 1) / splits;
    m_chunk = (m_chunk + 15) & ~15;
    const int zs = (M + m_chunk - 1) / m_chunk;
    float* out = zs > 1 ? reinterpret_cast<float*>(workspace) : gB;
    const int ktiles = (K + KT - 1) / KT;
    hipError_t e;
    if (wide) {
        // one 1024-thread workgroup per CU shares the staged band
        static std::atomic<uint64_t> done{0};
        auto kern = lutgemm_gradB_f32tab_kernel<KT, 16, true>;
        if ((e = allow_big_lds(kern, &done)) != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((N + 63) / 64, (ktiles + 15) / 16, zs), dim3(1024), lds, stream, gC, A, B, out, lut, g.rows,
                           g.cols, rows_pp, passes, M, K, N, m_chunk, scale, gate);
    } else {
        static std::atomic<uint64_t> done{0};
        auto kern = lutgemm_gradB_f32tab_kernel<KT, 4, false>;
        if ((e = allow_big_lds(kern, &done)) != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((N + 63) / 64, (ktiles + 3) / 4, zs), dim3(256), lds, stream, gC, A, B, out, lut, g.rows,
                           g.cols, rows_pp, passes, M, K, N, m_chunk, scale, gate);
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

template <int KT, int RM, int WAVES, bool VEC, bool SPLIT>
static hipError_t launch_gradA_f32tab_t(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                                        const LutGeom& g, int rows_pp, int passes, int M, int K, int N, float scale,
                                        hipStream_t stream, const uint32_t* gate, int rows_per_image) {
    const int vec_store = ((K & 3) == 0) && (((uintptr_t)gA & 15) == 0);
    auto kern = lutgemm_gradA_f32tab_kernel<KT, RM, WAVES, VEC, SPLIT>;
    static std::atomic<uint64_t> done{0};
    hipError_t e = allow_big_lds(kern, &done);
    if (e != hipSuccess) return e;
    const int rows_per_wg = 64 * RM * WAVES;
    dim3 grid((unsigned)((K + KT - 1) / KT) * (unsigned)((M + rows_per_wg - 1) / rows_per_wg));   // k tiles x row blocks, folded into x
    hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), (size_t)(rows_pp + 1) * g.cols * 4, stream, gC, A, B, gA, lut, g.rows, g.cols, rows_pp,
                       passes, M, K, N, scale, gate, rows_per_image, vec_store);
    return hipGetLastError();
}

hipError_t launch_gradA_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut, const LutGeom& g,
                               int M, int K, int N, float scale, int n_cu, hipStream_t stream, const uint32_t* gate,
                               int rows_per_image) {
    constexpr int KT = 16;
    int rows_pp, passes;
    f32tab_bands(g, &rows_pp, &passes);
    const bool vec = ((N & 3) == 0) && (((uintptr_t)gC & 15) == 0);   // rows of gC are read 16 bytes at a time
    const int ktiles = (K + KT - 1) / KT;
    const bool wide = passes > 1 || (size_t)rows_pp * g.cols * 4 > 80 * 1024;
    if (wide && M <= 1024) {
        // One block of rows: the k tiles are the only workgroups, one per CU at a time, and a launch lasts (rounds of n_cu
        // workgroups) x (k per tile): 16, 20 or 24 k per tile, whichever makes that smallest (4608 k: 231 tiles of 20 are one
        // round on 256 CUs, 288 tiles of 16 two).
        auto cost = [&](int kt) { return ((long)((K + kt - 1) / kt) + n_cu - 1) / n_cu * kt; };
        int kt = 16;
        if (cost(20) < cost(kt)) kt = 20;
        if (cost(24) < cost(kt)) kt = 24;
#define AMR_GA8F_CASE(t)                                                                                                                            \
    if (kt == t)                                                                                                                                    \
        return vec ? launch_gradA_f32tab_t<t, 1, 16, true, true>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image)  \
                   : launch_gradA_f32tab_t<t, 1, 16, false, true>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image);
        AMR_GA8F_CASE(20)
        AMR_GA8F_CASE(24)
        AMR_GA8F_CASE(16)
#undef AMR_GA8F_CASE
    }
    if (wide) {
        // one 1024-thread workgroup per CU shares the staged band; two rows per lane (half the scalar work per gather) unless
        // one row per lane needs fewer (rounds of n_cu workgroups) x (rows per workgroup)
        const long cost2 = (((long)ktiles * ((M + 2047) / 2048) + n_cu - 1) / n_cu) * 2048;
        const long cost1 = (((long)ktiles * ((M + 1023) / 1024) + n_cu - 1) / n_cu) * 1024;
        if (cost2 <= cost1)
            return vec ? launch_gradA_f32tab_t<KT, 2, 16, true, true>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image)
                       : launch_gradA_f32tab_t<KT, 2, 16, false, true>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image);
        return vec ? launch_gradA_f32tab_t<KT, 1, 16, true, true>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image)
                   : launch_gradA_f32tab_t<KT, 1, 16, false, true>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image);
    }
    // Two rows per lane amortise the scalar work per gather; one when that would leave CUs idle.
    const long wg2 = (long)ktiles * ((M + 511) / 512);
    if (wg2 >= 2L * n_cu) {
        return vec ? launch_gradA_f32tab_t<KT, 2, 4, true, false>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image)
                   : launch_gradA_f32tab_t<KT, 2, 4, false, false>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image);
    }
    return vec ? launch_gradA_f32tab_t<KT, 1, 4, true, false>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image)
               : launch_gradA_f32tab_t<KT, 1, 4, false, false>(gC, A, B, gA, lut, g, rows_pp, passes, M, K, N, scale, stream, gate, rows_per_image);
}

}  // namespace amr
