// Forward LUT-GEMM for gfx950:  C[m,n] = sum_k lut[A[m,k]][B[k,n]]  (uint32 accumulate).
//
// Replaces the reference kernel ApproxGemmForwardKernel (self_ops/src/approx_gemm_forward.cu:45-229).
//
// Mapping ("uniform-row gather"): the whole padded table sits in LDS.  A wave owns R rows of A and
// 64*TN columns of B; lane l owns columns n0 + l + 64*j.  For one (row, k) the code a = A[m,k] is
// wave-uniform (read from a loader lane with v_readlane), so all 64 lanes gather inside ONE table
// row, at the byte offset 2*b of their own column code.  A 7-bit row is 64 dwords: lanes that hit
// the same dword are served by one broadcast and the worst bank conflict is 2-way, independent of
// the data; a fully random (a,b) gather would average more than 3-way.
// Accumulators acc[R][TN] stay in VGPRs for the whole K loop; codes are read with unaligned dword
// loads so no alignment of A, K or N is assumed.  Tails are handled by clamping indices (results of
// clamped rows/columns are never stored) and by bounding the k loop, never by pad codes, so the
// same code serves 8-bit tables whose codes fill the whole byte.
#include "amr_common.h"

namespace amr {

hipError_t launch_zero_u32(void* p, size_t n_dwords, hipStream_t stream);
hipError_t launch_u32_to_f32(void* p, size_t n_dwords, hipStream_t stream);

// out_f32: C receives the sums converted to float32 (what the reference's callers do with the result at once,
// self_ops/ops_py/approx_ops.py:569), not the uint32 sums.
template <int R, int TN, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void lutgemm_fwd_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint32_t* __restrict__ C,
    const uint32_t* __restrict__ lut32, int lut_dwords, int row_bytes, int M, int K, int N, int k_chunk,
    int atomic_out, const uint32_t* __restrict__ gate, int out_f32) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (gate != nullptr && *gate == 0u) return;   // queued as a fallback that turned out not to be needed
    stage_table_dwords<WAVES * 64>(smem, lut32, lut_dwords);
    __syncthreads();

    const int wave = uniform(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    int tile_n, tile_m;
    folded_tile_xy((N + 64 * TN - 1) / (64 * TN), &tile_n, &tile_m);
    const int m0 = (tile_m * WAVES + wave) * R;
    if (m0 >= M) return;
    const int n0 = tile_n * (64 * TN);
    const int kb = blockIdx.z * k_chunk;
    const int ke = min(K, kb + k_chunk);
    if (kb >= ke) return;

    constexpr int SPL = 64 / R;  // k-steps (of 4 codes) covered by one loader instruction
    const int lrow = min(m0 + (lane % R), M - 1);
    const uint8_t* arow = A + (size_t)lrow * K;
    const int lstep = lane / R;

    int col[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) col[j] = min(n0 + lane + 64 * j, N - 1);

    uint32_t acc[R][TN];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0u;

    // Main loop: full groups of 4*SPL codes per row, no conditionals inside.
    int k = kb;
    for (; k + 4 * SPL <= ke; k += 4 * SPL) {
        const uint32_t a4 = load_u32_unaligned(arow + k + 4 * lstep);
#pragma unroll
        for (int s = 0; s < SPL; ++s) {
            const int ks = k + 4 * s;
            uint32_t boff[4][TN];
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int j = 0; j < TN; ++j) boff[kk][j] = 2u * (uint32_t)B[(size_t)(ks + kk) * N + col[j]];
            // Gathers are issued in batches of RB rows x 4 codes x TN columns before any result
            // is consumed, so that each wave keeps many LDS reads in flight.
            constexpr int RB = (TN >= 4) ? 1 : (TN == 2 ? 2 : 4);
#pragma unroll
            for (int i0 = 0; i0 < R; i0 += RB) {
                uint32_t t[RB][4][TN];
#pragma unroll
                for (int i = 0; i < RB; ++i) {
                    const uint32_t aw = __builtin_amdgcn_readlane(a4, s * R + i0 + i);
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) {
                        const uint32_t ro = ((aw >> (8 * kk)) & 0xffu) * (uint32_t)row_bytes;
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            t[i][kk][j] = *reinterpret_cast<const uint16_t*>(smem + ro + boff[kk][j]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i0 + i][j] += (t[i][0][j] + t[i][1][j]) + (t[i][2][j] + t[i][3][j]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // Tail: fewer than 4*SPL codes left, one k at a time (lane i < R carries the code of row i).
    for (; k < ke; ++k) {
        const uint32_t a1 = arow[k];
        uint32_t boff1[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) boff1[j] = 2u * (uint32_t)B[(size_t)k * N + col[j]];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const uint32_t ro = (uint32_t)__builtin_amdgcn_readlane(a1, i) * (uint32_t)row_bytes;
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] += *reinterpret_cast<const uint16_t*>(smem + ro + boff1[j]);
        }
    }

#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int m = m0 + i;
        if (m >= M) break;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + lane + 64 * j;
            if (n < N) {
                if (atomic_out)
                    atomicAdd(&C[(size_t)m * N + n], acc[i][j]);
                else if (out_f32)
                    C[(size_t)m * N + n] = __float_as_uint((float)acc[i][j]);
                else
                    C[(size_t)m * N + n] = acc[i][j];
            }
        }
    }
}

template <int R, int TN, int WAVES>
static hipError_t launch_fwd_t(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                               int M, int K, int N, int ksplit, hipStream_t stream, const uint32_t* gate = nullptr, int out_f32 = 0) {
    const int lut_dwords = g.rows * g.cols / 2;  // rows*cols is even for every supported bit-width
    const size_t lds = (size_t)lut_dwords * 4;
    auto kern = lutgemm_fwd_kernel<R, TN, WAVES>;
    static std::atomic<uint64_t> attr_done{0};
    if (hipError_t ea = allow_full_lds(reinterpret_cast<const void*>(kern), attr_done); ea != hipSuccess) return ea;
    const int k_chunk = ((K + ksplit - 1) / ksplit + 3) & ~3;
    const int zs = (K + k_chunk - 1) / k_chunk;
    // (column tiles x row blocks folded into x: a grid may be 65535 workgroups along y, and M / 64 can exceed that)
    dim3 grid((unsigned)((N + 64 * TN - 1) / (64 * TN)) * (unsigned)((M + WAVES * R - 1) / (WAVES * R)), 1, zs);
    if (zs > 1) {
        hipError_t e = launch_zero_u32(C, (size_t)M * N, stream);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), lds, stream, A, B, C, reinterpret_cast<const uint32_t*>(lut),
                       lut_dwords, g.cols * 2, M, K, N, k_chunk, zs > 1 ? 1 : 0, gate, out_f32);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess && zs > 1 && out_f32) e = launch_u32_to_f32(C, (size_t)M * N, stream);
    return e;
}

// Tile selection.  n_cu: compute units of the device.  The table occupies 33.5 KB (7-bit) so four
// 256-thread workgroups fit a CU; the 8-bit table (132.6 KB) leaves room for one workgroup, which
// is therefore made 1024 threads wide.
hipError_t launch_fwd(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g, int M,
                      int K, int N, int n_cu, hipStream_t stream, int out_f32) {
    const bool big = g.bits == 8;
    const int waves = big ? 16 : 4;
    int R, TN;
    if (N <= 64) { TN = 1; R = 32; }
    else if (N <= 128) { TN = 2; R = 32; }
    else { TN = 4; R = 16; }
    const long target_wg = (long)n_cu * (big ? 1 : 4);
    auto n_wg = [&](int r, int tn) { return (long)((N + 64 * tn - 1) / (64 * tn)) * ((M + waves * r - 1) / (waves * r)); };
    if (TN <= 2 && R == 32 && n_wg(R, TN) < target_wg) R = 16;
    long wgs = n_wg(R, TN);
    int ksplit = 1;
    if (wgs < target_wg) {
        ksplit = (int)((target_wg + wgs - 1) / wgs);
        const int max_split = K / 32 > 0 ? K / 32 : 1;  // keep at least 32 k per workgroup
        if (ksplit > max_split) ksplit = max_split;
        if (ksplit > 64) ksplit = 64;
    }
#define AMR_FWD_CASE(r, tn)                                                                                   \
    if (R == r && TN == tn)                                                                                   \
        return big ? launch_fwd_t<r, tn, 16>(A, B, C, lut, g, M, K, N, ksplit, stream, nullptr, out_f32)       \
                   : launch_fwd_t<r, tn, 4>(A, B, C, lut, g, M, K, N, ksplit, stream, nullptr, out_f32);
    AMR_FWD_CASE(32, 1)
    AMR_FWD_CASE(16, 1)
    AMR_FWD_CASE(32, 2)
    AMR_FWD_CASE(16, 2)
    AMR_FWD_CASE(16, 4)
#undef AMR_FWD_CASE
    return hipErrorInvalidValue;
}

// Direct kernel queued behind the expanded-table kernel: it runs only when *gate != 0 (the operand
// held a masked code) and then overwrites all of C, so it must not split K.
hipError_t launch_fwd_gated(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                            int M, int K, int N, const uint32_t* gate, hipStream_t stream, int out_f32) {
    if (N <= 64) return launch_fwd_t<32, 1, 4>(A, B, C, lut, g, M, K, N, 1, stream, gate, out_f32);
    if (N <= 128) return launch_fwd_t<32, 2, 4>(A, B, C, lut, g, M, K, N, 1, stream, gate, out_f32);
    return launch_fwd_t<16, 4, 4>(A, B, C, lut, g, M, K, N, 1, stream, gate, out_f32);
}

}  // namespace amr
