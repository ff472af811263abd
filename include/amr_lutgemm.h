/*
 * amr_lutgemm.h -- C ABI of the MI355X (gfx950) LUT-based approximate-multiplier GEMM.
 *
 * Shared library: libamr_lutgemm.so.  Plain pointers and sizes only; every pointer is a DEVICE
 * pointer on the current HIP device unless stated otherwise; `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  All launches are asynchronous on `stream`.
 *
 * Return value: 0 on success, a negative AMR_E* code on a rejected argument, or a positive
 * hipError_t value when the HIP runtime reported a failure.  amr_last_error() returns a
 * thread-local human readable message for the last non-zero return.
 *
 * Table layout ("padded table"), as the reference defines it
 * (self_ops/src/approx_mult.h:12-40, self_ops/ops_py/approx_ops.py:21-41,70-77):
 *   bits b in {4, 6, 7, 8};  rows = 2^b + 1, cols = 2^b + 2;
 *   entry (a, b) at a * cols + b;  total length rows * cols + tail, tail = 718 / 830 / 638 / 0;
 *   everything outside [0,2^b) x [0,2^b) is zero, so the code value 2^b is a "masked" operand
 *   that contributes 0 (self_ops/src/approx_mult.h:40).
 * The bit-width is derived from the table length at run time (1024 -> 4, 5120 -> 6, 17408 -> 7,
 * 66306 -> 8); the reference fixes it with a compile-time macro instead (approx_mult.h:12).
 * Operand codes above 2^b are a precondition violation exactly as in the reference
 * (approx_gemm_forward.cu:200 reads out of bounds); they are not checked on the device.
 */
#ifndef AMR_LUTGEMM_H
#define AMR_LUTGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AMR_OK 0
#define AMR_EINVAL (-1)    /* null pointer, negative size, misaligned table pointer            */
#define AMR_ELUTLEN (-2)   /* table length matches no supported bit-width                      */
#define AMR_EWORKSPACE (-3)/* caller workspace too small                                       */
#define AMR_EUNSUPPORTED (-4)

/* Library version (major*10000 + minor*100 + patch) and the gfx target it was built for. */
int amr_version(void);
const char *amr_target_arch(void);
const char *amr_last_error(void);

/* Geometry helpers (host only, no device work).
 * Mirrors self_ops/ops_py/approx_ops.py:21-41.  Return AMR_ELUTLEN for unsupported values. */
int amr_lut_geometry(int bits, int *rows, int *cols, int64_t *elem_num);
int amr_bits_from_lut_elems(int64_t lut_elems);

/*
 * Forward:  C[m,n] = sum_{k<K} lut[A[m,k] * cols + B[k,n]]   (uint32 wrap-around accumulate)
 * Replaces approx_gemm_forward_gpu (self_ops/src/approx_gemm_forward.cu:241-314), which is what
 * the pybind function approx_ops.approx_gemm_forward binds (self_ops/src/op_register.cpp:17).
 *   A   [M,K] uint8 row-major      B [K,N] uint8 row-major      C [M,N] uint32 row-major (overwritten)
 *   lut padded table, uint16, length lut_elems, 4-byte aligned.
 * M, K or N equal to 0 is accepted (K == 0 zero-fills C).
 */
int amr_lut_gemm_forward(const uint8_t *A, const uint8_t *B, uint32_t *C, const uint16_t *lut,
                         int64_t lut_elems, int M, int K, int N, void *stream);

/*
 * Same operation with caller-provided scratch.  For large M and tables of at most 7 bits the forward
 * pass first expands the table along B (E[k][a][n] = lut[a][B[k,n]]) into `workspace` and then adds
 * rows of E; amr_lut_gemm_forward_workspace_bytes gives the size that needs (0 = no scratch used for
 * this shape).  workspace must be 256-byte aligned; NULL makes the library use its own buffer for this
 * (device, stream), grown with hipMalloc when needed and never freed or waited for (amr_lut_gemm_forward does
 * exactly that; see amr_lut_gemm_backward for the rules).
 * No counterpart in the reference, whose forward kernel needs no scratch.
 */
size_t amr_lut_gemm_forward_workspace_bytes(int64_t lut_elems, int M, int K, int N);
int amr_lut_gemm_forward_ws(const uint8_t *A, const uint8_t *B, uint32_t *C, const uint16_t *lut,
                            int64_t lut_elems, int M, int K, int N, void *workspace, size_t workspace_bytes,
                            void *stream);

/*
 * The expansion of the forward table along B (K*N*256 B for tables of at most 7 bits: 604 MB for a 4608 x 512 layer) depends
 * on B and the table only, not on A: a caller whose B stays put between calls -- inference, evaluation, calibration
 * passes -- keeps it in an amr_fwd_cache, one per weight matrix, and the forward pass skips the expansion launch while the
 * caller's b_version (any number that changes whenever the contents of B change), the table pointer, K and N stay the
 * same.  The cache owns its device memory (hipMalloc on the first call and when a larger shape arrives; hipFree, which
 * waits for the device, on replacement and on destroy).  Calls that share a cache must be ordered with each other (one
 * stream, or events); results are those of amr_lut_gemm_forward.  Shapes that do not take the expanded-table kernels
 * ignore the cache.  No counterpart in the reference.
 *   amr_lut_gemm_forward_cached: C is uint32 [M,N], or float32 when c_is_f32 != 0 (amr_lut_gemm_forward_f32_ws).
 */
typedef struct amr_fwd_cache amr_fwd_cache;
int amr_fwd_cache_create(amr_fwd_cache **out);
int amr_fwd_cache_destroy(amr_fwd_cache *cache);
int amr_fwd_cache_stats(amr_fwd_cache *cache, uint64_t *hits, uint64_t *misses, size_t *device_bytes);   /* any pointer may be NULL */
int amr_lut_gemm_forward_cached(amr_fwd_cache *cache, uint64_t b_version, const uint8_t *A, const uint8_t *B, void *C,
                                int c_is_f32, const uint16_t *lut, int64_t lut_elems, int M, int K, int N, void *stream);

/*
 * Same sums, stored as float32: C[m,n] = (float)(uint32 sum), rounded to nearest even above 2^24, i.e. the
 * bits of the `.to(torch.float32)` the reference's callers apply to the result at once
 * (self_ops/ops_py/approx_ops.py:569, :165) without the pass over C that conversion costs.
 */
int amr_lut_gemm_forward_f32_ws(const uint8_t *A, const uint8_t *B, float *C, const uint16_t *lut,
                                int64_t lut_elems, int M, int K, int N, void *workspace, size_t workspace_bytes,
                                void *stream);

/*
 * Backward (both gradients, as the reference always produces both):
 *   gA[m,k] = (1/16) * sum_{n<N} gC[m,n] * (float)lut_grad_a[A[m,k] * cols + B[k,n]]
 *   gB[k,n] = (1/16) * sum_{m<M} (float)lut_grad_b[A[m,k] * cols + B[k,n]] * gC[m,n]
 * Replaces approx_gemm_backward_gpu (self_ops/src/approx_gemm_backward.cu:506-624), bound as
 * approx_ops.approx_gemm_backward (self_ops/src/op_register.cpp:19).  fp32 accumulation; the
 * summation order differs from the reference's sequential order (results agree to fp32
 * summation-order tolerance and are deterministic run to run).
 *   gC [M,N] fp32   A [M,K] uint8   B [K,N] uint8   gA [M,K] fp32 (overwritten)   gB [K,N] fp32 (overwritten)
 *   lut_grad_a / lut_grad_b: padded tables, int16 (slope x 16), length lut_elems, 4-byte aligned.
 * gA or gB may be NULL to skip that gradient (extension; the reference computes both).
 * workspace: device scratch for the split-M partial sums of gB and the expanded table of gradA, at least
 *   amr_lut_gemm_backward_workspace_bytes(M,K,N) bytes, 256-byte aligned; or NULL, in which case the
 *   library uses a buffer of its own, one per (device, stream): calls on one stream share it in stream order,
 *   calls on different streams (also from different host threads) never do.  The library grows such a buffer with
 *   hipMalloc when a call needs more than any earlier call on that stream did, keeps the old one until the
 *   process ends (queued work may still use it) and never waits for the device.  hipMalloc cannot run while the
 *   stream is being captured into a graph: capture with a workspace, after an uncaptured call of the same size,
 *   or through amr_lut_gemm_backward_static.
 */
size_t amr_lut_gemm_backward_workspace_bytes(int M, int K, int N);
/* The same for a known table width (lut_elems as passed to the call); the shape-only query above is an upper bound over all
 * widths.  What gradA adds to the partial sums of gB: tables of at most 7 bits K*N*256 B of expanded table (large M only);
 * 8-bit tables (N/64)*M*K*4 B of partial results for 2048 <= M < 16384, or K*N*512 B of int16 expanded table beyond that
 * (K*N*1 KB for float tables) -- e.g. 302 MB for 2048 x 4608 x 512, more than the 7-bit answer for that shape. */
size_t amr_lut_gemm_backward_workspace_bytes_for(int64_t lut_elems, int M, int K, int N);
int amr_lut_gemm_backward(const float *gC, const uint8_t *A, const uint8_t *B, float *gA, float *gB,
                          const int16_t *lut_grad_a, const int16_t *lut_grad_b, int64_t lut_elems,
                          int M, int K, int N, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Same as amr_lut_gemm_backward with a choice of layout for gA.  ga_rows_per_image = 0: row-major [M,K].
 * ga_rows_per_image = L > 0 (L must divide M): image-major transposed gA_T[M/L][K][L], i.e. the
 * [batch, C*kh*kw, oh*ow] layout that col2im (torch fold) consumes directly when the rows of A are
 * the im2col windows of M/L images -- saves the transpose copy between the GEMM and the fold in the
 * reference's conv glue (self_ops/ops_py/approx_ops.py:562-563, backward).  No counterpart in the reference.
 */
int amr_lut_gemm_backward_ex(const float *gC, const uint8_t *A, const uint8_t *B, float *gA, float *gB,
                             const int16_t *lut_grad_a, const int16_t *lut_grad_b, int64_t lut_elems,
                             int M, int K, int N, int ga_rows_per_image, void *workspace, size_t workspace_bytes,
                             void *stream);

/*
 * amr_lut_gemm_backward_ex for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, results and kernels; the scratch
 * (flags, partial sums of gB, expanded table of gradA) is a file-scope device array of AMR_STATIC_SCRATCH_BYTES inside the
 * library, one copy per GPU, held until the process ends.  The call allocates and frees nothing.  The array is sized for
 * the kernels the call launches: gradB splits M only as far as the array has room for partial sums (K*N*4 B each; with
 * room for fewer than two it does not split, which needs none), and a shape whose expanded table of gradA does not fit
 * behind them runs gradA on the direct kernel -- same results up to summation order, slower.  Only a shape whose column sums
 * of gC alone (64*N*4 B, N beyond 131 000) exceed the array is rejected with AMR_EWORKSPACE.  All calls on one GPU share
 * that array: calls that overlap in time on one GPU (two streams, two threads) race; calls queued on one stream do not.
 */
#define AMR_STATIC_SCRATCH_BYTES (32u << 20)
size_t amr_static_scratch_bytes(void);
int amr_lut_gemm_backward_static(const float *gC, const uint8_t *A, const uint8_t *B, float *gA, float *gB,
                                 const int16_t *lut_grad_a, const int16_t *lut_grad_b, int64_t lut_elems,
                                 int M, int K, int N, int ga_rows_per_image, void *stream);

/*
 * Backward with float32 gradient tables: the same two sums with lut_grad_a / lut_grad_b holding the slopes themselves
 * (padded tables of lut_elems float32 entries, entry (a,b) at a * cols + b) and `scale` in place of the 1/16:
 *   gA[m,k] = scale * sum_{n<N} gC[m,n] * lut_grad_a[A[m,k] * cols + B[k,n]]
 *   gB[k,n] = scale * sum_{m<M} lut_grad_b[A[m,k] * cols + B[k,n]] * gC[m,n]
 * The reference's entry point (approx_gemm_backward_gpu, self_ops/src/approx_gemm_backward.cu:506-624) takes int16
 * tables only, rounded from float slopes by scripts/gen_bp_lut.py:172-183; this one takes the unrounded slopes
 * (scale = 1) or any other float table.  A float table of int16 values with scale = 1/16 gives the results of
 * amr_lut_gemm_backward up to fp32 summation order.  An 8-bit float table (265 KB) exceeds the LDS of a CU and is
 * processed in two bands of rows.  Arguments otherwise as amr_lut_gemm_backward_ex; the workspace size is
 * amr_lut_gemm_backward_f32tab_workspace_bytes(M,K,N) (partial sums of gB and, for large M, the float32 expanded table
 * of gradA, twice the size of the int16 path's).
 */
size_t amr_lut_gemm_backward_f32tab_workspace_bytes(int M, int K, int N);
size_t amr_lut_gemm_backward_f32tab_workspace_bytes_for(int64_t lut_elems, int M, int K, int N);   /* for a known table width */
int amr_lut_gemm_backward_f32tab(const float *gC, const uint8_t *A, const uint8_t *B, float *gA, float *gB,
                                 const float *lut_grad_a, const float *lut_grad_b, int64_t lut_elems, float scale,
                                 int M, int K, int N, int ga_rows_per_image, void *workspace, size_t workspace_bytes,
                                 void *stream);

/*
 * im2col of operand codes: x [B,C,H,W] float32 holding integer codes 0..255 -> A [B*oh*ow, C*kh*kw] uint8,
 * row (b,oy,ox), column c*kh*kw + i*kw + j, same stride / padding / dilation on both axes, padding
 * positions = code 0.  One pass instead of the reference's pad + unfold + transpose + reshape + cast
 * (self_ops/ops_py/approx_ops.py:556-563, :161-164).
 */
int amr_im2col_u8_f32(const float *x, uint8_t *A, int B, int C, int H, int W, int kh, int kw, int stride, int pad,
                      int dil, void *stream);

/*
 * Adjoint of amr_im2col_u8_f32 for gradients: cols [B][C*kh*kw][oh*ow] float32 (the layout amr_lut_gemm_backward_ex
 * writes with ga_rows_per_image = oh*ow) -> x [B,C,H,W], every pixel the sum of the window entries it fed.  The
 * input-gradient step the reference leaves to autograd through F.unfold (self_ops/ops_py/approx_ops.py:558).
 * Overwrites x; fixed summation order (no atomics).
 */
int amr_col2im_f32(const float *cols, float *x, int B, int C, int H, int W, int kh, int kw, int stride, int pad,
                   int dil, void *stream);

/*
 * Process-wide switch for diagnostics, tests and benchmarks.  mode 0 sends every later call to the direct
 * gather kernels (the formulation of the reference's kernels, approx_gemm_forward.cu:45-229); 1 (the default)
 * lets the library pick by problem size; 2 takes the expanded-table kernels wherever the shape allows, also
 * where they are slower.  Returns the previous mode.  Results are the same in every mode (forward bit-exact,
 * backward to summation order); the workspace size queries answer for the mode in force.  No counterpart in
 * the reference.
 */
int amr_set_expanded_table_kernels(int mode);

/*
 * Process-wide switch, on by default: a backward call that computes both gradients of a small problem (M*K*N < 2e9,
 * where the latencies of the dependent launches outweigh the arithmetic) queues its gradB launches on a stream of the
 * library's own beside the gradA launches on the caller's stream; the caller's stream waits for that side stream before
 * the call returns, so results and stream order are those of the serial form (and the fork / join is captured like any
 * other cross-stream dependency when the caller's stream is being captured into a graph).  0 switches it off.  Returns
 * the previous setting.  No counterpart in the reference, which launches both kernels on the default stream
 * (self_ops/src/approx_gemm_backward.cu:560-608).
 */
int amr_set_backward_fork(int on);

/*
 * What the library has taken from the HIP runtime since it was loaded, over all devices: bytes of scratch it allocated for
 * callers that passed no workspace (never freed), and side streams it created (amr_set_backward_fork).  Either pointer may
 * be NULL.  A call with a caller workspace on a problem that does not fork, and amr_lut_gemm_backward_static, change neither.
 * Diagnostics; no counterpart in the reference.
 */
void amr_library_resources(size_t *scratch_bytes, int *side_streams);

/*
 * Dequantisation behind the LUT convolution, from the GEMM's row layout to the NCHW activation in one pass:
 *   out[b,n,pos] = (*s_a * *s_w) * (c[b*L+pos, n] + ((*z_w * x_sum[b*L+pos] + *z_a * w_resp[n*L+pos]) + (*z_a * *z_w) * taps[pos])) + bias[n]
 * with L = positions; c [batch*L, out_channels], x_sum [batch*L], w_resp [out_channels*L], taps [L], out [batch,
 * out_channels, L]; bias may be NULL; the four scalars are device pointers.  These are the zero-point terms and the
 * scaling of the reference's ApproxConv2d.forward (micronet+/app_layers.py:175-183), every operation rounded on its
 * own in that order.  The backward entry point gives g_c[b*L+pos, n] = (*s_a * *s_w) * g[b,n,pos].
 */
int amr_conv_dequant_f32(const float *c, const float *x_sum, const float *w_resp, const float *taps, const float *z_a,
                         const float *z_w, const float *s_a, const float *s_w, const float *bias, float *out,
                         int batch, int out_channels, int positions, void *stream);
int amr_conv_dequant_backward_f32(const float *g, const float *s_a, const float *s_w, float *g_c, int batch,
                                  int out_channels, int positions, void *stream);

/*
 * Forward LUT GEMM of a convolution with the dequantisation in the kernel's store: the sums of amr_lut_gemm_forward never
 * go to memory, the kernel writes the NCHW activation of amr_conv_dequant_f32 directly (same operations in the same order
 * on the float32 sums: the same bits),
 *   out[b,n,pos] = (*s_a * *s_w) * ((float)C[b*L+pos, n] + ((*z_w * x_sum[b*L+pos] + *z_a * w_resp[n*L+pos]) + (*z_a * *z_w) * taps[pos])) + bias[n]
 * with L = positions (must divide M); A [M,K], B [K,N] uint8 in any common order of k.  Replaces the LUT GEMM plus the
 * zero-point terms and scaling of the reference's ApproxConv2d.forward (self_ops/src/approx_gemm_forward.cu:241-314 called
 * from micronet+/app_layers.py:175-183).  Shapes the expanded-table kernel does not take whole (small problems, a K split
 * over workgroups) run the GEMM into the workspace and dequantise in a second pass.  workspace: at least
 * amr_lut_conv_forward_dequant_workspace_bytes(...) bytes, 256-byte aligned, required.
 */
size_t amr_lut_conv_forward_dequant_workspace_bytes(int64_t lut_elems, int M, int K, int N);
int amr_lut_conv_forward_dequant_f32(const uint8_t *A, const uint8_t *B, const uint16_t *lut, int64_t lut_elems, int M, int K,
                                     int N, int positions, const float *x_sum, const float *w_resp, const float *taps,
                                     const float *z_a, const float *z_w, const float *s_a, const float *s_w, const float *bias,
                                     float *out, void *workspace, size_t workspace_bytes, void *stream);
/* The same with the expansion kept in an amr_fwd_cache (cache = NULL: as above). */
int amr_lut_conv_forward_dequant_cached_f32(amr_fwd_cache *cache, uint64_t b_version, const uint8_t *A, const uint8_t *B,
                                            const uint16_t *lut, int64_t lut_elems, int M, int K, int N, int positions,
                                            const float *x_sum, const float *w_resp, const float *taps, const float *z_a,
                                            const float *z_w, const float *s_a, const float *s_w, const float *bias, float *out,
                                            void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same forward pass of a 3x3 convolution of stride 1 and padding 1 WITHOUT its window matrix (the reference builds it with
 * F.pad + F.unfold, self_ops/ops_py/approx_ops.py:556-563, and feeds it to self_ops/src/approx_gemm_forward.cu:241-314): the
 * rows of the GEMM are the B*H*W pixels of `codes` (pixel-major uint8 [B*H*W][C], what amr_quantize_codes_nhwc_u8 writes, 16-byte
 * aligned), column tap*C + c of a row is read from the neighbouring pixel the tap reaches, or as code 0 where that pixel is
 * padding; Bt [9*C][N] tap-major weight codes.  out and the dequantisation operands as above with positions = H*W.
 *   amr_lut_conv_forward_implicit_supported: 1 where the kernel serves the geometry and table width (tables of at most 7 bits,
 *     C a multiple of 16, the shapes the expanded-table kernel takes without a K split), else 0.
 *   A_fallback (optional): the window matrix [B*H*W][9*C]; with it a masked code in the operands or a table whose entries do not
 *     fit the packed sums is recomputed by the gated direct kernel as in the calls above; without it such a case leaves NaN in out.
 *   cache (optional) as in the _cached call.  workspace: amr_lut_conv_forward_implicit_workspace_bytes(..., cache != NULL,
 *     A_fallback != NULL) bytes, 256-byte aligned (0 bytes with a cache and no fall-back: workspace may then be NULL).
 */
int amr_lut_conv_forward_implicit_supported(int64_t lut_elems, int B, int C, int H, int W, int N);
size_t amr_lut_conv_forward_implicit_workspace_bytes(int64_t lut_elems, int B, int C, int H, int W, int N, int cached,
                                                     int with_fallback);
int amr_lut_conv_forward_implicit_f32(amr_fwd_cache *cache, uint64_t b_version, const uint8_t *codes, const uint8_t *Bt,
                                      const uint16_t *lut, int64_t lut_elems, int B, int C, int H, int W, int N,
                                      const float *x_sum, const float *w_resp, const float *taps, const float *z_a,
                                      const float *z_w, const float *s_a, const float *s_w, const float *bias, float *out,
                                      const uint8_t *A_fallback, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Range tracking and quantisation parameters of one tensor in one launch (all pointers: one float in device memory).
 * mode 0: min_val/max_val := cur_min/cur_max (first batch); 1: running extremes; 2: keep * old + momentum * current;
 * then *scale = max((max - min) / quant_max, eps) -- or (max - min) * inv_quant_max when inv_quant_max != 0, which is
 * what the tensor library computes for a division by a host-side scalar -- and *zp_neg = round(min / *scale).  The scalar tensor operations of the
 * reference's observers and quantisers (micronet+/app_layers.py:21-53, :154-160), each rounded on its own in that order.
 */
int amr_observer_update_f32(const float *cur_min, const float *cur_max, float *min_val, float *max_val, float *scale,
                            float *zp_neg, int mode, float keep, float momentum, float quant_max, float inv_quant_max,
                            float eps, void *stream);

/*
 * The extremes of x (n float32 values; what torch.min / torch.max give the reference's observers, micronet+/app_layers.py:41-46)
 * and amr_observer_update_f32 on them, in one launch.  A NaN in x makes both extremes NaN, as in the tensor library.
 * state: AMR_OBSERVE_STATE_WORDS 32-bit words of device memory owned by the caller, one set per observer, all zero before the
 * first call (word 0 counts the workgroups that have finished and is back at zero when the call ends; the others hold their
 * partial results).  Calls that share a state must not overlap in time.
 * mode | 4: the extremes of max(x, 0) instead of x (an observer behind a ReLU that the caller does not materialise).
 */
#define AMR_OBSERVE_STATE_WORDS (4 + 3 * 1024)
int amr_observe_minmax_f32(const float *x, int64_t n, uint32_t *state, float *min_val, float *max_val, float *scale,
                           float *zp_neg, int mode, float keep, float momentum, float quant_max, float inv_quant_max, float eps,
                           void *stream);

/*
 * Quantiser in front of the LUT GEMM: codes[i] = clamp(round(x[i] / *scale - *zp_neg), 0, qmax) as float32,
 * round half to even; scale and zp_neg are device pointers to one float each.  One pass instead of the
 * divide / subtract / round / straight-through / clamp chain of the reference's quantize_v2
 * (micronet+/app_layers.py:147-160).  The backward entry point gives the gradient of that expression with
 * straight-through rounding: gx[i] = g[i] / *scale where the rounded value lies in [0, qmax], else 0.
 */
int amr_quantize_codes_f32(const float *x, const float *scale, const float *zp_neg, float qmax, float *codes,
                           int64_t n, void *stream);
int amr_quantize_codes_backward_f32(const float *g, const float *x, const float *scale, const float *zp_neg,
                                    float qmax, float *gx, int64_t n, void *stream);

/*
 * The same quantiser producing what the LUT convolution consumes, with no float32 code tensor in between (the reference
 * keeps the codes as float32 and casts them in front of the GEMM, micronet+/app_layers.py:172-173 ->
 * self_ops/ops_py/approx_ops.py:161-164):
 *   codes  [B*L, C] uint8, "pixel-major": the C codes of pixel m = b*L + pix are adjacent (L = H*W)
 *   inside [B, C, L] uint8: 1 where the rounded value lay in [0, qmax] -- all the straight-through backward of the clamp
 *          needs (amr_conv_input_grad_f32), so that x is not read again
 *   x_sum  [B*L] float32: sum of a pixel's codes over the channels, the operand of the zero-point term conv(X, Zw)
 * x is [B, C, L] float32; qmax <= 255.  A NaN input gives code 0, inside 0.
 */
int amr_quantize_codes_nhwc_u8(const float *x, const float *scale, const float *zp_neg, float qmax, uint8_t *codes,
                               uint8_t *inside, float *x_sum, int B, int C, int L, void *stream);
/* relu != 0: the quantiser of max(x, 0) -- a ReLU in front of the layer (as in the reference's networks, micronet+/models.py:103)
 * without its own pass: codes and x_sum of max(x, 0); inside = 1 where x > 0 AND the rounded value lay in [0, qmax], i.e. the
 * product of the two backward masks, so that the backward pass of the layer yields the gradient in front of the ReLU. */
int amr_quantize_codes_nhwc_relu_u8(const float *x, const float *scale, const float *zp_neg, float qmax, uint8_t *codes,
                                    uint8_t *inside, float *x_sum, int B, int C, int L, int relu, void *stream);

/*
 * im2col of pixel-major codes: A [B*oh*ow, kh*kw*C] uint8, row (b,oy,ox), column (i*kw + j)*C + c ("tap-major": the
 * order of the GEMM's k index is free as long as the rows of B follow it; the reference's is c*kh*kw + i*kw + j,
 * self_ops/ops_py/approx_ops.py:556-563), padding positions = code 0.  A window row is kh*kw runs of C adjacent bytes.
 */
int amr_im2col_nhwc_u8(const uint8_t *codes, uint8_t *A, int B, int C, int H, int W, int kh, int kw, int stride, int pad,
                       int dil, void *stream);

/*
 * Input gradient of the quantised LUT convolution in one pass: the adjoint of amr_im2col_nhwc_u8, the gradient of the
 * zero-point term conv(X, Zw) and the quantiser's straight-through backward (micronet+/app_layers.py:147-160,175-181):
 *   gx[b,c,y,x] = inside[b,c,y,x] ? (sum over taps of cols[b][tap*C + c][pos(tap)] + *z_w * sum over taps of t[b][pos(tap)]) / *scale : 0
 * cols [B][kh*kw*C][oh*ow] float32 is what amr_lut_gemm_backward_ex writes with ga_rows_per_image = oh*ow for a tap-major A;
 * cols = NULL: gx already holds the sum over the taps and is finished in place.  t [B][oh*ow] = the row sums of the
 * GEMM's output gradient (amr_conv_dequant_backward_rowsum_f32); z_w, scale: device scalars.  Fixed summation order.
 */
int amr_conv_input_grad_f32(const float *cols, const float *t, const float *z_w, const uint8_t *inside, const float *scale,
                            float *gx, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil, void *stream);

/*
 * Weight side of the quantised LUT convolution, one launch each way (the reference: quantize_v2 on the weights, the cast and
 * transposes in front of the GEMM and the zero-point convolution conv(Za, W), micronet+/app_layers.py:173,179 with
 * self_ops/ops_py/approx_ops.py:560-561, and their autograd graph):
 *   prepare:  Bt[(tap*C + c)*N + n] = code of w[n][c][tap] (uint8, the GEMM's B with tap-major rows); inside[n][c][tap] = 1 where
 *             the rounded value lay in [0, qmax]; w_resp[n][pos] = sum over taps of (sum over c of the codes) * tapmask[tap][pos]
 *             -- the response of the weight codes to an all-ones image, tapmask[tap][pos] = 1 where tap `tap` of output position
 *             `pos` lies inside the image.  w [N][C][taps] float32; scale, zp_neg device scalars; at most 64 taps.
 *   zero-point gradient: g_wr[n][pos] = (*z_a * (*s_a * *s_w)) * sum over b of g[b][n][pos] (g the output gradient [B][N][L],
 *             16-byte aligned; g_wr may be null): the gradient of the term Za * w_resp with respect to w_resp; and the same folded
 *             onto the taps, gz[p][n][tap] = sum over the positions pos of block p of g_wr[n][pos] * tapmask[tap][pos], in
 *             P = amr_conv_zero_point_grad_parts(positions) blocks of positions (gz holds P*N*taps floats; the weight-gradient
 *             call adds the blocks).  Fixed summation order; workspace of amr_conv_zero_point_grad_workspace_bytes bytes, 16-byte
 *             aligned.
 *   grad:     gw[n][c][tap] = inside ? (gBt[(tap*C + c)*N + n] + sum over p < gz_parts of gz[p][n][tap]) / *scale : 0, gBt the
 *             gB of amr_lut_gemm_backward_ex for the tap-major operands.
 */
int amr_conv_weight_prepare_f32(const float *w, const float *scale, const float *zp_neg, float qmax, const float *tapmask,
                                uint8_t *Bt, uint8_t *inside, float *w_resp, int N, int C, int taps, int positions, void *stream);
size_t amr_conv_zero_point_grad_workspace_bytes(int batch, int N, int positions);
int amr_conv_zero_point_grad_parts(int positions);
int amr_conv_zero_point_grad_f32(const float *g, const float *z_a, const float *s_a, const float *s_w, const float *tapmask,
                                 float *g_wr, float *gz, int batch, int N, int positions, int taps, void *workspace,
                                 size_t workspace_bytes, void *stream);
int amr_conv_weight_grad_f32(const float *gBt, const float *gz, int gz_parts, const uint8_t *inside, const float *scale, float *gw,
                             int N, int C, int taps, void *stream);

/*
 * Everything the backward pass of the layer derives from the output gradient g [B][N][L] alone, in one call:
 * g_c and t of amr_conv_dequant_backward_rowsum_f32 and, with tapmask and gz given, gz of amr_conv_zero_point_grad_f32 (same
 * values; no g_wr).  Where the geometry allows (L a multiple of 128, N <= 128) the batch sums behind gz are formed by the
 * kernel that writes g_c, so that g is read once.  workspace: amr_conv_output_grad_workspace_bytes bytes, 16-byte aligned
 * (only needed with gz).
 */
size_t amr_conv_output_grad_workspace_bytes(int batch, int out_channels, int positions);
int amr_conv_output_grad_f32(const float *g, const float *z_a, const float *s_a, const float *s_w, const float *tapmask, float *g_c,
                             float *t, float *gz, int batch, int out_channels, int positions, int taps, void *workspace,
                             size_t workspace_bytes, void *stream);

/*
 * Input gradient of a quantised 3x3 LUT convolution of stride 1 and padding 1 WITHOUT the [M][9C] gradient matrix: gradA of
 * amr_lut_gemm_backward_ex, amr_col2im_f32 and amr_conv_input_grad_f32 as one implicit GEMM over the B*H*W input pixels,
 *   gx[b,c,y,x] = inside[b,c,y,x] ? ((1/16) * sum over taps (ti,tj) and n of gC[(b, y+1-ti, x+1-tj), n] *
 *                 (float)lut_grad_a[codes[(b,y,x), c] * cols + Bt[(ti*3+tj)*C + c, n]] + *z_w * sum over taps of t[(b, y+1-ti, x+1-tj)]) / *scale : 0
 * (positions outside the image contribute nothing).  gC [B*H*W, N] float32 (the GEMM rows of the output gradient), codes
 * [B*H*W, C] uint8 pixel-major (amr_quantize_codes_nhwc_u8), Bt [9*C, N] uint8 tap-major, t / z_w / inside / scale as in
 * amr_conv_input_grad_f32.  What the reference obtains from approx_gemm_backward_gpu
 * (self_ops/src/approx_gemm_backward.cu:506-624) followed by autograd's fold (self_ops/ops_py/approx_ops.py:558) and the
 * quantiser's backward (micronet+/app_layers.py:147-160); sums in another order, results to fp32 summation-order tolerance.
 * Served shapes: amr_lut_conv_input_grad_supported(...) != 0 (tables of at most 7 bits, C % 16 == 0, N % 32 == 0, at least
 * 1024 pixels, gC 16-byte aligned), else AMR_EUNSUPPORTED and nothing is launched.
 * A gradient table that cannot be held as halves (amr_grad_table_fits_halves(host copy) == 0) or an operand holding the masked
 * code 2^b needs the GEMM-shaped path: pass A_fallback [B*H*W, 9*C] (amr_im2col_nhwc_u8 of codes) and cols_fallback (scratch,
 * B*9*C*H*W floats) and the library queues it, gated on the device-side flag; with both NULL such a call fills gx with NaN.
 * workspace: amr_lut_conv_input_grad_workspace_bytes(...) bytes, 256-byte aligned, required.
 */
int amr_lut_conv_input_grad_supported(int64_t lut_elems, int B, int C, int H, int W, int N);
size_t amr_lut_conv_input_grad_workspace_bytes(int64_t lut_elems, int B, int C, int H, int W, int N);
int amr_grad_table_fits_halves(const int16_t *host_table, int64_t lut_elems);      /* host pointer; 1, 0 or a negative AMR_E* */
int amr_lut_conv_input_grad_f32(const float *gC, const uint8_t *codes, const uint8_t *Bt, const int16_t *lut_grad_a,
                                int64_t lut_elems, const float *t, const float *z_w, const uint8_t *inside, const float *scale,
                                float *gx, int B, int C, int H, int W, int N, const uint8_t *A_fallback, float *cols_fallback,
                                void *workspace, size_t workspace_bytes, void *stream);
/* The same with the gradient table expanded along Bt kept in an amr_fwd_cache of its own between calls (weights that do not
 * change between backward passes: frozen layers that still hand a gradient to their input, gradient accumulation over
 * micro-batches); b_version as in amr_lut_gemm_forward_cached.  cache = NULL: as above.  With a cache the workspace needs
 * amr_lut_conv_input_grad_cached_workspace_bytes bytes only. */
size_t amr_lut_conv_input_grad_cached_workspace_bytes(int64_t lut_elems, int B, int C, int H, int W, int N);
int amr_lut_conv_input_grad_cached_f32(amr_fwd_cache *cache, uint64_t b_version, const float *gC, const uint8_t *codes,
                                       const uint8_t *Bt, const int16_t *lut_grad_a, int64_t lut_elems, const float *t,
                                       const float *z_w, const uint8_t *inside, const float *scale, float *gx, int B, int C, int H,
                                       int W, int N, const uint8_t *A_fallback, float *cols_fallback, void *workspace,
                                       size_t workspace_bytes, void *stream);

/* amr_conv_dequant_backward_f32 that also leaves t[m] = sum over n of g_c[m, n] (ascending n), in the same pass. */
int amr_conv_dequant_backward_rowsum_f32(const float *g, const float *s_a, const float *s_w, float *g_c, float *t, int batch,
                                         int out_channels, int positions, void *stream);

/*
 * Accurate fp32 GEMM  C = A . B  (row-major), kept for API parity only.
 * Replaces acc_gemm_forward_fp32_gpu (self_ops/src/approx_gemm_forward.cu:494-571), bound as
 * approx_ops.acc_gemm_forward_fp32 (self_ops/src/op_register.cpp:18).
 */
int amr_acc_gemm_forward_fp32(const float *A, const float *B, float *C, int M, int K, int N, void *stream);

/*
 * LDS gather-rate probe used to calibrate the roofline denominator.  Runs `iters` rounds of 8
 * ds_read_u16 per wave with conflict-free (pattern 0) or uniform-random-in-a-256-byte-row
 * (pattern 1) addresses on every CU and writes the kernel time in milliseconds to *ms_out (host
 * pointer; the call synchronises the stream).  gathers = waves_per_cu * n_cu * iters * 8 * 64.
 * Patterns 2 and 3 measure the delivery of 32 KB chunks from the L2 into LDS by LDS-direct loads instead (one
 * 1024-thread workgroup per CU, two chunks in flight, `iters` chunks per CU, waves_per_cu ignored; every workgroup
 * walks the same 9 MB (pattern 2) or 1 MB (pattern 3, resident in every L2) of chunks): *gathers_out then receives
 * the BYTES delivered over all CUs.
 * No counterpart in the reference.
 */
int amr_lds_gather_probe(int pattern, int waves_per_cu, int iters, float *ms_out, double *gathers_out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* AMR_LUTGEMM_H */
