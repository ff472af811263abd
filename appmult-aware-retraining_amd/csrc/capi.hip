// extern "C" entry points of libamr_lutgemm.so (declared in include/amr_lutgemm.h): argument checks,
// bit-width dispatch from the table length, per-device caches, launches on the caller's stream.
#include "../../include/amr_lutgemm.h"

#include <atomic>
#include <mutex>
#include <new>
#include <vector>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "amr_common.h"

namespace amr {
hipError_t launch_fwd(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g, int M,
                      int K, int N, int n_cu, hipStream_t stream, int out_f32);
size_t fwd_slab_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
hipError_t launch_fwd_slab(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, const LutGeom& g,
                           int M, int K, int N, int n_cu, void* workspace, hipStream_t stream, int out_f32,
                           const SlabDequant* dq = nullptr, int expanded = 0, const SlabConv* cv = nullptr,
                           const uint8_t* a_fallback = nullptr);
bool fwd_slab_can_dequant(const LutGeom& g, int M, int K, int N, int n_cu, bool force);
bool fwd_slab_conv_applies(const LutGeom& g, long M, int C, int N, int n_cu, bool force);
size_t gradB_workspace_bytes(int M, int K, int N, int n_cu);
hipError_t launch_gradB(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                        const LutGeom& g, int M, int K, int N, float scale, void* workspace, int n_cu,
                        hipStream_t stream, const uint32_t* gate = nullptr, int split_cap = 0);
int gradB_direct_splits_for(const LutGeom& g, int M, int K, int N, int n_cu);
hipError_t launch_gradA(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                        const LutGeom& g, int M, int K, int N, float scale, int n_cu, hipStream_t stream,
                        const uint32_t* gate = nullptr, int rows_per_image = 0);
size_t gradA_slab_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
size_t gradA_slab_i16_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
bool gradA_rows8_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force);
size_t gradA_rows8_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
hipError_t launch_gradA_rows8(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                              const LutGeom& g, int M, int K, int N, float scale, int n_cu, void* P, size_t p_bytes,
                              int rows_per_image, hipStream_t stream);
hipError_t launch_gradA_slab_i16(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                                 const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                                 int rows_per_image, hipStream_t stream);
hipError_t launch_gradA_slab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const int16_t* lut,
                             const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                             int rows_per_image, hipStream_t stream);
hipError_t launch_observer_update(const float* cur_min, const float* cur_max, float* min_val, float* max_val, float* scale,
                                  float* zp_neg, int mode, float keep, float momentum, float qmax, float inv_qmax, float eps,
                                  hipStream_t stream);
hipError_t launch_observe_minmax(const float* x, size_t n, uint32_t* state, float* min_val, float* max_val, float* scale, float* zp_neg,
                                 int mode, float keep, float momentum, float qmax, float inv_qmax, float eps, int n_cu, hipStream_t stream);
hipError_t launch_quantize_codes(const float* x, const float* scale, const float* zp_neg, float qmax, float* codes, size_t n,
                                 hipStream_t stream);
hipError_t launch_quantize_codes_backward(const float* g, const float* x, const float* scale, const float* zp_neg, float qmax,
                                          float* gx, size_t n, hipStream_t stream);
hipError_t launch_zero_u32(void* p, size_t n_dwords, hipStream_t stream);
hipError_t launch_bwd_header(const int16_t* lut_a, const int16_t* lut_b, const LutGeom& g, uint32_t* flags, hipStream_t stream);
hipError_t launch_dequant(const float* c, const float* xs, const float* wr, const float* tp, const float* za, const float* zw,
                          const float* sa, const float* sw, const float* bias, float* out, int M, int N, int L, hipStream_t stream);
hipError_t launch_dequant_grad(const float* g, const float* sa, const float* sw, float* gc, int M, int N, int L, hipStream_t stream);
hipError_t launch_col2im_f32(const float* cols, float* x, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil,
                             int oh, int ow, hipStream_t stream);
hipError_t launch_im2col_u8_f32(const float* x, uint8_t* A, int B, int C, int H, int W, int kh, int kw, int stride, int pad,
                                int dil, int oh, int ow, hipStream_t stream);
bool bwd_slab_applies(const LutGeom& g, int M, int K, int N);
bool gradB_slab8_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force);
int gradB_slab8_splits(int M, int K, int N, int n_cu);
hipError_t launch_gradB_slab8(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                              const LutGeom& g, int M, int K, int N, float scale, float* partials, int n_cu,
                              hipStream_t stream, int split_cap = 0);
bool gradB_slab8f_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force);
int gradB_slab8f_splits(int M, int K, int N, int n_cu);
hipError_t launch_gradB_slab8f(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut,
                               const LutGeom& g, int M, int K, int N, float scale, float* partials, int n_cu,
                               hipStream_t stream);
int gradB_slab_splits(int M, int K, int N, int n_cu);
size_t gradB_slab_colsum_floats(int N);
hipError_t launch_gradB_slab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const int16_t* lut,
                             const LutGeom& g, int M, int K, int N, float scale, uint32_t* flags, float* partials,
                             int n_cu, hipStream_t stream, int split_cap = 0);
hipError_t launch_gradB_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut, const LutGeom& g,
                               int M, int K, int N, float scale, void* workspace, int n_cu, hipStream_t stream,
                               const uint32_t* gate);
hipError_t launch_gradA_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut, const LutGeom& g,
                               int M, int K, int N, float scale, int n_cu, hipStream_t stream, const uint32_t* gate,
                               int rows_per_image);
hipError_t launch_gradB_slab_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gB, const float* lut,
                                    const LutGeom& g, int M, int K, int N, float scale, uint32_t* flags, float* partials,
                                    int n_cu, hipStream_t stream);
size_t gradA_slab_f32_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
size_t gradA_slab_f32w_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
bool gradA_rows8f_applies(const LutGeom& g, int M, int K, int N, const float* gC, bool force);
size_t gradA_rows8f_workspace_bytes(const LutGeom& g, int M, int K, int N, bool force);
hipError_t launch_gradA_rows8f(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                               const LutGeom& g, int M, int K, int N, float scale, int n_cu, void* P, size_t p_bytes,
                               int rows_per_image, hipStream_t stream);
hipError_t launch_gradA_slab_f32w(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                                  const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                                  int rows_per_image, hipStream_t stream);
hipError_t launch_gradA_slab_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, const float* lut,
                                    const LutGeom& g, int M, int K, int N, float scale, int n_cu, uint32_t* flags, void* S,
                                    int rows_per_image, hipStream_t stream);
hipError_t launch_quantize_nhwc(const float* x, const float* scale, const float* zp_neg, float qmax, uint8_t* codes, uint8_t* inside,
                                float* xs, long B, int C, int L, hipStream_t stream, int relu);
hipError_t launch_im2col_nhwc(const uint8_t* codes, uint8_t* A, long B, int C, int H, int W, int kh, int kw, int stride, int pad,
                              int dil, int oh, int ow, hipStream_t stream);
hipError_t launch_conv_input_grad(const float* cols, const float* t, const float* zw, const uint8_t* inside, const float* scale,
                                  float* gx, long B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil, int oh, int ow,
                                  hipStream_t stream, const uint32_t* gate = nullptr, int gate_mode = 0);
bool gradA_slab_conv_applies(const LutGeom& g, long M, int C, int N, const float* gC, bool force);
size_t gradA_slab_conv_workspace_bytes(int C, int N);
hipError_t launch_gradA_slab_conv(const float* gC, const uint8_t* codes, const uint8_t* Bt, float* g_in, const int16_t* lut,
                                  const LutGeom& g, int Bn, int C, int H, int W, int N, float scale, int n_cu, uint32_t* flags,
                                  void* S, const float* zero_line, hipStream_t stream, const float* zt, const float* zw,
                                  const float* qscale, const uint8_t* inside, int expanded);
bool gradA_slab_conv_can_finish(int Bn, int H, int W, const float* g_in);
hipError_t launch_conv_weight_prepare(const float* w, const float* scale, const float* zp_neg, float qmax, const float* tapmask,
                                      uint8_t* Bt, uint8_t* inside, float* w_resp, int N, int C, int T, int L, hipStream_t stream);
int batch_sum_segments(int B, size_t inner, int n_cu);
hipError_t launch_batch_sum_taps(const float* g, const float* za, const float* sa, const float* sw, const float* tapmask, float* g_wr,
                                 float* gz, float* partial, int B, int N, int L, int T, int n_cu, hipStream_t stream);
int batch_sum_parts(int L);
int output_grad_segments(int B, int N, int L, int n_cu, bool* fused);
hipError_t launch_output_grad(const float* g, const float* za, const float* sa, const float* sw, const float* tapmask, float* gc, float* t,
                              float* gz, float* partial, int B, int N, int L, int T, int n_cu, hipStream_t stream);
hipError_t launch_conv_weight_grad(const float* gBt, const float* gz, int parts, const uint8_t* inside, const float* scale, float* gw,
                                   int N, int C, int T, int n_cu, hipStream_t stream);
hipError_t launch_poison_if_raised(float* gx, size_t total, const uint32_t* gate, hipStream_t stream);
hipError_t launch_window_sums_3x3(const float* t, float* zt, long B, int H, int W, hipStream_t stream);
hipError_t launch_dequant_grad_rowsum(const float* g, const float* sa, const float* sw, float* gc, float* t, int M, int N, int L,
                                      hipStream_t stream);
hipError_t launch_accgemm(const float* A, const float* B, float* C, int M, int K, int N, hipStream_t stream);
hipError_t run_lds_probe(int pattern, int waves_per_cu, int iters, int n_cu, float* ms_out, double* gathers_out,
                         hipStream_t stream);
hipError_t run_lds_direct_probe(int n_chunks, int iters, int n_cu, float* ms_out, double* bytes_out, hipStream_t stream);
}  // namespace amr

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* where) {
    snprintf(g_err, sizeof(g_err), "%s: %s", where, hipGetErrorString(e));
    return (int)e;
}

constexpr int kMaxDevices = 64;
// Scratch the library owns for callers that pass none: one buffer per (device, stream).  Work queued on a stream runs
// in order, so calls on one stream can share a buffer; calls on different streams (possibly from different host
// threads) never do.  A buffer that has become too small is replaced by a larger one and kept until the process ends:
// launches already queued may still be using it, and freeing it would need a device-wide wait in the middle of an
// asynchronous call.
struct StreamScratch {
    hipStream_t stream;
    void* ptr;
    size_t bytes;
};
// A second stream and two events per (device, caller's stream): small backward calls run their gradB launches there,
// beside the gradA launches on the caller's stream, and join the caller's stream again before the call returns.
struct StreamFork {
    hipStream_t stream;       // the caller's
    hipStream_t side;
    hipEvent_t forked, joined;
};
struct DeviceState {
    int n_cu = 0;
    std::vector<StreamScratch> scratch;
    std::vector<StreamFork> forks;
    void* static_scratch = nullptr;     // address of the file-scope device array on this device (amr_lut_gemm_backward_static)
};
DeviceState g_dev[kMaxDevices];
std::mutex g_mu;
// what the library itself has taken from the runtime so far (amr_library_resources)
size_t g_allocated_bytes = 0;
int g_side_streams = 0;

// Number of compute units of the current device (cached).
int current_device_cus(int* dev_out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_dev[dev].n_cu == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return -1;
        g_dev[dev].n_cu = n;
    }
    if (dev_out) *dev_out = dev;
    return g_dev[dev].n_cu;
}

// Library-owned scratch of `stream` on device `dev`, at least `bytes` large.  Grows by allocation only (hipMalloc: not
// possible while the stream is being captured into a graph -- the first call of a given size has to happen before the
// capture, or the caller passes a workspace); never waits for the device and never frees.
void* internal_workspace(int dev, hipStream_t stream, size_t bytes, hipError_t* err) {
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceState& d = g_dev[dev];
    *err = hipSuccess;
    StreamScratch* slot = nullptr;
    for (StreamScratch& sc : d.scratch)
        if (sc.stream == stream) slot = &sc;
    if (slot && slot->bytes >= bytes) return slot->ptr;
    size_t want = bytes + bytes / 4;
    if (slot && want < 2 * slot->bytes) want = 2 * slot->bytes;    // geometric growth: all retired buffers together stay below the live one
    void* p = nullptr;
    *err = hipMalloc(&p, want);
    if (*err != hipSuccess) return nullptr;
    g_allocated_bytes += want;
    if (slot) { slot->ptr = p; slot->bytes = want; }               // the old buffer stays allocated (see above)
    else d.scratch.push_back({stream, p, want});
    return p;
}

// The side stream of `stream` on device `dev` (created on first use, default priority, kept until the process ends).
bool stream_fork(int dev, hipStream_t stream, StreamFork* out) {
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceState& d = g_dev[dev];
    for (const StreamFork& f : d.forks)
        if (f.stream == stream) { *out = f; return true; }
    StreamFork f{stream, nullptr, nullptr, nullptr};
    if (hipStreamCreateWithFlags(&f.side, hipStreamNonBlocking) != hipSuccess) return false;
    if (hipEventCreateWithFlags(&f.forked, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&f.joined, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    d.forks.push_back(f);
    ++g_side_streams;
    *out = f;
    return true;
}

}  // namespace

extern "C" {

int amr_version(void) { return 100; }
const char* amr_target_arch(void) { return "gfx950"; }
const char* amr_last_error(void) { return g_err; }

int amr_lut_geometry(int bits, int* rows, int* cols, int64_t* elem_num) {
    amr::LutGeom g;
    if (!amr::lut_geom_from_bits(bits, &g)) return fail(AMR_ELUTLEN, "quantization_bit = %d is not supported", bits);
    if (rows) *rows = g.rows;
    if (cols) *cols = g.cols;
    if (elem_num) *elem_num = g.elems;
    return AMR_OK;
}

// Process-wide switch (diagnostics, tests, benchmarks): 0 sends every call to the direct gather kernels, 1 picks by
// problem size, 2 takes the expanded-table kernels wherever the shape allows (also where they are slower).
static std::atomic<int> g_expanded_kernels{1};
// 1: small backward calls run gradB on a side stream beside gradA (amr_set_backward_fork)
static std::atomic<int> g_fork_small{1};

int amr_set_expanded_table_kernels(int mode) {
    return g_expanded_kernels.exchange(mode <= 0 ? 0 : (mode >= 2 ? 2 : 1));
}

int amr_set_backward_fork(int on) { return g_fork_small.exchange(on ? 1 : 0); }

void amr_library_resources(size_t* scratch_bytes, int* side_streams) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (scratch_bytes) *scratch_bytes = g_allocated_bytes;
    if (side_streams) *side_streams = g_side_streams;
}

int amr_bits_from_lut_elems(int64_t lut_elems) {
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "table length %lld matches no supported bit-width (1024, 5120, 17408, 66306)", (long long)lut_elems);
    return g.bits;
}

size_t amr_lut_gemm_forward_workspace_bytes(int64_t lut_elems, int M, int K, int N) {
    amr::LutGeom g;
    if (M <= 0 || K <= 0 || N <= 0 || !amr::lut_geom_from_elems(lut_elems, &g)) return 0;
    const int mode = g_expanded_kernels.load();
    return mode ? amr::fwd_slab_workspace_bytes(g, M, K, N, mode == 2) : 0;
}

}  // extern "C"

// Expansion of the forward table along one weight matrix, kept between calls (amr_fwd_cache_* in the header).
struct amr_fwd_cache {
    std::mutex mu;
    int dev = -1;
    void* buf = nullptr;        // [256 B header][E], as the forward workspace
    size_t bytes = 0;
    bool valid = false;
    uint64_t version = 0;
    const void* lut = nullptr;
    int64_t lut_elems = 0;
    int K = 0, N = 0;
    uint64_t hits = 0, misses = 0;
};

// Buffer of `need` bytes for the expansion of (version, lut, K, N); *hit says whether it already holds it.  A miss leaves the
// cache claiming the new contents: the caller expands into the buffer on its stream right away.
static void* fwd_cache_lookup(amr_fwd_cache* c, int dev, size_t need, uint64_t version, const void* lut, int64_t lut_elems, int K, int N,
                              bool* hit, hipError_t* err) {
    std::lock_guard<std::mutex> lk(c->mu);
    *err = hipSuccess;
    *hit = c->valid && c->dev == dev && c->bytes >= need && c->version == version && c->lut == lut && c->lut_elems == lut_elems &&
           c->K == K && c->N == N;
    if (*hit) { ++c->hits; return c->buf; }
    ++c->misses;
    if (c->dev != dev || c->bytes < need) {
        // (hipFree waits for the device: work queued on the old buffer has finished before it goes)
        if (c->buf) (void)hipFree(c->buf);
        c->buf = nullptr; c->bytes = 0; c->valid = false;
        *err = hipMalloc(&c->buf, need);
        if (*err != hipSuccess) { c->buf = nullptr; return nullptr; }
        c->bytes = need;
        c->dev = dev;
    }
    c->valid = true; c->version = version; c->lut = lut; c->lut_elems = lut_elems; c->K = K; c->N = N;
    return c->buf;
}

static void fwd_cache_forget(amr_fwd_cache* c) {
    std::lock_guard<std::mutex> lk(c->mu);
    c->valid = false;
}

extern "C" {

int amr_fwd_cache_create(amr_fwd_cache** out) {
    if (!out) return fail(AMR_EINVAL, "null pointer argument");
    *out = new (std::nothrow) amr_fwd_cache();
    return *out ? AMR_OK : fail(AMR_EINVAL, "out of host memory");
}

int amr_fwd_cache_destroy(amr_fwd_cache* c) {
    if (!c) return AMR_OK;
    if (c->buf) (void)hipFree(c->buf);
    delete c;
    return AMR_OK;
}

int amr_fwd_cache_stats(amr_fwd_cache* c, uint64_t* hits, uint64_t* misses, size_t* device_bytes) {
    if (!c) return fail(AMR_EINVAL, "null pointer argument");
    std::lock_guard<std::mutex> lk(c->mu);
    if (hits) *hits = c->hits;
    if (misses) *misses = c->misses;
    if (device_bytes) *device_bytes = c->bytes;
    return AMR_OK;
}

static int forward_impl(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, int64_t lut_elems, int M, int K, int N,
                        void* workspace, size_t workspace_bytes, void* stream, int out_f32, amr_fwd_cache* cache = nullptr,
                        uint64_t b_version = 0) {
    if (M < 0 || K < 0 || N < 0) return fail(AMR_EINVAL, "negative dimension M=%d K=%d N=%d", M, K, N);
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "lut size should be one of 1024/5120/17408/66306, got %lld", (long long)lut_elems);
    if (M == 0 || N == 0) return AMR_OK;
    if (!C || !lut || (K > 0 && (!A || !B))) return fail(AMR_EINVAL, "null pointer argument");
    if ((uintptr_t)lut & 3) return fail(AMR_EINVAL, "lut must be 4-byte aligned");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (K == 0) {
        hipError_t e = amr::launch_zero_u32(C, (size_t)M * N, s);
        return e == hipSuccess ? AMR_OK : hip_fail(e, "zero fill launch");
    }
    int dev = 0;
    const int n_cu = current_device_cus(&dev);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    const int mode = g_expanded_kernels.load();
    const size_t need = mode ? amr::fwd_slab_workspace_bytes(g, M, K, N, mode == 2) : 0;
    hipError_t e;
    if (need > 0) {
        void* ws = workspace;
        bool hit = false;
        if (cache) {
            ws = fwd_cache_lookup(cache, dev, need, b_version, lut, lut_elems, K, N, &hit, &e);
            if (!ws) return hip_fail(e, "cache hipMalloc");
        } else if (ws) {
            if (workspace_bytes < need) return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace_bytes, need);
            if ((uintptr_t)ws & 255) return fail(AMR_EINVAL, "workspace must be 256-byte aligned");
        } else {
            ws = internal_workspace(dev, s, need, &e);
            if (!ws) return hip_fail(e, "workspace hipMalloc");
        }
        e = amr::launch_fwd_slab(A, B, C, lut, g, M, K, N, n_cu, ws, s, out_f32, nullptr, hit ? 1 : 0);
        if (cache && e != hipSuccess) fwd_cache_forget(cache);      // (whether the expansion got there is unknown)
    } else {
        e = amr::launch_fwd(A, B, C, lut, g, M, K, N, n_cu, s, out_f32);
    }
    return e == hipSuccess ? AMR_OK : hip_fail(e, "forward launch");
}

size_t amr_lut_conv_forward_dequant_workspace_bytes(int64_t lut_elems, int M, int K, int N) {
    if (M <= 0 || N <= 0) return 0;
    // [the expanded table of the forward pass, if this shape takes it][float32 sums, M x N]
    const size_t e = (amr_lut_gemm_forward_workspace_bytes(lut_elems, M, K, N) + 255) & ~(size_t)255;
    return e + (size_t)M * N * sizeof(float);
}

int amr_lut_conv_forward_dequant_f32(const uint8_t* A, const uint8_t* B, const uint16_t* lut, int64_t lut_elems, int M, int K, int N,
                                     int positions, const float* x_sum, const float* w_resp, const float* taps, const float* z_a,
                                     const float* z_w, const float* s_a, const float* s_w, const float* bias, float* out,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    return amr_lut_conv_forward_dequant_cached_f32(nullptr, 0, A, B, lut, lut_elems, M, K, N, positions, x_sum, w_resp, taps, z_a, z_w, s_a,
                                                   s_w, bias, out, workspace, workspace_bytes, stream);
}

int amr_lut_conv_forward_dequant_cached_f32(amr_fwd_cache* cache, uint64_t b_version, const uint8_t* A, const uint8_t* B,
                                            const uint16_t* lut, int64_t lut_elems, int M, int K, int N, int positions,
                                            const float* x_sum, const float* w_resp, const float* taps, const float* z_a,
                                            const float* z_w, const float* s_a, const float* s_w, const float* bias, float* out,
                                            void* workspace, size_t workspace_bytes, void* stream) {
    if (M < 0 || K < 0 || N < 0) return fail(AMR_EINVAL, "negative dimension M=%d K=%d N=%d", M, K, N);
    if (positions <= 0 || M % positions != 0) return fail(AMR_EINVAL, "positions=%d must divide M=%d", positions, M);
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "lut size should be one of 1024/5120/17408/66306, got %lld", (long long)lut_elems);
    if (M == 0 || N == 0) return AMR_OK;
    if (!lut || (K > 0 && (!A || !B)) || !x_sum || !w_resp || !taps || !z_a || !z_w || !s_a || !s_w || !out)
        return fail(AMR_EINVAL, "null pointer argument");
    if ((uintptr_t)lut & 3) return fail(AMR_EINVAL, "lut must be 4-byte aligned");
    const size_t need = amr_lut_conv_forward_dequant_workspace_bytes(lut_elems, M, K, N);
    if (!workspace || workspace_bytes < need)
        return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace ? workspace_bytes : (size_t)0, need);
    if ((uintptr_t)workspace & 255) return fail(AMR_EINVAL, "workspace must be 256-byte aligned");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int dev = 0;
    const int n_cu = current_device_cus(&dev);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    const size_t e_bytes = need - (size_t)M * N * sizeof(float);
    float* sums = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(workspace) + e_bytes);
    const int mode = g_expanded_kernels.load();
    hipError_t e;
    if (K > 0 && mode && e_bytes && amr::fwd_slab_can_dequant(g, M, K, N, n_cu, mode == 2)) {
        // one launch stores the activation; `sums` is touched by the gated fall-back only
        const amr::SlabDequant dq{x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out, positions};
        void* e_buf = workspace;
        bool hit = false;
        if (cache) {
            e_buf = fwd_cache_lookup(cache, dev, amr::fwd_slab_workspace_bytes(g, M, K, N, mode == 2), b_version, lut, lut_elems, K, N, &hit, &e);
            if (!e_buf) return hip_fail(e, "cache hipMalloc");
        }
        e = amr::launch_fwd_slab(A, B, reinterpret_cast<uint32_t*>(sums), lut, g, M, K, N, n_cu, e_buf, s, 1, &dq, hit ? 1 : 0);
        if (cache && e != hipSuccess) fwd_cache_forget(cache);
        return e == hipSuccess ? AMR_OK : hip_fail(e, "forward launch");
    }
    // K split over workgroups, small problems, direct kernels: the sums meet in memory first, a second pass dequantises them
    const int rc = forward_impl(A, B, reinterpret_cast<uint32_t*>(sums), lut, lut_elems, M, K, N, e_bytes ? workspace : nullptr, e_bytes, stream, 1,
                                cache, b_version);
    if (rc != AMR_OK) return rc;
    e = amr::launch_dequant(sums, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out, M, N, positions, s);
    return e == hipSuccess ? AMR_OK : hip_fail(e, "dequant launch");
}

int amr_lut_conv_forward_implicit_supported(int64_t lut_elems, int B, int C, int H, int W, int N) {
    amr::LutGeom g;
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || N <= 0 || !amr::lut_geom_from_elems(lut_elems, &g)) return 0;
    const int mode = g_expanded_kernels.load();
    const int n_cu = current_device_cus(nullptr);
    const long M = (long)B * H * W;
    if (!mode || (double)M * 9 * C >= 2147483648.0) return 0;
    return amr::fwd_slab_conv_applies(g, M, C, N, n_cu > 0 ? n_cu : 256, mode == 2) ? 1 : 0;
}

size_t amr_lut_conv_forward_implicit_workspace_bytes(int64_t lut_elems, int B, int C, int H, int W, int N, int cached, int with_fallback) {
    if (!amr_lut_conv_forward_implicit_supported(lut_elems, B, C, H, W, N)) return 0;
    const int M = B * H * W;
    const size_t e = cached ? 0 : (amr_lut_gemm_forward_workspace_bytes(lut_elems, M, 9 * C, N) + 255) & ~(size_t)255;
    return e + (with_fallback ? (size_t)M * N * sizeof(float) : 0);
}

int amr_lut_conv_forward_implicit_f32(amr_fwd_cache* cache, uint64_t b_version, const uint8_t* codes, const uint8_t* Bt,
                                      const uint16_t* lut, int64_t lut_elems, int B, int C, int H, int W, int N, const float* x_sum,
                                      const float* w_resp, const float* taps, const float* z_a, const float* z_w, const float* s_a,
                                      const float* s_w, const float* bias, float* out, const uint8_t* A_fallback, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "lut size should be one of 1024/5120/17408/66306, got %lld", (long long)lut_elems);
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || N <= 0) return fail(AMR_EINVAL, "bad shape B=%d C=%d H=%d W=%d N=%d", B, C, H, W, N);
    if (!amr_lut_conv_forward_implicit_supported(lut_elems, B, C, H, W, N))
        return fail(AMR_EUNSUPPORTED, "shape or table not served by the convolution-shaped forward kernel (ask amr_lut_conv_forward_implicit_supported)");
    if (!codes || !Bt || !lut || !x_sum || !w_resp || !taps || !z_a || !z_w || !s_a || !s_w || !out) return fail(AMR_EINVAL, "null pointer argument");
    if (((uintptr_t)lut & 3) || ((uintptr_t)codes & 15)) return fail(AMR_EINVAL, "lut must be 4-byte and codes 16-byte aligned");
    const size_t need = amr_lut_conv_forward_implicit_workspace_bytes(lut_elems, B, C, H, W, N, cache ? 1 : 0, A_fallback ? 1 : 0);
    if (need && (!workspace || workspace_bytes < need))
        return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace ? workspace_bytes : (size_t)0, need);
    if (need && ((uintptr_t)workspace & 255)) return fail(AMR_EINVAL, "workspace must be 256-byte aligned");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int dev = 0;
    const int n_cu = current_device_cus(&dev);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    const int M = B * H * W, K = 9 * C;
    const int mode = g_expanded_kernels.load();
    const size_t e_bytes = cache ? 0 : (amr_lut_gemm_forward_workspace_bytes(lut_elems, M, K, N) + 255) & ~(size_t)255;
    float* sums = A_fallback ? reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(workspace) + e_bytes) : nullptr;
    const amr::SlabDequant dq{x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out, H * W};
    const amr::SlabConv cv{nullptr, C, H, W};
    void* e_buf = workspace;
    bool hit = false;
    hipError_t e;
    if (cache) {
        e_buf = fwd_cache_lookup(cache, dev, amr::fwd_slab_workspace_bytes(g, M, K, N, mode == 2), b_version, lut, lut_elems, K, N, &hit, &e);
        if (!e_buf) return hip_fail(e, "cache hipMalloc");
    }
    e = amr::launch_fwd_slab(codes, Bt, reinterpret_cast<uint32_t*>(sums), lut, g, M, K, N, n_cu, e_buf, s, 1, &dq, hit ? 1 : 0, &cv, A_fallback);
    if (cache && e != hipSuccess) fwd_cache_forget(cache);
    return e == hipSuccess ? AMR_OK : hip_fail(e, "forward launch");
}

int amr_lut_gemm_forward_ws(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, int64_t lut_elems,
                            int M, int K, int N, void* workspace, size_t workspace_bytes, void* stream) {
    return forward_impl(A, B, C, lut, lut_elems, M, K, N, workspace, workspace_bytes, stream, 0);
}

int amr_lut_gemm_forward_f32_ws(const uint8_t* A, const uint8_t* B, float* C, const uint16_t* lut, int64_t lut_elems,
                                int M, int K, int N, void* workspace, size_t workspace_bytes, void* stream) {
    // (a zero of either type has the same bits: the empty sums of K == 0 need no conversion)
    return forward_impl(A, B, reinterpret_cast<uint32_t*>(C), lut, lut_elems, M, K, N, workspace, workspace_bytes, stream, 1);
}

int amr_lut_gemm_forward_cached(amr_fwd_cache* cache, uint64_t b_version, const uint8_t* A, const uint8_t* B, void* C, int c_is_f32,
                                const uint16_t* lut, int64_t lut_elems, int M, int K, int N, void* stream) {
    if (!cache) return fail(AMR_EINVAL, "null cache");
    return forward_impl(A, B, reinterpret_cast<uint32_t*>(C), lut, lut_elems, M, K, N, nullptr, 0, stream, c_is_f32 ? 1 : 0, cache, b_version);
}

int amr_lut_gemm_forward(const uint8_t* A, const uint8_t* B, uint32_t* C, const uint16_t* lut, int64_t lut_elems,
                         int M, int K, int N, void* stream) {
    return amr_lut_gemm_forward_ws(A, B, C, lut, lut_elems, M, K, N, nullptr, 0, stream);
}

// Scratch layout of the backward pass: [256 B of flags][partial sums of gB over the M splits][expanded
// gradient table of gradA]; each part a multiple of 256 bytes.
static size_t backward_partial_bytes(int M, int K, int N, int n_cu) {
    size_t direct = amr::gradB_workspace_bytes(M, K, N, n_cu);
    const int s7 = amr::gradB_slab_splits(M, K, N, n_cu), s8 = amr::gradB_slab8_splits(M, K, N, n_cu),
              s8f = amr::gradB_slab8f_splits(M, K, N, n_cu);
    const int s = s7 > s8 ? (s7 > s8f ? s7 : s8f) : (s8 > s8f ? s8 : s8f);
    size_t slab = (s > 1 ? (size_t)s * K * N * sizeof(float) : 0) + amr::gradB_slab_colsum_floats(N) * sizeof(float);
    const size_t b = direct > slab ? direct : slab;
    return (b + 255) & ~(size_t)255;
}

// Size of the expanded table of gradA.  bits == 0: the table width is not known (a query by shape alone), so the scratch
// is sized for the larger of the 7-bit and the 8-bit expanded table.
static size_t backward_gradA_bytes(int mode, int bits, int M, int K, int N) {
    if (!mode) return 0;
    amr::LutGeom g7, g8;
    amr::lut_geom_from_bits(bits && bits < 8 ? bits : 7, &g7);
    amr::lut_geom_from_bits(8, &g8);
    const size_t b7 = bits == 8 ? 0 : amr::gradA_slab_workspace_bytes(g7, M, K, N, mode == 2);
    size_t b8 = 0;
    if (bits == 0 || bits == 8) {
        // (a layer takes one of the two: partial results of the kernel with the table in LDS, or the expanded table)
        const size_t rows8 = amr::gradA_rows8_workspace_bytes(g8, M, K, N, mode == 2);
        b8 = rows8 ? rows8 : amr::gradA_slab_i16_workspace_bytes(g8, M, K, N, mode == 2);
    }
    return b7 > b8 ? b7 : b8;
}

size_t amr_lut_gemm_backward_workspace_bytes(int M, int K, int N) {
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    const int n_cu = current_device_cus(nullptr);
    // Without a device (e.g. a host-only query) size for a 256-CU part.
    return 256 + backward_partial_bytes(M, K, N, n_cu > 0 ? n_cu : 256) + backward_gradA_bytes(g_expanded_kernels.load(), 0, M, K, N);
}

size_t amr_lut_gemm_backward_workspace_bytes_for(int64_t lut_elems, int M, int K, int N) {
    amr::LutGeom g;
    if (M <= 0 || K <= 0 || N <= 0 || !amr::lut_geom_from_elems(lut_elems, &g)) return 0;
    const int n_cu = current_device_cus(nullptr);
    return 256 + backward_partial_bytes(M, K, N, n_cu > 0 ? n_cu : 256) + backward_gradA_bytes(g_expanded_kernels.load(), g.bits, M, K, N);
}

int amr_lut_gemm_backward(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, float* gB,
                          const int16_t* lut_grad_a, const int16_t* lut_grad_b, int64_t lut_elems, int M, int K,
                          int N, void* workspace, size_t workspace_bytes, void* stream) {
    return amr_lut_gemm_backward_ex(gC, A, B, gA, gB, lut_grad_a, lut_grad_b, lut_elems, M, K, N, 0, workspace,
                                    workspace_bytes, stream);
}

// File-scope scratch of amr_lut_gemm_backward_static: every device the library runs on holds its own copy until the
// process ends.  Host code never uses the array's name as an address: static_scratch_ptr() asks the runtime once per
// device where that device's copy lives.
constexpr size_t kStaticScratchBytes = (size_t)AMR_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static void* static_scratch_ptr(int dev, hipError_t* err) {
    std::lock_guard<std::mutex> lk(g_mu);
    *err = hipSuccess;
    if (!g_dev[dev].static_scratch) {
        void* p = nullptr;
        *err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));     // (the caller's device `dev` is current)
        if (*err != hipSuccess) return nullptr;
        g_dev[dev].static_scratch = p;
    }
    return g_dev[dev].static_scratch;
}

// where the scratch of a backward call comes from
enum class ScratchFrom { Caller, Library, Static };

static int backward_impl(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, float* gB,
                         const int16_t* lut_grad_a, const int16_t* lut_grad_b, int64_t lut_elems, int M, int K,
                         int N, int ga_rows_per_image, ScratchFrom from, void* workspace, size_t workspace_bytes, void* stream) {
    if (ga_rows_per_image < 0 || (ga_rows_per_image > 0 && M % ga_rows_per_image != 0))
        return fail(AMR_EINVAL, "ga_rows_per_image=%d must divide M=%d", ga_rows_per_image, M);
    if (M < 0 || K < 0 || N < 0) return fail(AMR_EINVAL, "negative dimension M=%d K=%d N=%d", M, K, N);
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "lut size should be one of 1024/5120/17408/66306, got %lld", (long long)lut_elems);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const float scale = 1.0f / 16.0f;  // FACTOR, self_ops/src/approx_mult.h:41
    if (gA && !lut_grad_a) return fail(AMR_EINVAL, "lut_grad_a is null");
    if (gB && !lut_grad_b) return fail(AMR_EINVAL, "lut_grad_b is null");
    if (((uintptr_t)lut_grad_a & 3) || ((uintptr_t)lut_grad_b & 3)) return fail(AMR_EINVAL, "gradient tables must be 4-byte aligned");
    // Degenerate reductions: an empty sum is zero.
    if (M == 0 || K == 0 || N == 0) {
        hipError_t e = hipSuccess;
        if (gA && (size_t)M * K) e = amr::launch_zero_u32(gA, (size_t)M * K, s);
        if (e == hipSuccess && gB && (size_t)K * N) e = amr::launch_zero_u32(gB, (size_t)K * N, s);
        return e == hipSuccess ? AMR_OK : hip_fail(e, "zero fill launch");
    }
    if (!gC || !A || !B) return fail(AMR_EINVAL, "null pointer argument");
    if (!gA && !gB) return AMR_OK;
    int dev = 0;
    const int n_cu = current_device_cus(&dev);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    hipError_t e;
    const int mode = g_expanded_kernels.load();
    size_t partial_bytes = backward_partial_bytes(M, K, N, n_cu);
    // (what this table width needs: never more than the shape-only query answers)
    size_t gradA_bytes = backward_gradA_bytes(mode, g.bits, M, K, N);
    bool allow_slab_a = true;
    int split_cap = 0;
    void* ws = workspace;
    const bool slab = mode && amr::bwd_slab_applies(g, M, K, N);
    const bool slab_b8 = !slab && mode && amr::gradB_slab8_applies(g, M, K, N, gC, mode == 2);
    if (from == ScratchFrom::Static) {
        // The array is sized for the kernels this call will launch, not for the largest any width could take: gradB splits
        // M as far as the array has room for partial sums (down to no split at all, which needs none), gradA keeps its
        // expanded table if that still fits behind them and runs on the direct kernel otherwise.
        const size_t per_split = (size_t)K * N * sizeof(float);
        const size_t colsum = (gB && slab) ? amr::gradB_slab_colsum_floats(N) * sizeof(float) : 0;
        if (256 + colsum + 256 > kStaticScratchBytes)
            return fail(AMR_EWORKSPACE, "N = %d needs %zu bytes of column sums, the static scratch holds %zu: use amr_lut_gemm_backward with a workspace",
                        N, colsum, kStaticScratchBytes);
        int want = !gB ? 1 : slab ? amr::gradB_slab_splits(M, K, N, n_cu) : slab_b8 ? amr::gradB_slab8_splits(M, K, N, n_cu)
                                                                                   : amr::gradB_direct_splits_for(g, M, K, N, n_cu);
        const size_t room = kStaticScratchBytes - 256 - colsum - 256;
        // (half the array at most for partial sums while gradA has an expanded table to place behind them)
        size_t cap = room / per_split;
        if (gA && gradA_bytes && gradA_bytes < room && (room - gradA_bytes) / per_split >= 2) cap = (room - gradA_bytes) / per_split;
        if (cap < 1) cap = 1;
        if ((size_t)want > cap) want = (int)cap;
        split_cap = (int)cap;
        partial_bytes = (colsum + (want > 1 ? (size_t)want * per_split : 0) + 255) & ~(size_t)255;
        if (256 + partial_bytes + gradA_bytes > kStaticScratchBytes) {   // gradA without its expanded table (direct kernel)
            gradA_bytes = 0;
            allow_slab_a = false;
        }
        ws = static_scratch_ptr(dev, &e);
        if (!ws) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    }
    const size_t need = 256 + partial_bytes + gradA_bytes;
    if (from == ScratchFrom::Caller) {
        if (workspace_bytes < need) return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace_bytes, need);
        if ((uintptr_t)ws & 255) return fail(AMR_EINVAL, "workspace must be 256-byte aligned");
    } else if (from == ScratchFrom::Library) {
        ws = internal_workspace(dev, s, need, &e);
        if (!ws) return hip_fail(e, "workspace hipMalloc");
    }
    uint32_t* flags = reinterpret_cast<uint32_t*>(ws);
    float* partials = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(ws) + 256);
    const bool slab_a = mode && allow_slab_a && gA && amr::gradA_slab_workspace_bytes(g, M, K, N, mode == 2) != 0 && ((uintptr_t)gC & 15) == 0;
    // (8-bit tables: the expanded table holds the int16 entries, nothing to decide in a header)
    // (or, for layers of a few thousand rows, none at all: the table is expanded in LDS and the scratch holds partial results)
    const bool rows_a8 = mode && allow_slab_a && gA && amr::gradA_rows8_applies(g, M, K, N, gC, mode == 2);
    const bool slab_a8 = !rows_a8 && mode && allow_slab_a && gA && amr::gradA_slab_i16_workspace_bytes(g, M, K, N, mode == 2) != 0 && ((uintptr_t)gC & 15) == 0;
    if ((slab && gB) || slab_a) {
        // flags cleared, offsets of the half-precision tables decided from the tables' extremes
        e = amr::launch_bwd_header(slab_a ? lut_grad_a : nullptr, (slab && gB) ? lut_grad_b : nullptr, g, flags, s);
        if (e != hipSuccess) return hip_fail(e, "scratch header launch");
    }
    // Small problems are bound by the latency of their launches (three or four dependent ones per gradient), not by
    // arithmetic: the launches of gradB then go to a side stream and run beside those of gradA (the two gradients share
    // inputs only; their parts of the scratch are disjoint), and the caller's stream waits for the side stream before
    // the call returns, so that everything stays ordered with the caller's stream.
    hipStream_t sb = s;
    StreamFork fork{};
    const bool forked = gA && gB && from != ScratchFrom::Static && (double)M * K * N < 2.0e9 && g_fork_small.load() &&
                        stream_fork(dev, s, &fork);
    if (forked) {
        if ((e = hipEventRecord(fork.forked, s)) != hipSuccess || (e = hipStreamWaitEvent(fork.side, fork.forked, 0)) != hipSuccess)
            return hip_fail(e, "side stream fork");
        sb = fork.side;
    }
    if (gA) {
        if (slab_a)
            e = amr::launch_gradA_slab(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu, flags,
                                       reinterpret_cast<unsigned char*>(ws) + 256 + partial_bytes, ga_rows_per_image, s);
        else if (rows_a8)
            e = amr::launch_gradA_rows8(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu,
                                        reinterpret_cast<unsigned char*>(ws) + 256 + partial_bytes, gradA_bytes, ga_rows_per_image, s);
        else if (slab_a8)
            e = amr::launch_gradA_slab_i16(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu, flags,
                                           reinterpret_cast<unsigned char*>(ws) + 256 + partial_bytes, ga_rows_per_image, s);
        else
            e = amr::launch_gradA(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu, s, nullptr, ga_rows_per_image);
    }
    hipError_t eb = hipSuccess;
    if (gB) {     // (queued also when the gradA launch failed: a forked side stream must be joined again either way)
        if (slab) {
            eb = amr::launch_gradB_slab(gC, A, B, gB, lut_grad_b, g, M, K, N, scale, flags, partials, n_cu, sb, split_cap);
        } else if (slab_b8) {
            eb = amr::launch_gradB_slab8(gC, A, B, gB, lut_grad_b, g, M, K, N, scale, partials, n_cu, sb, split_cap);
        } else {
            eb = amr::launch_gradB(gC, A, B, gB, lut_grad_b, g, M, K, N, scale, partials, n_cu, sb, nullptr, split_cap);
        }
    }
    if (forked) {
        hipError_t ej;
        if ((ej = hipEventRecord(fork.joined, fork.side)) != hipSuccess || (ej = hipStreamWaitEvent(s, fork.joined, 0)) != hipSuccess)
            return hip_fail(ej, "side stream join");
    }
    if (gA && e != hipSuccess) return hip_fail(e, "gradA launch");
    if (eb != hipSuccess) return hip_fail(eb, "gradB launch");
    return AMR_OK;
}

int amr_lut_gemm_backward_ex(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, float* gB,
                             const int16_t* lut_grad_a, const int16_t* lut_grad_b, int64_t lut_elems, int M, int K,
                             int N, int ga_rows_per_image, void* workspace, size_t workspace_bytes, void* stream) {
    return backward_impl(gC, A, B, gA, gB, lut_grad_a, lut_grad_b, lut_elems, M, K, N, ga_rows_per_image,
                         workspace ? ScratchFrom::Caller : ScratchFrom::Library, workspace, workspace_bytes, stream);
}

size_t amr_static_scratch_bytes(void) { return kStaticScratchBytes; }

int amr_lut_gemm_backward_static(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, float* gB,
                                 const int16_t* lut_grad_a, const int16_t* lut_grad_b, int64_t lut_elems, int M, int K,
                                 int N, int ga_rows_per_image, void* stream) {
    return backward_impl(gC, A, B, gA, gB, lut_grad_a, lut_grad_b, lut_elems, M, K, N, ga_rows_per_image, ScratchFrom::Static,
                         nullptr, 0, stream);
}

// Scratch of the float-table backward pass: [256 B of flags][partial sums of gB][float32 expanded table of gradA].
static size_t backward_gradA_f32_bytes(int mode, int bits, int M, int K, int N) {
    if (!mode) return 0;
    // (bits == 0: a query by shape alone, answered for the larger of the 7-bit and the 8-bit expanded table)
    amr::LutGeom g7, g8;
    amr::lut_geom_from_bits(bits && bits < 8 ? bits : 7, &g7);
    amr::lut_geom_from_bits(8, &g8);
    const size_t b7 = bits == 8 ? 0 : amr::gradA_slab_f32_workspace_bytes(g7, M, K, N, mode == 2);
    size_t b8 = 0;
    if (bits == 0 || bits == 8) {
        const size_t rows8 = amr::gradA_rows8f_workspace_bytes(g8, M, K, N, mode == 2);
        b8 = rows8 ? rows8 : amr::gradA_slab_f32w_workspace_bytes(g8, M, K, N, mode == 2);
    }
    return b7 > b8 ? b7 : b8;
}

size_t amr_lut_gemm_backward_f32tab_workspace_bytes(int M, int K, int N) {
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    const int n_cu = current_device_cus(nullptr);
    return 256 + backward_partial_bytes(M, K, N, n_cu > 0 ? n_cu : 256) + backward_gradA_f32_bytes(g_expanded_kernels.load(), 0, M, K, N);
}

size_t amr_lut_gemm_backward_f32tab_workspace_bytes_for(int64_t lut_elems, int M, int K, int N) {
    amr::LutGeom g;
    if (M <= 0 || K <= 0 || N <= 0 || !amr::lut_geom_from_elems(lut_elems, &g)) return 0;
    const int n_cu = current_device_cus(nullptr);
    return 256 + backward_partial_bytes(M, K, N, n_cu > 0 ? n_cu : 256) + backward_gradA_f32_bytes(g_expanded_kernels.load(), g.bits, M, K, N);
}

int amr_lut_gemm_backward_f32tab(const float* gC, const uint8_t* A, const uint8_t* B, float* gA, float* gB,
                                 const float* lut_grad_a, const float* lut_grad_b, int64_t lut_elems, float scale, int M, int K,
                                 int N, int ga_rows_per_image, void* workspace, size_t workspace_bytes, void* stream) {
    if (ga_rows_per_image < 0 || (ga_rows_per_image > 0 && M % ga_rows_per_image != 0))
        return fail(AMR_EINVAL, "ga_rows_per_image=%d must divide M=%d", ga_rows_per_image, M);
    if (M < 0 || K < 0 || N < 0) return fail(AMR_EINVAL, "negative dimension M=%d K=%d N=%d", M, K, N);
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "lut size should be one of 1024/5120/17408/66306, got %lld", (long long)lut_elems);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (gA && !lut_grad_a) return fail(AMR_EINVAL, "lut_grad_a is null");
    if (gB && !lut_grad_b) return fail(AMR_EINVAL, "lut_grad_b is null");
    if (((uintptr_t)lut_grad_a & 3) || ((uintptr_t)lut_grad_b & 3)) return fail(AMR_EINVAL, "gradient tables must be 4-byte aligned");
    if (M == 0 || K == 0 || N == 0) {   // an empty sum is zero
        hipError_t e = hipSuccess;
        if (gA && (size_t)M * K) e = amr::launch_zero_u32(gA, (size_t)M * K, s);
        if (e == hipSuccess && gB && (size_t)K * N) e = amr::launch_zero_u32(gB, (size_t)K * N, s);
        return e == hipSuccess ? AMR_OK : hip_fail(e, "zero fill launch");
    }
    if (!gC || !A || !B) return fail(AMR_EINVAL, "null pointer argument");
    if (!gA && !gB) return AMR_OK;
    int dev = 0;
    const int n_cu = current_device_cus(&dev);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    hipError_t e;
    const size_t partial_bytes = backward_partial_bytes(M, K, N, n_cu);
    const int mode = g_expanded_kernels.load();
    const size_t need = 256 + partial_bytes + backward_gradA_f32_bytes(mode, g.bits, M, K, N);
    void* ws = workspace;
    if (ws) {
        if (workspace_bytes < need) return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace_bytes, need);
        if ((uintptr_t)ws & 255) return fail(AMR_EINVAL, "workspace must be 256-byte aligned");
    } else {
        ws = internal_workspace(dev, s, need, &e);
        if (!ws) return hip_fail(e, "workspace hipMalloc");
    }
    uint32_t* flags = reinterpret_cast<uint32_t*>(ws);
    float* partials = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(ws) + 256);
    const bool slab_b = mode && gB && amr::bwd_slab_applies(g, M, K, N);
    const bool slab_a = mode && gA && amr::gradA_slab_f32_workspace_bytes(g, M, K, N, mode == 2) != 0 &&
                        ((uintptr_t)gC & 15) == 0;
    const bool rows_a8 = mode && gA && amr::gradA_rows8f_applies(g, M, K, N, gC, mode == 2);
    const bool slab_a8 = !rows_a8 && mode && gA && amr::gradA_slab_f32w_workspace_bytes(g, M, K, N, mode == 2) != 0 &&
                         ((uintptr_t)gC & 15) == 0;
    if (slab_a || slab_b) {
        e = amr::launch_zero_u32(flags, 64, s);
        if (e != hipSuccess) return hip_fail(e, "scratch header launch");
    }
    if (gA) {
        if (slab_a)
            e = amr::launch_gradA_slab_f32tab(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu, flags,
                                              reinterpret_cast<unsigned char*>(ws) + 256 + partial_bytes, ga_rows_per_image, s);
        else if (rows_a8)
            e = amr::launch_gradA_rows8f(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu,
                                         reinterpret_cast<unsigned char*>(ws) + 256 + partial_bytes,
                                         backward_gradA_f32_bytes(mode, g.bits, M, K, N), ga_rows_per_image, s);
        else if (slab_a8)
            e = amr::launch_gradA_slab_f32w(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu, flags,
                                            reinterpret_cast<unsigned char*>(ws) + 256 + partial_bytes, ga_rows_per_image, s);
        else
            e = amr::launch_gradA_f32tab(gC, A, B, gA, lut_grad_a, g, M, K, N, scale, n_cu, s, nullptr, ga_rows_per_image);
        if (e != hipSuccess) return hip_fail(e, "gradA launch");
    }
    if (gB) {
        if (slab_b) {
            e = amr::launch_gradB_slab_f32tab(gC, A, B, gB, lut_grad_b, g, M, K, N, scale, flags, partials, n_cu, s);
        } else if (mode && amr::gradB_slab8f_applies(g, M, K, N, gC, mode == 2)) {
            e = amr::launch_gradB_slab8f(gC, A, B, gB, lut_grad_b, g, M, K, N, scale, partials, n_cu, s);
        } else {
            e = amr::launch_gradB_f32tab(gC, A, B, gB, lut_grad_b, g, M, K, N, scale, partials, n_cu, s, nullptr);
        }
        if (e != hipSuccess) return hip_fail(e, "gradB launch");
    }
    return AMR_OK;
}

int amr_im2col_u8_f32(const float* x, uint8_t* A, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil,
                      void* stream) {
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || pad < 0 || dil <= 0)
        return fail(AMR_EINVAL, "bad convolution geometry");
    const int oh = (H + 2 * pad - dil * (kh - 1) - 1) / stride + 1;
    const int ow = (W + 2 * pad - dil * (kw - 1) - 1) / stride + 1;
    if (oh <= 0 || ow <= 0) return fail(AMR_EINVAL, "empty convolution output");
    if (B == 0) return AMR_OK;
    if ((long)B * oh * ow >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 output positions");
    if (!x || !A) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_im2col_u8_f32(x, A, B, C, H, W, kh, kw, stride, pad, dil, oh, ow, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "im2col launch");
}

int amr_col2im_f32(const float* cols, float* x, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil,
                   void* stream) {
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || pad < 0 || dil <= 0)
        return fail(AMR_EINVAL, "bad convolution geometry");
    const int oh = (H + 2 * pad - dil * (kh - 1) - 1) / stride + 1;
    const int ow = (W + 2 * pad - dil * (kw - 1) - 1) / stride + 1;
    if (oh <= 0 || ow <= 0) return fail(AMR_EINVAL, "empty convolution output");
    if (B == 0) return AMR_OK;
    if ((size_t)B * C * H * W >= ((size_t)1 << 40)) return fail(AMR_EUNSUPPORTED, "more than 2^40 pixels");
    if (!cols || !x) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_col2im_f32(cols, x, B, C, H, W, kh, kw, stride, pad, dil, oh, ow, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "col2im launch");
}

int amr_conv_dequant_f32(const float* c, const float* x_sum, const float* w_resp, const float* taps, const float* z_a,
                         const float* z_w, const float* s_a, const float* s_w, const float* bias, float* out, int batch,
                         int out_channels, int positions, void* stream) {
    if (batch < 0 || out_channels <= 0 || positions <= 0) return fail(AMR_EINVAL, "bad shape");
    if (batch == 0) return AMR_OK;
    if ((long)batch * positions >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 output positions");
    if (!c || !x_sum || !w_resp || !taps || !z_a || !z_w || !s_a || !s_w || !out) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_dequant(c, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out, batch * positions, out_channels, positions,
                                       reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "dequant launch");
}

int amr_conv_dequant_backward_f32(const float* g, const float* s_a, const float* s_w, float* g_c, int batch, int out_channels,
                                  int positions, void* stream) {
    if (batch < 0 || out_channels <= 0 || positions <= 0) return fail(AMR_EINVAL, "bad shape");
    if (batch == 0) return AMR_OK;
    if ((long)batch * positions >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 output positions");
    if (!g || !s_a || !s_w || !g_c) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_dequant_grad(g, s_a, s_w, g_c, batch * positions, out_channels, positions, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "dequant backward launch");
}

int amr_observer_update_f32(const float* cur_min, const float* cur_max, float* min_val, float* max_val, float* scale,
                            float* zp_neg, int mode, float keep, float momentum, float quant_max, float inv_quant_max, float eps,
                            void* stream) {
    if (mode < 0 || mode > 2 || !(quant_max > 0.f)) return fail(AMR_EINVAL, "bad observer mode or code range");
    if (!cur_min || !cur_max || !min_val || !max_val || !scale || !zp_neg) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_observer_update(cur_min, cur_max, min_val, max_val, scale, zp_neg, mode, keep, momentum, quant_max, inv_quant_max, eps,
                                               reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "observer update launch");
}

int amr_observe_minmax_f32(const float* x, int64_t n, uint32_t* state, float* min_val, float* max_val, float* scale, float* zp_neg,
                           int mode, float keep, float momentum, float quant_max, float inv_quant_max, float eps, void* stream) {
    if (mode < 0 || (mode & 3) > 2 || mode > 7 || !(quant_max > 0.f) || n <= 0)
        return fail(AMR_EINVAL, "bad observer mode, code range or element count");
    if (!x || !state || !min_val || !max_val || !scale || !zp_neg) return fail(AMR_EINVAL, "null pointer argument");
    if ((uintptr_t)state & 3) return fail(AMR_EINVAL, "state must be 4-byte aligned");
    const int n_cu = current_device_cus(nullptr);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    hipError_t e = amr::launch_observe_minmax(x, (size_t)n, state, min_val, max_val, scale, zp_neg, mode, keep, momentum, quant_max,
                                              inv_quant_max, eps, n_cu, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "observer launch");
}

int amr_quantize_codes_f32(const float* x, const float* scale, const float* zp_neg, float qmax, float* codes, int64_t n,
                           void* stream) {
    if (n < 0 || !(qmax >= 0.f)) return fail(AMR_EINVAL, "bad element count or code range");
    if (n == 0) return AMR_OK;
    if (n >= ((int64_t)1 << 40)) return fail(AMR_EUNSUPPORTED, "more than 2^40 elements");
    if (!x || !scale || !zp_neg || !codes) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_quantize_codes(x, scale, zp_neg, qmax, codes, (size_t)n, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "quantize launch");
}

int amr_quantize_codes_backward_f32(const float* g, const float* x, const float* scale, const float* zp_neg, float qmax,
                                    float* gx, int64_t n, void* stream) {
    if (n < 0 || !(qmax >= 0.f)) return fail(AMR_EINVAL, "bad element count or code range");
    if (n == 0) return AMR_OK;
    if (n >= ((int64_t)1 << 40)) return fail(AMR_EUNSUPPORTED, "more than 2^40 elements");
    if (!g || !x || !scale || !zp_neg || !gx) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_quantize_codes_backward(g, x, scale, zp_neg, qmax, gx, (size_t)n, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "quantize backward launch");
}

static bool conv_geometry(int C, int H, int W, int kh, int kw, int stride, int pad, int dil, int* oh, int* ow) {
    if (C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || pad < 0 || dil <= 0) return false;
    *oh = (H + 2 * pad - dil * (kh - 1) - 1) / stride + 1;
    *ow = (W + 2 * pad - dil * (kw - 1) - 1) / stride + 1;
    return *oh > 0 && *ow > 0;
}

int amr_quantize_codes_nhwc_u8(const float* x, const float* scale, const float* zp_neg, float qmax, uint8_t* codes, uint8_t* inside,
                               float* x_sum, int B, int C, int L, void* stream) {
    return amr_quantize_codes_nhwc_relu_u8(x, scale, zp_neg, qmax, codes, inside, x_sum, B, C, L, 0, stream);
}

int amr_quantize_codes_nhwc_relu_u8(const float* x, const float* scale, const float* zp_neg, float qmax, uint8_t* codes, uint8_t* inside,
                                    float* x_sum, int B, int C, int L, int relu, void* stream) {
    if (B < 0 || C <= 0 || L <= 0 || !(qmax >= 0.f) || qmax > 255.f) return fail(AMR_EINVAL, "bad shape or code range");
    if (B == 0) return AMR_OK;
    if ((long)B * L >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 pixels");
    if (!x || !scale || !zp_neg || !codes || !inside || !x_sum) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_quantize_nhwc(x, scale, zp_neg, qmax, codes, inside, x_sum, B, C, L, reinterpret_cast<hipStream_t>(stream),
                                             relu ? 1 : 0);
    return e == hipSuccess ? AMR_OK : hip_fail(e, "quantize launch");
}

int amr_im2col_nhwc_u8(const uint8_t* codes, uint8_t* A, int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil,
                       void* stream) {
    int oh, ow;
    if (B < 0 || !conv_geometry(C, H, W, kh, kw, stride, pad, dil, &oh, &ow)) return fail(AMR_EINVAL, "bad convolution geometry");
    if (B == 0) return AMR_OK;
    if ((long)B * oh * ow >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 output positions");
    if (!codes || !A) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_im2col_nhwc(codes, A, B, C, H, W, kh, kw, stride, pad, dil, oh, ow, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "im2col launch");
}

int amr_conv_input_grad_f32(const float* cols, const float* t, const float* z_w, const uint8_t* inside, const float* scale, float* gx,
                            int B, int C, int H, int W, int kh, int kw, int stride, int pad, int dil, void* stream) {
    int oh, ow;
    if (B < 0 || !conv_geometry(C, H, W, kh, kw, stride, pad, dil, &oh, &ow)) return fail(AMR_EINVAL, "bad convolution geometry");
    if (B == 0) return AMR_OK;
    if ((size_t)B * C * H * W >= ((size_t)1 << 40)) return fail(AMR_EUNSUPPORTED, "more than 2^40 pixels");
    if ((size_t)C * H * W > 0x7fffffffull) return fail(AMR_EUNSUPPORTED, "more than 2^31 pixels in one image");
    if (!t || !z_w || !inside || !scale || !gx) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_conv_input_grad(cols, t, z_w, inside, scale, gx, B, C, H, W, kh, kw, stride, pad, dil, oh, ow,
                                               reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "input gradient launch");
}

int amr_lut_conv_input_grad_supported(int64_t lut_elems, int B, int C, int H, int W, int N) {
    amr::LutGeom g;
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || N <= 0 || !amr::lut_geom_from_elems(lut_elems, &g)) return 0;
    const int mode = g_expanded_kernels.load();
    return mode && amr::gradA_slab_conv_applies(g, (long)B * H * W, C, N, nullptr, mode == 2) ? 1 : 0;
}

// scratch of the convolution-shaped gradA: [256 B of flags][window sums of t, B*H*W floats][expanded table]
static size_t conv_grad_zt_bytes(int B, int H, int W) { return ((size_t)B * H * W * sizeof(float) + 255) & ~(size_t)255; }

size_t amr_lut_conv_input_grad_workspace_bytes(int64_t lut_elems, int B, int C, int H, int W, int N) {
    if (!amr_lut_conv_input_grad_supported(lut_elems, B, C, H, W, N)) return 0;
    return 256 + conv_grad_zt_bytes(B, H, W) + amr::gradA_slab_conv_workspace_bytes(C, N);
}

size_t amr_lut_conv_input_grad_cached_workspace_bytes(int64_t lut_elems, int B, int C, int H, int W, int N) {
    if (!amr_lut_conv_input_grad_supported(lut_elems, B, C, H, W, N)) return 0;
    return 256 + conv_grad_zt_bytes(B, H, W);
}

// The decision bwd_header_kernel takes on the device (lutgemm_bwd_slab.hip), for a table in host memory.
int amr_grad_table_fits_halves(const int16_t* host_table, int64_t lut_elems) {
    amr::LutGeom g;
    if (!host_table || !amr::lut_geom_from_elems(lut_elems, &g)) return fail(AMR_ELUTLEN, "bad table");
    int lo = 0, hi = 0;
    unsigned long long mag = 0;
    for (int64_t i = 0; i < (int64_t)g.rows * g.cols; ++i) {
        const int v = host_table[i];
        lo = v < lo ? v : lo;
        hi = v > hi ? v : hi;
        mag += (unsigned long long)(v < 0 ? -v : v);
    }
    if (lo >= -2048 && hi <= 2048) return 1;
    if (hi - lo > 4096) return 0;
    const int need = hi > 2048 ? hi - 2048 : -(lo + 2048), room = hi > 2048 ? lo + 2048 : -(hi - 2048);
    int p = 1;
    while (p < need) p <<= 1;
    const int off = p <= room ? p : need;
    const unsigned long long n_entries = (unsigned long long)(1 << g.bits) * (1 << g.bits);
    return (unsigned long long)off * n_entries > 8ull * mag ? 0 : 1;
}

int amr_lut_conv_input_grad_f32(const float* gC, const uint8_t* codes, const uint8_t* Bt, const int16_t* lut_grad_a, int64_t lut_elems,
                                const float* t, const float* z_w, const uint8_t* inside, const float* scale, float* gx, int B, int C,
                                int H, int W, int N, const uint8_t* A_fallback, float* cols_fallback, void* workspace,
                                size_t workspace_bytes, void* stream) {
    return amr_lut_conv_input_grad_cached_f32(nullptr, 0, gC, codes, Bt, lut_grad_a, lut_elems, t, z_w, inside, scale, gx, B, C, H, W, N,
                                              A_fallback, cols_fallback, workspace, workspace_bytes, stream);
}

int amr_lut_conv_input_grad_cached_f32(amr_fwd_cache* cache, uint64_t b_version, const float* gC, const uint8_t* codes, const uint8_t* Bt,
                                       const int16_t* lut_grad_a, int64_t lut_elems, const float* t, const float* z_w,
                                       const uint8_t* inside, const float* scale, float* gx, int B, int C, int H, int W, int N,
                                       const uint8_t* A_fallback, float* cols_fallback, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    amr::LutGeom g;
    if (!amr::lut_geom_from_elems(lut_elems, &g))
        return fail(AMR_ELUTLEN, "lut size should be one of 1024/5120/17408/66306, got %lld", (long long)lut_elems);
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || N <= 0) return fail(AMR_EINVAL, "bad shape");
    if (!gC || !codes || !Bt || !lut_grad_a || !t || !z_w || !inside || !scale || !gx) return fail(AMR_EINVAL, "null pointer argument");
    if ((uintptr_t)lut_grad_a & 3) return fail(AMR_EINVAL, "gradient tables must be 4-byte aligned");
    if ((A_fallback == nullptr) != (cols_fallback == nullptr)) return fail(AMR_EINVAL, "A_fallback and cols_fallback go together");
    const int mode = g_expanded_kernels.load();
    const long M = (long)B * H * W;
    if (!mode || !amr::gradA_slab_conv_applies(g, M, C, N, gC, mode == 2))
        return fail(AMR_EUNSUPPORTED, "shape, alignment or mode not served by the convolution-shaped gradA (ask amr_lut_conv_input_grad_supported)");
    const size_t zt_bytes = conv_grad_zt_bytes(B, H, W);
    const size_t s_bytes = amr::gradA_slab_conv_workspace_bytes(C, N);
    const size_t need = 256 + zt_bytes + (cache ? 0 : s_bytes);      // (with a cache the expanded table lives there)
    if (!workspace || workspace_bytes < need)
        return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace ? workspace_bytes : (size_t)0, need);
    if ((uintptr_t)workspace & 255) return fail(AMR_EINVAL, "workspace must be 256-byte aligned");
    int dev = 0;
    const int n_cu = current_device_cus(&dev);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const float factor = 1.0f / 16.0f;  // FACTOR, self_ops/src/approx_mult.h:41
    uint32_t* flags = reinterpret_cast<uint32_t*>(workspace);
    hipError_t e = amr::launch_bwd_header(lut_grad_a, nullptr, g, flags, s);      // clears the 64 flag words: words 32..63 stay zero
    if (e != hipSuccess) return hip_fail(e, "scratch header launch");
    // Where every wave stores whole 16-byte pieces the kernel finishes the gradient in its store (mask, zero-point term,
    // quantiser scale); the channel-independent window sums of t it needs for that are formed first.
    const bool finish = amr::gradA_slab_conv_can_finish(B, H, W, gx);
    float* zt = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(workspace) + 256);
    if (finish && (e = amr::launch_window_sums_3x3(t, zt, B, H, W, s)) != hipSuccess) return hip_fail(e, "window sums launch");
    void* s_buf = reinterpret_cast<unsigned char*>(workspace) + 256 + zt_bytes;
    bool hit = false;
    if (cache) {
        hipError_t ec;
        s_buf = fwd_cache_lookup(cache, dev, s_bytes, b_version, lut_grad_a, lut_elems, 9 * C, N, &hit, &ec);
        if (!s_buf) return hip_fail(ec, "cache hipMalloc");
    }
    e = amr::launch_gradA_slab_conv(gC, codes, Bt, gx, lut_grad_a, g, B, C, H, W, N, factor, n_cu, flags, s_buf,
                                    reinterpret_cast<const float*>(flags + 32), s, finish ? zt : nullptr, z_w, scale, inside, hit ? 1 : 0);
    if (e != hipSuccess) {
        if (cache) fwd_cache_forget(cache);      // (whether the expansion got there is unknown)
        return hip_fail(e, "gradA launch");
    }
    // flags[2]: a masked code, an entry a half cannot hold, or a table that cannot be held as halves at all
    const bool fallback = A_fallback != nullptr;
    if (!finish)
        e = amr::launch_conv_input_grad(nullptr, t, z_w, inside, scale, gx, B, C, H, W, 3, 3, 1, 1, 1, H, W, s, flags + 2, fallback ? 1 : 3);
    else if (!fallback)
        e = amr::launch_poison_if_raised(gx, (size_t)B * C * H * W, flags + 2, s);
    if (e != hipSuccess) return hip_fail(e, "input gradient launch");
    if (fallback) {
        e = amr::launch_gradA(gC, A_fallback, Bt, cols_fallback, lut_grad_a, g, (int)M, 9 * C, N, factor, n_cu, s, flags + 2, H * W);
        if (e != hipSuccess) return hip_fail(e, "gradA fall-back launch");
        e = amr::launch_conv_input_grad(cols_fallback, t, z_w, inside, scale, gx, B, C, H, W, 3, 3, 1, 1, 1, H, W, s, flags + 2, 2);
        if (e != hipSuccess) return hip_fail(e, "input gradient fall-back launch");
    }
    return AMR_OK;
}

int amr_conv_weight_prepare_f32(const float* w, const float* scale, const float* zp_neg, float qmax, const float* tapmask, uint8_t* Bt,
                                uint8_t* inside, float* w_resp, int N, int C, int taps, int positions, void* stream) {
    if (N <= 0 || C <= 0 || taps <= 0 || taps > 64 || positions <= 0 || !(qmax >= 0.f) || qmax > 255.f)
        return fail(AMR_EINVAL, "bad shape or code range (at most 64 taps)");
    if (!w || !scale || !zp_neg || !tapmask || !Bt || !inside || !w_resp) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_conv_weight_prepare(w, scale, zp_neg, qmax, tapmask, Bt, inside, w_resp, N, C, taps, positions,
                                                   reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "weight prepare launch");
}

size_t amr_conv_zero_point_grad_workspace_bytes(int batch, int N, int positions) {
    if (batch <= 0 || N <= 0 || positions <= 0) return 0;
    const int n_cu = current_device_cus(nullptr);
    const size_t inner = (size_t)N * positions;
    return (size_t)amr::batch_sum_segments(batch, inner, n_cu > 0 ? n_cu : 256) * inner * sizeof(float);
}

int amr_conv_zero_point_grad_parts(int positions) { return positions > 0 ? amr::batch_sum_parts(positions) : 0; }

int amr_conv_zero_point_grad_f32(const float* g, const float* z_a, const float* s_a, const float* s_w, const float* tapmask, float* g_wr,
                                 float* gz, int batch, int N, int positions, int taps, void* workspace, size_t workspace_bytes,
                                 void* stream) {
    if (batch <= 0 || N <= 0 || positions <= 0 || taps <= 0 || taps > 64) return fail(AMR_EINVAL, "bad shape (at most 64 taps)");
    if (!g || !z_a || !s_a || !s_w || !tapmask || !gz) return fail(AMR_EINVAL, "null pointer argument");
    const int n_cu = current_device_cus(nullptr);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    const size_t inner = (size_t)N * positions;
    const size_t need = (size_t)amr::batch_sum_segments(batch, inner, n_cu) * inner * sizeof(float);
    if (!workspace || workspace_bytes < need)
        return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace ? workspace_bytes : (size_t)0, need);
    if (((uintptr_t)workspace | (uintptr_t)g) & 15) return fail(AMR_EINVAL, "g and workspace must be 16-byte aligned");
    hipError_t e = amr::launch_batch_sum_taps(g, z_a, s_a, s_w, tapmask, g_wr, gz, reinterpret_cast<float*>(workspace), batch, N, positions,
                                              taps, n_cu, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "zero-point gradient launch");
}

int amr_conv_weight_grad_f32(const float* gBt, const float* gz, int gz_parts, const uint8_t* inside, const float* scale, float* gw, int N,
                             int C, int taps, void* stream) {
    if (N <= 0 || C <= 0 || taps <= 0 || taps > 64 || gz_parts <= 0) return fail(AMR_EINVAL, "bad shape (at most 64 taps)");
    if (!gBt || !gz || !inside || !scale || !gw) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_conv_weight_grad(gBt, gz, gz_parts, inside, scale, gw, N, C, taps, current_device_cus(nullptr),
                                                reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "weight gradient launch");
}

int amr_conv_dequant_backward_rowsum_f32(const float* g, const float* s_a, const float* s_w, float* g_c, float* t, int batch,
                                         int out_channels, int positions, void* stream) {
    if (batch < 0 || out_channels <= 0 || positions <= 0) return fail(AMR_EINVAL, "bad shape");
    if (batch == 0) return AMR_OK;
    if ((long)batch * positions >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 output positions");
    if (!g || !s_a || !s_w || !g_c || !t) return fail(AMR_EINVAL, "null pointer argument");
    hipError_t e = amr::launch_dequant_grad_rowsum(g, s_a, s_w, g_c, t, batch * positions, out_channels, positions,
                                                   reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "dequant backward launch");
}

size_t amr_conv_output_grad_workspace_bytes(int batch, int out_channels, int positions) {
    if (batch <= 0 || out_channels <= 0 || positions <= 0) return 0;
    const int n_cu = current_device_cus(nullptr);
    bool fused = false;
    const int segs = amr::output_grad_segments(batch, out_channels, positions, n_cu > 0 ? n_cu : 256, &fused);
    return (size_t)segs * out_channels * positions * sizeof(float);
}

int amr_conv_output_grad_f32(const float* g, const float* z_a, const float* s_a, const float* s_w, const float* tapmask, float* g_c, float* t,
                             float* gz, int batch, int out_channels, int positions, int taps, void* workspace, size_t workspace_bytes,
                             void* stream) {
    if (batch <= 0 || out_channels <= 0 || positions <= 0) return fail(AMR_EINVAL, "bad shape");
    if ((long)batch * positions >= (1L << 31)) return fail(AMR_EUNSUPPORTED, "more than 2^31 output positions");
    if (!g || !s_a || !s_w || !g_c || !t) return fail(AMR_EINVAL, "null pointer argument");
    if ((tapmask != nullptr) != (gz != nullptr)) return fail(AMR_EINVAL, "tapmask and gz go together");
    const int n_cu = current_device_cus(nullptr);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    if (tapmask) {
        if (taps <= 0 || taps > 64 || !z_a) return fail(AMR_EINVAL, "bad tap count (at most 64) or null z_a");
        const size_t need = amr_conv_output_grad_workspace_bytes(batch, out_channels, positions);
        if (!workspace || workspace_bytes < need)
            return fail(AMR_EWORKSPACE, "workspace of %zu bytes is smaller than the %zu required", workspace ? workspace_bytes : (size_t)0, need);
        if (((uintptr_t)workspace | (uintptr_t)g) & 15) return fail(AMR_EINVAL, "g and workspace must be 16-byte aligned");
    }
    hipError_t e = amr::launch_output_grad(g, z_a, s_a, s_w, tapmask, g_c, t, gz, reinterpret_cast<float*>(workspace), batch, out_channels,
                                           positions, taps, n_cu, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "output gradient launch");
}

int amr_acc_gemm_forward_fp32(const float* A, const float* B, float* C, int M, int K, int N, void* stream) {
    if (M < 0 || K < 0 || N < 0) return fail(AMR_EINVAL, "negative dimension M=%d K=%d N=%d", M, K, N);
    if (M == 0 || N == 0) return AMR_OK;
    if (!C || (K > 0 && (!A || !B))) return fail(AMR_EINVAL, "null pointer argument");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (K == 0) {
        hipError_t e = amr::launch_zero_u32(C, (size_t)M * N, s);
        return e == hipSuccess ? AMR_OK : hip_fail(e, "zero fill launch");
    }
    hipError_t e = amr::launch_accgemm(A, B, C, M, K, N, s);
    return e == hipSuccess ? AMR_OK : hip_fail(e, "accgemm launch");
}

int amr_lds_gather_probe(int pattern, int waves_per_cu, int iters, float* ms_out, double* gathers_out, void* stream) {
    if (pattern < 0 || pattern > 3 || iters <= 0) return fail(AMR_EINVAL, "bad probe arguments");
    const int n_cu = current_device_cus(nullptr);
    if (n_cu <= 0) return fail(AMR_EINVAL, "no HIP device available");
    if (pattern >= 2) {
        hipError_t e2 = amr::run_lds_direct_probe(pattern == 2 ? 288 : 32, iters, n_cu, ms_out, gathers_out, reinterpret_cast<hipStream_t>(stream));
        return e2 == hipSuccess ? AMR_OK : hip_fail(e2, "lds-direct probe");
    }
    hipError_t e = amr::run_lds_probe(pattern, waves_per_cu, iters, n_cu, ms_out, gathers_out, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AMR_OK : hip_fail(e, "lds probe");
}

}  // extern "C"
