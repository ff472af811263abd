"""``approx_ops`` -- the native operator module of the LUT-based approximate-multiplier GEMM, for MI355X.

Drop-in for the reference's compiled extension of the same name (module name:
``setup.py:37``; the three registered functions: ``self_ops/src/op_register.cpp:16-19``).  The
functions take the same tensors in the same order, require the same devices / dtypes / contiguity /
shapes as the reference's ``CHECK_INPUT`` and ``TORCH_CHECK`` lines and raise ``RuntimeError`` when they
are violated; outputs are caller-allocated and overwritten.  Behind them sits ``libamr_lutgemm.so``
(HIP kernels for gfx950) reached through its C ABI with ctypes -- torch is used for device memory
and streams only.

Differences from the reference, all on the safe side:
  * the bit-width is taken from the table length at run time (the reference bakes it in at compile
    time, ``self_ops/src/approx_mult.h:12``);
  * kernels run on torch's current stream of the tensors' device, under a device guard
    (reference: legacy default stream, bare ``cudaSetDevice``, ``approx_gemm_forward.cu:256,287``);
  * a failed launch raises instead of printing (``approx_gemm_forward.cu:304-306``).

There is no CPU implementation: importing this module without the built library raises ImportError.
"""
import ctypes
import os

import torch

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB_PATH = os.path.join(_PKG_DIR, "libamr_lutgemm.so")

if not os.path.exists(_LIB_PATH):
    raise ImportError(
        f"{_LIB_PATH} is missing: build the HIP library first (python {os.path.join(_PKG_DIR, 'build.py')}); "
        "approx_ops has no CPU fallback")
_lib = ctypes.CDLL(_LIB_PATH)

_vp, _i, _i64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
_lib.amr_last_error.restype = ctypes.c_char_p
_lib.amr_target_arch.restype = ctypes.c_char_p
_lib.amr_lut_gemm_forward.argtypes = [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]
_lib.amr_lut_gemm_forward_ws.argtypes = [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_lut_gemm_forward_f32_ws.argtypes = [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_lut_gemm_forward_workspace_bytes.argtypes = [_i64, _i, _i, _i]
_lib.amr_lut_gemm_forward_workspace_bytes.restype = _sz
_lib.amr_lut_gemm_backward.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_lut_gemm_backward_ex.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_lut_gemm_backward_f32tab_workspace_bytes.argtypes = [_i, _i, _i]
_lib.amr_lut_gemm_backward_f32tab_workspace_bytes.restype = _sz
_lib.amr_lut_gemm_backward_f32tab.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, ctypes.c_float, _i, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_im2col_u8_f32.argtypes = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]
_lib.amr_col2im_f32.argtypes = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]
_lib.amr_conv_dequant_f32.argtypes = [_vp] * 10 + [_i, _i, _i, _vp]
_lib.amr_conv_dequant_backward_f32.argtypes = [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]
_lib.amr_observer_update_f32.argtypes = [_vp] * 6 + [_i] + [ctypes.c_float] * 5 + [_vp]
_lib.amr_observe_minmax_f32.argtypes = [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _i] + [ctypes.c_float] * 5 + [_vp]
_lib.amr_quantize_codes_f32.argtypes = [_vp, _vp, _vp, ctypes.c_float, _vp, _i64, _vp]
_lib.amr_quantize_codes_backward_f32.argtypes = [_vp, _vp, _vp, _vp, ctypes.c_float, _vp, _i64, _vp]
_lib.amr_lut_conv_forward_dequant_workspace_bytes.argtypes = [_i64, _i, _i, _i]
_lib.amr_lut_conv_forward_dequant_workspace_bytes.restype = _sz
_lib.amr_lut_conv_forward_dequant_f32.argtypes = [_vp, _vp, _vp, _i64, _i, _i, _i, _i] + [_vp] * 9 + [_vp, _sz, _vp]
_lib.amr_lut_conv_input_grad_supported.argtypes = [_i64, _i, _i, _i, _i, _i]
_lib.amr_lut_conv_input_grad_workspace_bytes.argtypes = [_i64, _i, _i, _i, _i, _i]
_lib.amr_lut_conv_input_grad_workspace_bytes.restype = _sz
_lib.amr_grad_table_fits_halves.argtypes = [_vp, _i64]
_lib.amr_lut_conv_input_grad_f32.argtypes = [_vp] * 4 + [_i64] + [_vp] * 5 + [_i] * 5 + [_vp, _vp, _vp, _sz, _vp]
_lib.amr_lut_conv_input_grad_cached_workspace_bytes.argtypes = [_i64, _i, _i, _i, _i, _i]
_lib.amr_lut_conv_input_grad_cached_workspace_bytes.restype = _sz
_lib.amr_lut_conv_input_grad_cached_f32.argtypes = [_vp, ctypes.c_uint64] + [_vp] * 4 + [_i64] + [_vp] * 5 + [_i] * 5 + [_vp, _vp, _vp, _sz, _vp]
_u64 = ctypes.c_uint64
_lib.amr_fwd_cache_create.argtypes = [ctypes.POINTER(_vp)]
_lib.amr_fwd_cache_destroy.argtypes = [_vp]
_lib.amr_fwd_cache_stats.argtypes = [_vp, ctypes.POINTER(_u64), ctypes.POINTER(_u64), ctypes.POINTER(_sz)]
_lib.amr_lut_gemm_forward_cached.argtypes = [_vp, _u64, _vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _vp]
_lib.amr_lut_conv_forward_dequant_cached_f32.argtypes = [_vp, _u64, _vp, _vp, _vp, _i64, _i, _i, _i, _i] + [_vp] * 9 + [_vp, _sz, _vp]
_lib.amr_lut_conv_forward_implicit_supported.argtypes = [_i64, _i, _i, _i, _i, _i]
_lib.amr_lut_conv_forward_implicit_workspace_bytes.argtypes = [_i64, _i, _i, _i, _i, _i, _i, _i]
_lib.amr_lut_conv_forward_implicit_workspace_bytes.restype = _sz
_lib.amr_lut_conv_forward_implicit_f32.argtypes = [_vp, ctypes.c_uint64, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i] + [_vp] * 10 + [_vp, _sz, _vp]
_lib.amr_conv_weight_prepare_f32.argtypes = [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]
_lib.amr_conv_zero_point_grad_workspace_bytes.argtypes = [_i, _i, _i]
_lib.amr_conv_zero_point_grad_workspace_bytes.restype = _sz
_lib.amr_conv_zero_point_grad_f32.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_conv_zero_point_grad_parts.argtypes = [_i]
_lib.amr_conv_output_grad_workspace_bytes.argtypes = [_i, _i, _i]
_lib.amr_conv_output_grad_workspace_bytes.restype = _sz
_lib.amr_conv_output_grad_f32.argtypes = [_vp] * 8 + [_i, _i, _i, _i, _vp, _sz, _vp]
_lib.amr_conv_weight_grad_f32.argtypes = [_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _vp]
_lib.amr_quantize_codes_nhwc_relu_u8.argtypes = [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _i, _i, _i, _i, _vp]
_lib.amr_quantize_codes_nhwc_u8.argtypes = [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _i, _i, _i, _vp]
_lib.amr_im2col_nhwc_u8.argtypes = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]
_lib.amr_conv_input_grad_f32.argtypes = [_vp] * 6 + [_i] * 9 + [_vp]
_lib.amr_conv_dequant_backward_rowsum_f32.argtypes = [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]
_lib.amr_lut_gemm_backward_workspace_bytes.argtypes = [_i, _i, _i]
_lib.amr_lut_gemm_backward_workspace_bytes.restype = _sz
_lib.amr_lut_gemm_backward_workspace_bytes_for.argtypes = [_i64, _i, _i, _i]
_lib.amr_lut_gemm_backward_workspace_bytes_for.restype = _sz
_lib.amr_lut_gemm_backward_f32tab_workspace_bytes_for.argtypes = [_i64, _i, _i, _i]
_lib.amr_lut_gemm_backward_f32tab_workspace_bytes_for.restype = _sz
_lib.amr_lut_gemm_backward_static.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp]
_lib.amr_static_scratch_bytes.restype = _sz
_lib.amr_acc_gemm_forward_fp32.argtypes = [_vp, _vp, _vp, _i, _i, _i, _vp]
_lib.amr_bits_from_lut_elems.argtypes = [_i64]
_lib.amr_lut_geometry.argtypes = [_i, ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_i64)]
_lib.amr_lds_gather_probe.argtypes = [_i, _i, _i, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double), _vp]

LIBRARY_PATH = _LIB_PATH


def _check_input(x, dtype, name):
    # same three conditions, same order and wording as CHECK_INPUT (self_ops/src/cuda_helper.h:64-68)
    if not (isinstance(x, torch.Tensor) and x.device.type == "cuda"):
        raise RuntimeError(f"{name} must be a CUDAtensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if x.dtype != dtype:
        raise RuntimeError(f"{name} must be of type {dtype}")


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _raise_for(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed ({rc}): {_lib.amr_last_error().decode()}")


def _lut_len_check(lut, name):
    _check(lut.dim() == 1 and _lib.amr_bits_from_lut_elems(lut.size(0)) > 0,
           f"{name} size should be 1024, 5120, 17408 or 66306 (4-, 6-, 7-, 8-bit padded table), got {tuple(lut.shape)}; "
           "please check the value of QUANTIZATION_BIT")


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class ForwardCache:
    """The expansion of the forward table along one weight matrix, kept on the device between forward calls whose B does not
    change (amr_fwd_cache): pass it, with a number that changes whenever B's contents do, to approx_gemm_forward or
    approx_conv_forward_dequant.  Calls sharing a cache must be stream-ordered."""

    def __init__(self):
        self._h = _vp()
        _raise_for(_lib.amr_fwd_cache_create(ctypes.byref(self._h)), "amr_fwd_cache_create")

    def stats(self):
        """(hits, misses, bytes of device memory held)."""
        h, m, b = _u64(0), _u64(0), _sz(0)
        _raise_for(_lib.amr_fwd_cache_stats(self._h, ctypes.byref(h), ctypes.byref(m), ctypes.byref(b)), "amr_fwd_cache_stats")
        return h.value, m.value, b.value

    def close(self):
        if self._h:
            _lib.amr_fwd_cache_destroy(self._h)
            self._h = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __deepcopy__(self, memo):
        return ForwardCache()         # a copied layer expands for itself


def approx_gemm_forward(a_tensor, b_tensor, c_tensor, lut_appmult_tensor, cache=None, b_version=0):
    """c[m,n] = sum_k lut[a[m,k]][b[k,n]]; a u8 [M,K], b u8 [K,N], c u32 [M,N] (out), lut u16 padded table.
    Contract of approx_gemm_forward_gpu (self_ops/src/approx_gemm_forward.cu:241-259).
    A float32 c_tensor receives the same sums converted to float32 (what the reference's callers do with the uint32
    result at once, self_ops/ops_py/approx_ops.py:569) without the extra pass over it."""
    _check_input(a_tensor, torch.uint8, "a_tensor")
    _check_input(b_tensor, torch.uint8, "b_tensor")
    as_float = c_tensor.dtype == torch.float32
    _check_input(c_tensor, torch.float32 if as_float else torch.uint32, "c_tensor")
    _check_input(lut_appmult_tensor, torch.uint16, "lut_appmult_tensor")
    _check(a_tensor.dim() == 2 and b_tensor.dim() == 2 and c_tensor.dim() == 2, "a, b and c must be 2-D")
    M, K = a_tensor.shape
    N = b_tensor.size(1)
    _check(K == b_tensor.size(0), f"b_tensor's shape should be {K} x {N}")
    _check(M == c_tensor.size(0) and N == c_tensor.size(1), f"c_tensor's shape should be {M} x {N}")
    _lut_len_check(lut_appmult_tensor, "lut_appmult_tensor")
    dev = a_tensor.device
    _check(dev == b_tensor.device and dev == c_tensor.device and dev == lut_appmult_tensor.device, "device id not match")
    with torch.cuda.device(dev):
        # scratch (the expanded table of large problems) comes from torch's caching allocator, so that it is
        # ordered with the stream like any other tensor and freed with the process' other device memory
        if cache is not None:
            # (an extension: the expansion of the table along b is kept in `cache` while b_version stays the same)
            rc = _lib.amr_lut_gemm_forward_cached(cache._h, int(b_version) & 0xFFFFFFFFFFFFFFFF, a_tensor.data_ptr(), b_tensor.data_ptr(),
                                                  c_tensor.data_ptr(), 1 if as_float else 0, lut_appmult_tensor.data_ptr(),
                                                  lut_appmult_tensor.size(0), M, K, N, _stream_ptr(dev))
            _raise_for(rc, "approx_gemm_forward")
            return
        need = _lib.amr_lut_gemm_forward_workspace_bytes(lut_appmult_tensor.size(0), M, K, N)
        ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
        entry = _lib.amr_lut_gemm_forward_f32_ws if as_float else _lib.amr_lut_gemm_forward_ws
        rc = entry(a_tensor.data_ptr(), b_tensor.data_ptr(), c_tensor.data_ptr(), lut_appmult_tensor.data_ptr(),
                   lut_appmult_tensor.size(0), M, K, N, ws.data_ptr() if ws is not None else None, need, _stream_ptr(dev))
    _raise_for(rc, "approx_gemm_forward")


def acc_gemm_forward_fp32(a_tensor, b_tensor, c_tensor):
    """c = a @ b in fp32; contract of acc_gemm_forward_fp32_gpu (self_ops/src/approx_gemm_forward.cu:500-520)."""
    _check_input(a_tensor, torch.float32, "a_tensor")
    _check_input(b_tensor, torch.float32, "b_tensor")
    _check_input(c_tensor, torch.float32, "c_tensor")
    _check(a_tensor.dim() == 2 and b_tensor.dim() == 2 and c_tensor.dim() == 2, "a, b and c must be 2-D")
    M, K = a_tensor.shape
    N = b_tensor.size(1)
    _check(K == b_tensor.size(0), f"b_tensor's shape should be {K} x {N}")
    _check(M == c_tensor.size(0) and N == c_tensor.size(1), f"c_tensor's shape should be {M} x {N}")
    dev = a_tensor.device
    _check(dev == b_tensor.device and dev == c_tensor.device, "device id not match")
    with torch.cuda.device(dev):
        rc = _lib.amr_acc_gemm_forward_fp32(a_tensor.data_ptr(), b_tensor.data_ptr(), c_tensor.data_ptr(), M, K, N, _stream_ptr(dev))
    _raise_for(rc, "acc_gemm_forward_fp32")


def approx_gemm_backward(gc_tensor, a_tensor, b_tensor, ga_tensor, gb_tensor, lut_grad_a_tensor, lut_grad_b_tensor,
                         ga_rows_per_image=0, grad_scale=None):
    """ga[m,k] = 1/16 sum_n gc[m,n]*lutA[a][b], gb[k,n] = 1/16 sum_m lutB[a][b]*gc[m,n]; outputs overwritten.
    Contract of approx_gemm_backward_gpu (self_ops/src/approx_gemm_backward.cu:506-529).

    The tables are int16 (slope x 16, as the reference's) or, as an extension, both float32: then the entries are the
    slopes themselves and the factor in front of the sums is grad_scale (default 1).  grad_scale is not accepted
    with int16 tables (their factor is the reference's 1/16).

    ga_rows_per_image = L > 0 (an extension; the reference has no such argument) makes ga_tensor the image-major
    transposed gradient of shape [M/L, K, L], the layout torch's fold takes."""
    _check_input(gc_tensor, torch.float32, "gc_tensor")
    _check_input(a_tensor, torch.uint8, "a_tensor")
    _check_input(b_tensor, torch.uint8, "b_tensor")
    # ga_tensor / gb_tensor may be None (an extension): that gradient is then not computed
    _check(ga_tensor is not None or gb_tensor is not None, "ga_tensor and gb_tensor must not both be None")
    if ga_tensor is not None:
        _check_input(ga_tensor, torch.float32, "ga_tensor")
    if gb_tensor is not None:
        _check_input(gb_tensor, torch.float32, "gb_tensor")
    float_tables = lut_grad_a_tensor.dtype == torch.float32 and lut_grad_b_tensor.dtype == torch.float32
    _check_input(lut_grad_a_tensor, torch.float32 if float_tables else torch.int16, "lut_grad_a_tensor")
    _check_input(lut_grad_b_tensor, torch.float32 if float_tables else torch.int16, "lut_grad_b_tensor")
    _check(float_tables or grad_scale is None, "grad_scale needs float32 gradient tables")
    L = int(ga_rows_per_image)
    _check(all(t.dim() == 2 for t in (gc_tensor, a_tensor, b_tensor)) and (gb_tensor is None or gb_tensor.dim() == 2), "gc, a, b and gb must be 2-D")
    M, K = a_tensor.shape
    N = b_tensor.size(1)
    _check(gc_tensor.size(0) == M and gc_tensor.size(1) == N, f"gc_tensor's shape should be {M} x {N}")
    _check(K == b_tensor.size(0), f"b_tensor's shape should be {K} x {N}")
    _check(L >= 0, "ga_rows_per_image must not be negative")
    if L > 0:
        _check(M % L == 0, f"ga_rows_per_image={L} must divide {M}")
    if ga_tensor is not None and L > 0:
        _check(tuple(ga_tensor.shape) == (M // L, K, L), f"ga_tensor's shape should be {M // L} x {K} x {L}")
    elif ga_tensor is not None:
        _check(ga_tensor.dim() == 2 and ga_tensor.size(0) == M and ga_tensor.size(1) == K, f"ga_tensor's shape should be {M} x {K}")
    _check(gb_tensor is None or (gb_tensor.size(0) == K and gb_tensor.size(1) == N), f"gb_tensor's shape should be {K} x {N}")
    _lut_len_check(lut_grad_a_tensor, "lut_grad_a_tensor")
    _lut_len_check(lut_grad_b_tensor, "lut_grad_b_tensor")
    _check(lut_grad_a_tensor.size(0) == lut_grad_b_tensor.size(0), "the two gradient tables must have the same length")
    dev = gc_tensor.device
    _check(all(t.device == dev for t in (a_tensor, b_tensor, ga_tensor, gb_tensor, lut_grad_a_tensor, lut_grad_b_tensor) if t is not None),
           "All tensors should be on the same device")
    with torch.cuda.device(dev):
        need = (_lib.amr_lut_gemm_backward_f32tab_workspace_bytes_for if float_tables else
                _lib.amr_lut_gemm_backward_workspace_bytes_for)(lut_grad_a_tensor.size(0), M, K, N)
        ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
        ga_ptr = ga_tensor.data_ptr() if ga_tensor is not None else None
        gb_ptr = gb_tensor.data_ptr() if gb_tensor is not None else None
        ws_ptr = ws.data_ptr() if ws is not None else None
        if float_tables:
            rc = _lib.amr_lut_gemm_backward_f32tab(gc_tensor.data_ptr(), a_tensor.data_ptr(), b_tensor.data_ptr(), ga_ptr, gb_ptr,
                                                   lut_grad_a_tensor.data_ptr(), lut_grad_b_tensor.data_ptr(),
                                                   lut_grad_a_tensor.size(0), 1.0 if grad_scale is None else float(grad_scale),
                                                   M, K, N, L, ws_ptr, need, _stream_ptr(dev))
        else:
            rc = _lib.amr_lut_gemm_backward_ex(gc_tensor.data_ptr(), a_tensor.data_ptr(), b_tensor.data_ptr(), ga_ptr, gb_ptr,
                                               lut_grad_a_tensor.data_ptr(), lut_grad_b_tensor.data_ptr(),
                                               lut_grad_a_tensor.size(0), M, K, N, L, ws_ptr, need, _stream_ptr(dev))
    _raise_for(rc, "approx_gemm_backward")


def im2col_codes(x_tensor, a_tensor, kernel_size, stride, padding, dilation):
    """a[(b,oy,ox), c*kh*kw+i*kw+j] = uint8(x[b,c,oy*s-p+i*d,ox*s-p+j*d]) (0 outside the image): the operand matrix that
    the reference builds by pad + unfold + transpose + reshape + cast (self_ops/ops_py/approx_ops.py:556-563, :161-164).
    x is a contiguous float32 [B,C,H,W] tensor of integer codes; a is uint8 [B*oh*ow, C*kh*kw]."""
    _check_input(x_tensor, torch.float32, "x_tensor")
    _check_input(a_tensor, torch.uint8, "a_tensor")
    _check(x_tensor.dim() == 4 and a_tensor.dim() == 2, "x must be 4-D and a 2-D")
    kh, kw = kernel_size
    Bn, C, H, W = x_tensor.shape
    oh = (H + 2 * padding - dilation * (kh - 1) - 1) // stride + 1
    ow = (W + 2 * padding - dilation * (kw - 1) - 1) // stride + 1
    _check(oh > 0 and ow > 0, "empty convolution output")
    _check(tuple(a_tensor.shape) == (Bn * oh * ow, C * kh * kw), f"a_tensor's shape should be {Bn * oh * ow} x {C * kh * kw}")
    dev = x_tensor.device
    _check(dev == a_tensor.device, "device id not match")
    with torch.cuda.device(dev):
        rc = _lib.amr_im2col_u8_f32(x_tensor.data_ptr(), a_tensor.data_ptr(), Bn, C, H, W, kh, kw, stride, padding, dilation,
                                    _stream_ptr(dev))
    _raise_for(rc, "im2col_codes")


def col2im(cols_tensor, x_tensor, kernel_size, stride, padding, dilation):
    """x[b,c,y,x] = sum of the window entries cols[b, c*kh*kw + i*kw + j, oy*ow + ox] that pixel fed (the adjoint of
    im2col_codes; torch.nn.functional.fold of the same arguments).  cols float32 [B, C*kh*kw, oh*ow], x float32 [B,C,H,W]."""
    _check_input(cols_tensor, torch.float32, "cols_tensor")
    _check_input(x_tensor, torch.float32, "x_tensor")
    _check(cols_tensor.dim() == 3 and x_tensor.dim() == 4, "cols must be 3-D and x 4-D")
    kh, kw = kernel_size
    Bn, C, H, W = x_tensor.shape
    oh = (H + 2 * padding - dilation * (kh - 1) - 1) // stride + 1
    ow = (W + 2 * padding - dilation * (kw - 1) - 1) // stride + 1
    _check(oh > 0 and ow > 0, "empty convolution output")
    _check(tuple(cols_tensor.shape) == (Bn, C * kh * kw, oh * ow), f"cols_tensor's shape should be {Bn} x {C * kh * kw} x {oh * ow}")
    dev = x_tensor.device
    _check(dev == cols_tensor.device, "device id not match")
    with torch.cuda.device(dev):
        rc = _lib.amr_col2im_f32(cols_tensor.data_ptr(), x_tensor.data_ptr(), Bn, C, H, W, kh, kw, stride, padding, dilation,
                                 _stream_ptr(dev))
    _raise_for(rc, "col2im")


def conv_dequant(c_rows, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out_tensor):
    """out[b,n,pos] = (s_a*s_w) * (c_rows[b*L+pos, n] + ((z_w*x_sum[b,pos] + z_a*w_resp[n,pos]) + (z_a*z_w)*taps[pos])) + bias[n]:
    the zero-point terms and scaling of the reference's ApproxConv2d.forward (micronet+/app_layers.py:175-183) in one pass.
    c_rows float32 [B*L, N]; x_sum B*L elements; w_resp N*L; taps L; scalars one element each; out float32 [B, N, oh, ow]."""
    tensors = [(c_rows, "c_rows"), (x_sum, "x_sum"), (w_resp, "w_resp"), (taps, "taps"), (z_a, "z_a"), (z_w, "z_w"), (s_a, "s_a"),
               (s_w, "s_w"), (out_tensor, "out_tensor")] + ([(bias, "bias")] if bias is not None else [])
    for t, name in tensors:
        _check_input(t, torch.float32, name)
    _check(out_tensor.dim() == 4 and c_rows.dim() == 2, "out must be 4-D and c_rows 2-D")
    Bn, N = out_tensor.size(0), out_tensor.size(1)
    L = out_tensor.size(2) * out_tensor.size(3)
    _check(tuple(c_rows.shape) == (Bn * L, N), f"c_rows's shape should be {Bn * L} x {N}")
    _check(x_sum.numel() == Bn * L and w_resp.numel() == N * L and taps.numel() == L, "x_sum, w_resp or taps has the wrong size")
    _check(all(t.numel() == 1 for t in (z_a, z_w, s_a, s_w)), "z_a, z_w, s_a and s_w must hold one element")
    _check(bias is None or bias.numel() == N, f"bias should have {N} elements")
    dev = out_tensor.device
    _check(all(t.device == dev for t, _ in tensors), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_conv_dequant_f32(c_rows.data_ptr(), x_sum.data_ptr(), w_resp.data_ptr(), taps.data_ptr(), z_a.data_ptr(),
                                       z_w.data_ptr(), s_a.data_ptr(), s_w.data_ptr(), bias.data_ptr() if bias is not None else None,
                                       out_tensor.data_ptr(), Bn, N, L, _stream_ptr(dev))
    _raise_for(rc, "conv_dequant")


def approx_conv_forward_dequant(a_tensor, b_tensor, lut_appmult_tensor, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out_tensor,
                                cache=None, b_version=0):
    """approx_gemm_forward followed by conv_dequant without the sums going to memory: out float32 [B, N, oh, ow] from the uint8
    operand matrices a [B*L, K], b [K, N] (any common order of k) and the operands of conv_dequant."""
    _check_input(a_tensor, torch.uint8, "a_tensor")
    _check_input(b_tensor, torch.uint8, "b_tensor")
    _check_input(lut_appmult_tensor, torch.uint16, "lut_appmult_tensor")
    tensors = [(x_sum, "x_sum"), (w_resp, "w_resp"), (taps, "taps"), (z_a, "z_a"), (z_w, "z_w"), (s_a, "s_a"), (s_w, "s_w"),
               (out_tensor, "out_tensor")] + ([(bias, "bias")] if bias is not None else [])
    for t, name in tensors:
        _check_input(t, torch.float32, name)
    _check(a_tensor.dim() == 2 and b_tensor.dim() == 2 and out_tensor.dim() == 4, "a and b must be 2-D, out 4-D")
    M, K = a_tensor.shape
    N = b_tensor.size(1)
    Bn, L = out_tensor.size(0), out_tensor.size(2) * out_tensor.size(3)
    _check(K == b_tensor.size(0), f"b_tensor's shape should be {K} x {N}")
    _check(out_tensor.size(1) == N and Bn * L == M, f"out_tensor should hold {M} positions of {N} channels")
    _check(x_sum.numel() == M and w_resp.numel() == N * L and taps.numel() == L, "x_sum, w_resp or taps has the wrong size")
    _check(all(t.numel() == 1 for t in (z_a, z_w, s_a, s_w)), "z_a, z_w, s_a and s_w must hold one element")
    _check(bias is None or bias.numel() == N, f"bias should have {N} elements")
    _lut_len_check(lut_appmult_tensor, "lut_appmult_tensor")
    dev = a_tensor.device
    _check(all(t.device == dev for t, _ in tensors) and b_tensor.device == dev and lut_appmult_tensor.device == dev, "device id not match")
    with torch.cuda.device(dev):
        need = _lib.amr_lut_conv_forward_dequant_workspace_bytes(lut_appmult_tensor.size(0), M, K, N)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
        rc = _lib.amr_lut_conv_forward_dequant_cached_f32(cache._h if cache is not None else None, int(b_version) & 0xFFFFFFFFFFFFFFFF,
                                                   a_tensor.data_ptr(), b_tensor.data_ptr(), lut_appmult_tensor.data_ptr(),
                                                   lut_appmult_tensor.size(0), M, K, N, L, x_sum.data_ptr(), w_resp.data_ptr(),
                                                   taps.data_ptr(), z_a.data_ptr(), z_w.data_ptr(), s_a.data_ptr(), s_w.data_ptr(),
                                                   bias.data_ptr() if bias is not None else None, out_tensor.data_ptr(), ws.data_ptr(),
                                                   ws.numel(), _stream_ptr(dev))
    _raise_for(rc, "approx_conv_forward_dequant")


def conv_forward_implicit_supported(lut_appmult_tensor, x_shape, out_channels):
    """Whether approx_conv_forward_implicit serves a 3x3 / stride 1 / padding 1 convolution of an input of shape
    x_shape = (B, C, H, W) with this table (asks the library)."""
    Bn, C, H, W = (int(v) for v in x_shape)
    dev = lut_appmult_tensor.device
    if not lut_appmult_tensor.is_cuda:
        return False
    with torch.cuda.device(dev):
        return bool(_lib.amr_lut_conv_forward_implicit_supported(lut_appmult_tensor.numel(), Bn, C, H, W, int(out_channels)))


def approx_conv_forward_implicit(codes, bt_tensor, lut_appmult_tensor, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out_tensor, x_shape,
                                 a_fallback=None, cache=None, b_version=0):
    """approx_conv_forward_dequant of a 3x3 / stride 1 / padding 1 convolution without its window matrix: codes uint8
    [B*H*W, C] pixel-major (quantize_codes_nhwc), bt uint8 [9*C, N] tap-major weight codes, out float32 [B, N, H, W].
    a_fallback (optional): the window matrix [B*H*W, 9*C]; without it a masked code or a table the packed sums cannot hold
    leaves NaN in out."""
    _check_input(codes, torch.uint8, "codes")
    _check_input(bt_tensor, torch.uint8, "bt_tensor")
    _check_input(lut_appmult_tensor, torch.uint16, "lut_appmult_tensor")
    tensors = [(x_sum, "x_sum"), (w_resp, "w_resp"), (taps, "taps"), (z_a, "z_a"), (z_w, "z_w"), (s_a, "s_a"), (s_w, "s_w"),
               (out_tensor, "out_tensor")] + ([(bias, "bias")] if bias is not None else [])
    for t, name in tensors:
        _check_input(t, torch.float32, name)
    Bn, C, H, W = (int(v) for v in x_shape)
    M, L = Bn * H * W, H * W
    _check(codes.dim() == 2 and tuple(codes.shape) == (M, C), f"codes' shape should be {M} x {C}")
    _check(bt_tensor.dim() == 2 and bt_tensor.size(0) == 9 * C, f"bt_tensor should have {9 * C} rows")
    N = bt_tensor.size(1)
    _check(tuple(out_tensor.shape) == (Bn, N, H, W), f"out_tensor's shape should be {(Bn, N, H, W)}")
    _check(x_sum.numel() == M and w_resp.numel() == N * L and taps.numel() == L, "x_sum, w_resp or taps has the wrong size")
    _check(all(t.numel() == 1 for t in (z_a, z_w, s_a, s_w)), "z_a, z_w, s_a and s_w must hold one element")
    _check(bias is None or bias.numel() == N, f"bias should have {N} elements")
    if a_fallback is not None:
        _check_input(a_fallback, torch.uint8, "a_fallback")
        _check(tuple(a_fallback.shape) == (M, 9 * C), f"a_fallback's shape should be {M} x {9 * C}")
    _lut_len_check(lut_appmult_tensor, "lut_appmult_tensor")
    dev = codes.device
    _check(all(t.device == dev for t, _ in tensors) and bt_tensor.device == dev and lut_appmult_tensor.device == dev
           and (a_fallback is None or a_fallback.device == dev), "device id not match")
    with torch.cuda.device(dev):
        need = _lib.amr_lut_conv_forward_implicit_workspace_bytes(lut_appmult_tensor.size(0), Bn, C, H, W, N, 1 if cache is not None else 0,
                                                                  1 if a_fallback is not None else 0)
        ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
        rc = _lib.amr_lut_conv_forward_implicit_f32(cache._h if cache is not None else None, int(b_version) & 0xFFFFFFFFFFFFFFFF,
                                                    codes.data_ptr(), bt_tensor.data_ptr(), lut_appmult_tensor.data_ptr(),
                                                    lut_appmult_tensor.size(0), Bn, C, H, W, N, x_sum.data_ptr(), w_resp.data_ptr(),
                                                    taps.data_ptr(), z_a.data_ptr(), z_w.data_ptr(), s_a.data_ptr(), s_w.data_ptr(),
                                                    bias.data_ptr() if bias is not None else None, out_tensor.data_ptr(),
                                                    a_fallback.data_ptr() if a_fallback is not None else None,
                                                    ws.data_ptr() if ws is not None else None, need, _stream_ptr(dev))
    _raise_for(rc, "approx_conv_forward_implicit")


def conv_dequant_backward(g_tensor, s_a, s_w, gc_rows):
    """gc_rows[b*L+pos, n] = (s_a*s_w) * g[b,n,pos]; g float32 [B,N,oh,ow] contiguous, gc_rows float32 [B*L, N]."""
    for t, name in ((g_tensor, "g_tensor"), (s_a, "s_a"), (s_w, "s_w"), (gc_rows, "gc_rows")):
        _check_input(t, torch.float32, name)
    _check(g_tensor.dim() == 4 and gc_rows.dim() == 2, "g must be 4-D and gc_rows 2-D")
    Bn, N = g_tensor.size(0), g_tensor.size(1)
    L = g_tensor.size(2) * g_tensor.size(3)
    _check(tuple(gc_rows.shape) == (Bn * L, N), f"gc_rows's shape should be {Bn * L} x {N}")
    dev = g_tensor.device
    with torch.cuda.device(dev):
        rc = _lib.amr_conv_dequant_backward_f32(g_tensor.data_ptr(), s_a.data_ptr(), s_w.data_ptr(), gc_rows.data_ptr(), Bn, N, L,
                                                _stream_ptr(dev))
    _raise_for(rc, "conv_dequant_backward")


def observer_update(cur_min, cur_max, min_val, max_val, scale, zp_neg, mode, momentum, quant_max, eps, inv_quant_max=0.0):
    """One launch for the range update of an observer (mode 0 first batch, 1 running extremes, 2 moving average) and the
    scale / zero point that follow from it; all tensors one float32 element on the device, the last four updated in place.
    inv_quant_max != 0: the range is multiplied by it instead of divided by quant_max."""
    for t, name in ((cur_min, "cur_min"), (cur_max, "cur_max"), (min_val, "min_val"), (max_val, "max_val"), (scale, "scale"),
                    (zp_neg, "zp_neg")):
        _check_input(t, torch.float32, name)
        _check(t.numel() == 1, f"{name} must hold one element")
    dev = cur_min.device
    with torch.cuda.device(dev):
        rc = _lib.amr_observer_update_f32(cur_min.data_ptr(), cur_max.data_ptr(), min_val.data_ptr(), max_val.data_ptr(),
                                          scale.data_ptr(), zp_neg.data_ptr(), int(mode), float(1 - momentum), float(momentum),
                                          float(quant_max), float(inv_quant_max), float(eps), _stream_ptr(dev))
    _raise_for(rc, "observer_update")


MINMAX_STATE_WORDS = 4 + 3 * 1024     # AMR_OBSERVE_STATE_WORDS: int32 words of an observer's state, all zero before the first call


def observe_minmax(x_tensor, state_tensor, min_val, max_val, scale, zp_neg, mode, momentum, quant_max, eps, inv_quant_max=0.0,
                   relu=False):
    """observer_update on the extremes of x_tensor, which the same launch finds (x float32, contiguous; state int32
    [MINMAX_STATE_WORDS] on the device, zeros before the first call).  relu: the extremes of max(x, 0)."""
    _check_input(x_tensor, torch.float32, "x_tensor")
    _check_input(state_tensor, torch.int32, "state_tensor")
    _check(state_tensor.numel() >= MINMAX_STATE_WORDS and x_tensor.numel() > 0, "state too small, or x empty")
    for t, name in ((min_val, "min_val"), (max_val, "max_val"), (scale, "scale"), (zp_neg, "zp_neg")):
        _check_input(t, torch.float32, name)
        _check(t.numel() == 1, f"{name} must hold one element")
    dev = x_tensor.device
    _check(all(t.device == dev for t in (state_tensor, min_val, max_val, scale, zp_neg)), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_observe_minmax_f32(x_tensor.data_ptr(), x_tensor.numel(), state_tensor.data_ptr(), min_val.data_ptr(),
                                         max_val.data_ptr(), scale.data_ptr(), zp_neg.data_ptr(), int(mode) | (4 if relu else 0), float(1 - momentum),
                                         float(momentum), float(quant_max), float(inv_quant_max), float(eps), _stream_ptr(dev))
    _raise_for(rc, "observe_minmax")


def quantize_codes(x_tensor, scale_tensor, zp_neg_tensor, quant_max, codes_tensor):
    """codes = clamp(round(x / scale - zp_neg), 0, quant_max) in one pass (the forward value of the reference's
    quantize_v2, micronet+/app_layers.py:147-160); scale and zp_neg are one-element float32 device tensors."""
    for t, name in ((x_tensor, "x_tensor"), (scale_tensor, "scale_tensor"), (zp_neg_tensor, "zp_neg_tensor"), (codes_tensor, "codes_tensor")):
        _check_input(t, torch.float32, name)
    _check(scale_tensor.numel() == 1 and zp_neg_tensor.numel() == 1, "scale and zp_neg must hold one element")
    _check(codes_tensor.shape == x_tensor.shape, "codes_tensor must have the shape of x_tensor")
    dev = x_tensor.device
    _check(all(t.device == dev for t in (scale_tensor, zp_neg_tensor, codes_tensor)), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_quantize_codes_f32(x_tensor.data_ptr(), scale_tensor.data_ptr(), zp_neg_tensor.data_ptr(), float(quant_max),
                                         codes_tensor.data_ptr(), x_tensor.numel(), _stream_ptr(dev))
    _raise_for(rc, "quantize_codes")


def quantize_codes_backward(g_tensor, x_tensor, scale_tensor, zp_neg_tensor, quant_max, gx_tensor):
    """gx = g / scale where round(x / scale - zp_neg) lies in [0, quant_max], else 0 (straight-through rounding)."""
    for t, name in ((g_tensor, "g_tensor"), (x_tensor, "x_tensor"), (scale_tensor, "scale_tensor"), (zp_neg_tensor, "zp_neg_tensor"),
                    (gx_tensor, "gx_tensor")):
        _check_input(t, torch.float32, name)
    _check(scale_tensor.numel() == 1 and zp_neg_tensor.numel() == 1, "scale and zp_neg must hold one element")
    _check(g_tensor.shape == x_tensor.shape and gx_tensor.shape == x_tensor.shape, "g, x and gx must have the same shape")
    dev = x_tensor.device
    _check(all(t.device == dev for t in (g_tensor, scale_tensor, zp_neg_tensor, gx_tensor)), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_quantize_codes_backward_f32(g_tensor.data_ptr(), x_tensor.data_ptr(), scale_tensor.data_ptr(),
                                                  zp_neg_tensor.data_ptr(), float(quant_max), gx_tensor.data_ptr(), x_tensor.numel(),
                                                  _stream_ptr(dev))
    _raise_for(rc, "quantize_codes_backward")


def _conv_out_size(H, W, kh, kw, stride, padding, dilation):
    oh = (H + 2 * padding - dilation * (kh - 1) - 1) // stride + 1
    ow = (W + 2 * padding - dilation * (kw - 1) - 1) // stride + 1
    _check(oh > 0 and ow > 0, "empty convolution output")
    return oh, ow


def quantize_codes_nhwc(x_tensor, scale_tensor, zp_neg_tensor, quant_max, codes_tensor, inside_tensor, xsum_tensor, relu=False):
    """The quantiser of the reference's quantize_v2 (micronet+/app_layers.py:147-160) writing what the LUT convolution
    consumes: codes uint8 [B*H*W, C] (a pixel's channel codes adjacent), inside uint8 [B,C,H,W] (the mask of the
    straight-through backward) and xsum float32 [B*H*W] (a pixel's codes summed over the channels), from x float32 [B,C,H,W].
    relu: the quantiser of max(x, 0); inside is then also 0 where x <= 0 (the ReLU's own backward mask)."""
    for t, name, dt in ((x_tensor, "x_tensor", torch.float32), (scale_tensor, "scale_tensor", torch.float32),
                        (zp_neg_tensor, "zp_neg_tensor", torch.float32), (codes_tensor, "codes_tensor", torch.uint8),
                        (inside_tensor, "inside_tensor", torch.uint8), (xsum_tensor, "xsum_tensor", torch.float32)):
        _check_input(t, dt, name)
    _check(x_tensor.dim() == 4, "x must be 4-D")
    Bn, C, H, W = x_tensor.shape
    _check(scale_tensor.numel() == 1 and zp_neg_tensor.numel() == 1, "scale and zp_neg must hold one element")
    _check(tuple(codes_tensor.shape) == (Bn * H * W, C), f"codes_tensor's shape should be {Bn * H * W} x {C}")
    _check(inside_tensor.shape == x_tensor.shape, "inside_tensor must have the shape of x_tensor")
    _check(xsum_tensor.numel() == Bn * H * W, f"xsum_tensor should have {Bn * H * W} elements")
    _check(0 <= quant_max <= 255, "quant_max must fit a byte")
    dev = x_tensor.device
    _check(all(t.device == dev for t in (scale_tensor, zp_neg_tensor, codes_tensor, inside_tensor, xsum_tensor)), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_quantize_codes_nhwc_relu_u8(x_tensor.data_ptr(), scale_tensor.data_ptr(), zp_neg_tensor.data_ptr(), float(quant_max),
                                                  codes_tensor.data_ptr(), inside_tensor.data_ptr(), xsum_tensor.data_ptr(), Bn, C, H * W,
                                                  1 if relu else 0, _stream_ptr(dev))
    _raise_for(rc, "quantize_codes_nhwc")


def im2col_nhwc(codes_tensor, a_tensor, image_shape, kernel_size, stride, padding, dilation):
    """a[(b,oy,ox), (i*kw+j)*C + c] = codes[(b, oy*s-p+i*d, ox*s-p+j*d), c] (0 outside the image); codes uint8 [B*H*W, C],
    image_shape = (B, C, H, W), a uint8 [B*oh*ow, kh*kw*C]."""
    _check_input(codes_tensor, torch.uint8, "codes_tensor")
    _check_input(a_tensor, torch.uint8, "a_tensor")
    Bn, C, H, W = image_shape
    kh, kw = kernel_size
    oh, ow = _conv_out_size(H, W, kh, kw, stride, padding, dilation)
    _check(tuple(codes_tensor.shape) == (Bn * H * W, C), f"codes_tensor's shape should be {Bn * H * W} x {C}")
    _check(tuple(a_tensor.shape) == (Bn * oh * ow, kh * kw * C), f"a_tensor's shape should be {Bn * oh * ow} x {kh * kw * C}")
    dev = codes_tensor.device
    _check(dev == a_tensor.device, "device id not match")
    with torch.cuda.device(dev):
        rc = _lib.amr_im2col_nhwc_u8(codes_tensor.data_ptr(), a_tensor.data_ptr(), Bn, C, H, W, kh, kw, stride, padding, dilation,
                                     _stream_ptr(dev))
    _raise_for(rc, "im2col_nhwc")


def conv_input_grad(cols_tensor, t_tensor, z_w, inside_tensor, scale_tensor, gx_tensor, kernel_size, stride, padding, dilation):
    """gx = inside ? (col2im(cols) + z_w * window sums of t) / scale : 0 for a tap-major cols float32 [B, kh*kw*C, oh*ow] (None:
    gx already holds col2im(cols)); t float32 [B*oh*ow]; inside uint8 and gx float32 [B,C,H,W]."""
    for t, name, dt in ((t_tensor, "t_tensor", torch.float32), (z_w, "z_w", torch.float32), (inside_tensor, "inside_tensor", torch.uint8),
                        (scale_tensor, "scale_tensor", torch.float32), (gx_tensor, "gx_tensor", torch.float32)):
        _check_input(t, dt, name)
    _check(gx_tensor.dim() == 4 and inside_tensor.shape == gx_tensor.shape, "gx must be 4-D and inside of its shape")
    Bn, C, H, W = gx_tensor.shape
    kh, kw = kernel_size
    oh, ow = _conv_out_size(H, W, kh, kw, stride, padding, dilation)
    if cols_tensor is not None:
        _check_input(cols_tensor, torch.float32, "cols_tensor")
        _check(tuple(cols_tensor.shape) == (Bn, kh * kw * C, oh * ow), f"cols_tensor's shape should be {Bn} x {kh * kw * C} x {oh * ow}")
    _check(t_tensor.numel() == Bn * oh * ow, f"t_tensor should have {Bn * oh * ow} elements")
    _check(z_w.numel() == 1 and scale_tensor.numel() == 1, "z_w and scale must hold one element")
    dev = gx_tensor.device
    with torch.cuda.device(dev):
        rc = _lib.amr_conv_input_grad_f32(cols_tensor.data_ptr() if cols_tensor is not None else None, t_tensor.data_ptr(), z_w.data_ptr(),
                                          inside_tensor.data_ptr(), scale_tensor.data_ptr(), gx_tensor.data_ptr(), Bn, C, H, W, kh, kw,
                                          stride, padding, dilation, _stream_ptr(dev))
    _raise_for(rc, "conv_input_grad")


def conv_weight_prepare(w_tensor, scale_tensor, zp_neg_tensor, quant_max, tapmask, bt_tensor, inside_tensor, wresp_tensor):
    """Weight operand of the quantised LUT convolution in one launch: bt uint8 [taps*C, N] (codes, tap-major rows), inside
    uint8 [N,C,kh,kw] (mask of the straight-through backward), wresp float32 [N, L] (response of the codes to an all-ones
    image) from w float32 [N,C,kh,kw] and tapmask float32 [taps, L]."""
    for t, name, dt in ((w_tensor, "w_tensor", torch.float32), (scale_tensor, "scale_tensor", torch.float32),
                        (zp_neg_tensor, "zp_neg_tensor", torch.float32), (tapmask, "tapmask", torch.float32),
                        (bt_tensor, "bt_tensor", torch.uint8), (inside_tensor, "inside_tensor", torch.uint8),
                        (wresp_tensor, "wresp_tensor", torch.float32)):
        _check_input(t, dt, name)
    _check(w_tensor.dim() == 4 and tapmask.dim() == 2, "w must be 4-D and tapmask 2-D")
    N, C, kh, kw = w_tensor.shape
    T, L = kh * kw, tapmask.size(1)
    _check(tapmask.size(0) == T and T <= 64, f"tapmask should have {T} rows (at most 64 taps)")
    _check(tuple(bt_tensor.shape) == (T * C, N), f"bt_tensor's shape should be {T * C} x {N}")
    _check(inside_tensor.shape == w_tensor.shape and wresp_tensor.numel() == N * L, "inside or wresp has the wrong size")
    _check(scale_tensor.numel() == 1 and zp_neg_tensor.numel() == 1 and 0 <= quant_max <= 255, "bad scale, zero point or code range")
    dev = w_tensor.device
    _check(all(t.device == dev for t in (scale_tensor, zp_neg_tensor, tapmask, bt_tensor, inside_tensor, wresp_tensor)), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_conv_weight_prepare_f32(w_tensor.data_ptr(), scale_tensor.data_ptr(), zp_neg_tensor.data_ptr(), float(quant_max),
                                              tapmask.data_ptr(), bt_tensor.data_ptr(), inside_tensor.data_ptr(), wresp_tensor.data_ptr(),
                                              N, C, T, L, _stream_ptr(dev))
    _raise_for(rc, "conv_weight_prepare")


def conv_zero_point_grad(g_tensor, z_a, s_a, s_w, tapmask, gz_tensor, gwr_tensor=None):
    """Gradient of the zero-point term Za * w_resp: gwr[n, pos] = (z_a * (s_a * s_w)) * sum over the batch of g[b, n, pos]
    (optional output) and gz[p, n, tap] = sum over the positions pos of block p of gwr[n, pos] * tapmask[tap, pos], in
    ``conv_zero_point_grad_parts(L)`` blocks of positions (``conv_weight_grad`` adds the blocks; gz.sum(0) is the whole sum).
    g float32 [B, N, ...] contiguous, tapmask float32 [taps, L], gz float32 [parts, N, taps]; scalars one-element device
    tensors.  Fixed summation order."""
    tensors = [(g_tensor, "g_tensor"), (z_a, "z_a"), (s_a, "s_a"), (s_w, "s_w"), (tapmask, "tapmask"), (gz_tensor, "gz_tensor")]
    if gwr_tensor is not None:
        tensors.append((gwr_tensor, "gwr_tensor"))
    for t, name in tensors:
        _check_input(t, torch.float32, name)
    _check(g_tensor.dim() >= 2 and tapmask.dim() == 2, "g must be [B, N, ...] and tapmask [taps, L]")
    Bn, N = g_tensor.size(0), g_tensor.size(1)
    T, L = tapmask.shape
    _check(Bn > 0 and N > 0 and g_tensor.numel() == Bn * N * L, "g does not hold N x L elements per batch entry")
    parts = _lib.amr_conv_zero_point_grad_parts(L)
    _check(tuple(gz_tensor.shape) == (parts, N, T) and T <= 64, f"gz_tensor's shape should be {parts} x {N} x {T} (at most 64 taps)")
    _check(gwr_tensor is None or gwr_tensor.numel() == N * L, "gwr_tensor has the wrong size")
    _check(all(t.numel() == 1 for t in (z_a, s_a, s_w)), "z_a, s_a and s_w must hold one element")
    dev = g_tensor.device
    _check(all(t.device == dev for t, _ in tensors), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        need = _lib.amr_conv_zero_point_grad_workspace_bytes(Bn, N, L)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
        rc = _lib.amr_conv_zero_point_grad_f32(g_tensor.data_ptr(), z_a.data_ptr(), s_a.data_ptr(), s_w.data_ptr(), tapmask.data_ptr(),
                                               gwr_tensor.data_ptr() if gwr_tensor is not None else None, gz_tensor.data_ptr(), Bn, N, L, T,
                                               ws.data_ptr(), ws.numel(), _stream_ptr(dev))
    _raise_for(rc, "conv_zero_point_grad")


def conv_zero_point_grad_parts(positions):
    """Blocks of positions ``conv_zero_point_grad`` folds separately."""
    return _lib.amr_conv_zero_point_grad_parts(int(positions))


def conv_weight_grad(gbt_tensor, gz_tensor, inside_tensor, scale_tensor, gw_tensor):
    """gw[n,c,tap] = inside ? (gbt[tap*C + c, n] + sum over p of gz[p, n, tap]) / scale : 0; gbt float32 [taps*C, N], gz
    float32 [parts, N, taps], inside uint8 and gw float32 [N,C,kh,kw]."""
    for t, name, dt in ((gbt_tensor, "gbt_tensor", torch.float32), (gz_tensor, "gz_tensor", torch.float32),
                        (inside_tensor, "inside_tensor", torch.uint8), (scale_tensor, "scale_tensor", torch.float32), (gw_tensor, "gw_tensor", torch.float32)):
        _check_input(t, dt, name)
    _check(gw_tensor.dim() == 4 and inside_tensor.shape == gw_tensor.shape, "gw must be 4-D and inside of its shape")
    N, C, kh, kw = gw_tensor.shape
    T = kh * kw
    _check(T <= 64 and tuple(gbt_tensor.shape) == (T * C, N) and gz_tensor.dim() == 3 and tuple(gz_tensor.shape[1:]) == (N, T)
           and gz_tensor.size(0) > 0 and scale_tensor.numel() == 1, "gbt, gz or scale has the wrong size (at most 64 taps)")
    dev = gw_tensor.device
    _check(all(t.device == dev for t in (gbt_tensor, gz_tensor, inside_tensor, scale_tensor)), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        rc = _lib.amr_conv_weight_grad_f32(gbt_tensor.data_ptr(), gz_tensor.data_ptr(), gz_tensor.size(0), inside_tensor.data_ptr(), scale_tensor.data_ptr(),
                                           gw_tensor.data_ptr(), N, C, T, _stream_ptr(dev))
    _raise_for(rc, "conv_weight_grad")


def grad_table_fits_halves(table_i16):
    """Whether the expanded-table backward kernels can hold this int16 gradient table (a NumPy array, padded layout) as
    halves; the decision the library takes on the device for every backward call."""
    import numpy as np
    arr = np.ascontiguousarray(table_i16, np.int16)
    rc = _lib.amr_grad_table_fits_halves(arr.ctypes.data, arr.size)
    _check(rc >= 0, f"grad_table_fits_halves failed ({rc}): {_lib.amr_last_error().decode()}")
    return bool(rc)


def conv_input_grad_supported(lut_grad_a_tensor, image_shape, out_channels):
    """Whether approx_conv_input_grad serves this shape (3x3, stride 1, padding 1 is the caller's to check)."""
    Bn, C, H, W = image_shape
    return (lut_grad_a_tensor.dtype == torch.int16 and
            bool(_lib.amr_lut_conv_input_grad_supported(lut_grad_a_tensor.numel(), Bn, C, H, W, out_channels)))


def approx_conv_input_grad(gc_rows, codes_tensor, bt_tensor, lut_grad_a_tensor, t_tensor, z_w, inside_tensor, scale_tensor, gx_tensor,
                           a_fallback=None, cache=None, b_version=0):
    """Input gradient of the quantised 3x3 / stride 1 / padding 1 LUT convolution as one implicit GEMM over the input pixels
    (amr_lut_conv_input_grad_f32): gc_rows float32 [B*H*W, N], codes uint8 [B*H*W, C], bt uint8 [9*C, N] tap-major, gx float32
    [B,C,H,W].  a_fallback: the window matrix uint8 [B*H*W, 9*C]; given, tables that do not fit halves and masked codes are
    served too (through a scratch of 9*C*B*H*W floats), else such a call yields NaN.  cache (a ForwardCache of its own) and
    b_version: the gradient table expanded along bt stays on the device between calls, as in approx_gemm_forward."""
    _check_input(gc_rows, torch.float32, "gc_rows")
    _check_input(codes_tensor, torch.uint8, "codes_tensor")
    _check_input(bt_tensor, torch.uint8, "bt_tensor")
    _check_input(lut_grad_a_tensor, torch.int16, "lut_grad_a_tensor")
    for t, name, dt in ((t_tensor, "t_tensor", torch.float32), (z_w, "z_w", torch.float32), (inside_tensor, "inside_tensor", torch.uint8),
                        (scale_tensor, "scale_tensor", torch.float32), (gx_tensor, "gx_tensor", torch.float32)):
        _check_input(t, dt, name)
    _check(gx_tensor.dim() == 4 and inside_tensor.shape == gx_tensor.shape, "gx must be 4-D and inside of its shape")
    Bn, C, H, W = gx_tensor.shape
    M = Bn * H * W
    N = bt_tensor.size(1)
    _check(tuple(gc_rows.shape) == (M, N), f"gc_rows's shape should be {M} x {N}")
    _check(tuple(codes_tensor.shape) == (M, C), f"codes_tensor's shape should be {M} x {C}")
    _check(tuple(bt_tensor.shape) == (9 * C, N), f"bt_tensor's shape should be {9 * C} x {N}")
    _check(t_tensor.numel() == M and z_w.numel() == 1 and scale_tensor.numel() == 1, "t, z_w or scale has the wrong size")
    _lut_len_check(lut_grad_a_tensor, "lut_grad_a_tensor")
    dev = gx_tensor.device
    cols = None
    if a_fallback is not None:
        _check_input(a_fallback, torch.uint8, "a_fallback")
        _check(tuple(a_fallback.shape) == (M, 9 * C), f"a_fallback's shape should be {M} x {9 * C}")
    with torch.cuda.device(dev):
        if a_fallback is not None:
            cols = torch.empty((Bn, 9 * C, H * W), dtype=torch.float32, device=dev)
        query = _lib.amr_lut_conv_input_grad_cached_workspace_bytes if cache is not None else _lib.amr_lut_conv_input_grad_workspace_bytes
        need = query(lut_grad_a_tensor.numel(), Bn, C, H, W, N)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
        rc = _lib.amr_lut_conv_input_grad_cached_f32(cache._h if cache is not None else None, int(b_version) & 0xFFFFFFFFFFFFFFFF,
                                              gc_rows.data_ptr(), codes_tensor.data_ptr(), bt_tensor.data_ptr(), lut_grad_a_tensor.data_ptr(),
                                              lut_grad_a_tensor.numel(), t_tensor.data_ptr(), z_w.data_ptr(), inside_tensor.data_ptr(),
                                              scale_tensor.data_ptr(), gx_tensor.data_ptr(), Bn, C, H, W, N,
                                              a_fallback.data_ptr() if a_fallback is not None else None,
                                              cols.data_ptr() if cols is not None else None, ws.data_ptr(), ws.numel(), _stream_ptr(dev))
    _raise_for(rc, "approx_conv_input_grad")


def conv_dequant_backward_rowsum(g_tensor, s_a, s_w, gc_rows, t_tensor):
    """conv_dequant_backward that also leaves t[m] = sum over n of gc_rows[m, n] (float32 [B*L])."""
    for t, name in ((g_tensor, "g_tensor"), (s_a, "s_a"), (s_w, "s_w"), (gc_rows, "gc_rows"), (t_tensor, "t_tensor")):
        _check_input(t, torch.float32, name)
    _check(g_tensor.dim() == 4 and gc_rows.dim() == 2, "g must be 4-D and gc_rows 2-D")
    Bn, N = g_tensor.size(0), g_tensor.size(1)
    L = g_tensor.size(2) * g_tensor.size(3)
    _check(tuple(gc_rows.shape) == (Bn * L, N), f"gc_rows's shape should be {Bn * L} x {N}")
    _check(t_tensor.numel() == Bn * L, f"t_tensor should have {Bn * L} elements")
    dev = g_tensor.device
    with torch.cuda.device(dev):
        rc = _lib.amr_conv_dequant_backward_rowsum_f32(g_tensor.data_ptr(), s_a.data_ptr(), s_w.data_ptr(), gc_rows.data_ptr(),
                                                       t_tensor.data_ptr(), Bn, N, L, _stream_ptr(dev))
    _raise_for(rc, "conv_dequant_backward_rowsum")


def conv_output_grad(g_tensor, z_a, s_a, s_w, tapmask, gc_rows, t_tensor, gz_tensor):
    """conv_dequant_backward_rowsum and conv_zero_point_grad (without its optional output) in one call: the output gradient
    is read once where the geometry allows.  tapmask and gz_tensor may both be None (then only gc_rows and t are written)."""
    tensors = [(g_tensor, "g_tensor"), (s_a, "s_a"), (s_w, "s_w"), (gc_rows, "gc_rows"), (t_tensor, "t_tensor")]
    _check((tapmask is None) == (gz_tensor is None), "tapmask and gz_tensor go together")
    if tapmask is not None:
        tensors += [(z_a, "z_a"), (tapmask, "tapmask"), (gz_tensor, "gz_tensor")]
    for t, name in tensors:
        _check_input(t, torch.float32, name)
    _check(g_tensor.dim() == 4 and gc_rows.dim() == 2, "g must be 4-D and gc_rows 2-D")
    Bn, N = g_tensor.size(0), g_tensor.size(1)
    L = g_tensor.size(2) * g_tensor.size(3)
    _check(tuple(gc_rows.shape) == (Bn * L, N), f"gc_rows's shape should be {Bn * L} x {N}")
    _check(t_tensor.numel() == Bn * L, f"t_tensor should have {Bn * L} elements")
    T = 0
    if tapmask is not None:
        T = tapmask.size(0)
        parts = _lib.amr_conv_zero_point_grad_parts(L)
        _check(tapmask.dim() == 2 and tapmask.size(1) == L and T <= 64, f"tapmask should be [taps <= 64, {L}]")
        _check(tuple(gz_tensor.shape) == (parts, N, T), f"gz_tensor's shape should be {parts} x {N} x {T}")
        _check(all(t.numel() == 1 for t in (z_a, s_a, s_w)), "z_a, s_a and s_w must hold one element")
    dev = g_tensor.device
    _check(all(t.device == dev for t, _ in tensors), "All tensors should be on the same device")
    with torch.cuda.device(dev):
        need = _lib.amr_conv_output_grad_workspace_bytes(Bn, N, L) if tapmask is not None else 0
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev) if need else None
        rc = _lib.amr_conv_output_grad_f32(g_tensor.data_ptr(), z_a.data_ptr() if tapmask is not None else None, s_a.data_ptr(), s_w.data_ptr(),
                                           tapmask.data_ptr() if tapmask is not None else None, gc_rows.data_ptr(), t_tensor.data_ptr(),
                                           gz_tensor.data_ptr() if gz_tensor is not None else None, Bn, N, L, T,
                                           ws.data_ptr() if ws is not None else None, need, _stream_ptr(dev))
    _raise_for(rc, "conv_output_grad")


def lds_gather_probe(pattern=0, waves_per_cu=16, iters=4000):
    """Measured LDS gather rate (gathers per second; pattern 2: bytes per second of LDS-direct chunk loads from the L2) of
    the current device; see amr_lds_gather_probe."""
    ms, n = ctypes.c_float(0), ctypes.c_double(0)
    rc = _lib.amr_lds_gather_probe(pattern, waves_per_cu, iters, ctypes.byref(ms), ctypes.byref(n),
                                   _stream_ptr(torch.device("cuda", torch.cuda.current_device())))
    _raise_for(rc, "lds_gather_probe")
    return n.value / (ms.value * 1e-3)
