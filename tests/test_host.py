"""Host-side checks that need no GPU: the C-ABI library loads and exports what include/*.h declares,
the Python operator surface matches the reference's, argument validation raises like the
reference's CHECK_INPUT / TORCH_CHECK, and the table-file reader agrees with the oracle's parser."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from conftest import PKG, ROOT


def _lib():
    path = os.path.join(PKG, "libamr_lutgemm.so")
    assert os.path.exists(path), "build the library first: python appmult-aware-retraining_amd/build.py"
    return ctypes.CDLL(path)


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "amr_lutgemm.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    names = set(re.findall(r"\b(amr_[a-z0-9_]+)\s*\(", hdr))
    assert {"amr_lut_gemm_forward", "amr_lut_gemm_backward", "amr_acc_gemm_forward_fp32"} <= names
    lib = _lib()
    for n in sorted(names):
        assert hasattr(lib, n), n


def test_geometry_and_bits_helpers(oracle):
    lib = _lib()
    lib.amr_bits_from_lut_elems.argtypes = [ctypes.c_int64]
    lib.amr_target_arch.restype = ctypes.c_char_p
    assert lib.amr_target_arch() == b"gfx950"
    for bits in (4, 6, 7, 8):
        r, c, e = ctypes.c_int(), ctypes.c_int(), ctypes.c_int64()
        assert lib.amr_lut_geometry(bits, ctypes.byref(r), ctypes.byref(c), ctypes.byref(e)) == 0
        assert (r.value, c.value, e.value) == oracle.geometry(bits)
        assert lib.amr_bits_from_lut_elems(e.value) == bits
    assert lib.amr_lut_geometry(5, None, None, None) < 0
    assert lib.amr_bits_from_lut_elems(12345) < 0


def test_c_abi_rejects_bad_arguments_without_touching_a_device():
    lib = _lib()
    lib.amr_last_error.restype = ctypes.c_char_p
    vp, i64, i = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.amr_lut_gemm_forward.argtypes = [vp, vp, vp, vp, i64, i, i, i, vp]
    assert lib.amr_lut_gemm_forward(None, None, None, None, 17408, -1, 2, 2, None) == -1
    assert lib.amr_lut_gemm_forward(None, None, None, None, 17000, 2, 2, 2, None) == -2
    assert b"17000" in lib.amr_last_error()
    assert lib.amr_lut_gemm_forward(None, None, None, None, 17408, 0, 5, 0, None) == 0      # empty problem
    assert lib.amr_lut_gemm_forward(None, None, None, None, 17408, 2, 2, 2, None) == -1     # null pointers


def test_float_table_entry_point_checks_arguments_without_touching_a_device():
    lib = _lib()
    vp, i64, i, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    lib.amr_lut_gemm_backward_f32tab.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, ctypes.c_float, i, i, i, i, vp, sz, vp]
    call = lambda elems, M, K, N, L: lib.amr_lut_gemm_backward_f32tab(None, None, None, None, None, None, None, elems, 1.0, M, K, N, L,
                                                                        None, 0, None)
    assert call(66306, -1, 2, 2, 0) == -1          # negative dimension
    assert call(66000, 2, 2, 2, 0) == -2           # not a padded table length
    assert call(66306, 10, 2, 2, 3) == -1          # rows per image must divide M
    assert call(66306, 0, 5, 0, 0) == 0            # empty problem
    assert call(17408, 2, 2, 2, 0) == -1           # null pointers


def test_gradient_tables_keep_their_kind_and_float_tables_need_both(golden_dir):
    import approx_ops
    from self_ops.ops_py import approx_ops as P
    fwd, ga, gb = P.read_lut_file(os.path.join(golden_dir, "lut6_vert_trunc_bp2.txt.gz"), 6)
    saved = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
    try:
        P.set_lookup_tables("cpu", fwd, ga.astype(np.float64) / 16, gb.astype(np.float32) / 16)
        assert P.lut_grad_a.dtype == torch.float32 and P.lut_grad_b.dtype == torch.float32
        assert (P.lut_grad_a.numpy() * 16 == ga).all()
        P.set_lookup_tables("cpu", fwd, ga, gb.astype(np.float32))       # one integer table: both stay int16
        assert P.lut_grad_a.dtype == torch.int16 and P.lut_grad_b.dtype == torch.int16
    finally:
        P.lut_appmult, P.lut_grad_a, P.lut_grad_b = saved
    # the dtype checks come after the device checks, as in the reference: a CPU tensor is reported first
    with pytest.raises(RuntimeError, match="gc_tensor must be a CUDAtensor"):
        approx_ops.approx_gemm_backward(torch.zeros(2, 2), torch.zeros(2, 2, dtype=torch.uint8), torch.zeros(2, 2, dtype=torch.uint8),
                                        torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(5120), torch.zeros(5120), grad_scale=0.5)


def test_python_surface_matches_reference_names():
    import approx_ops
    import self_ops
    from self_ops.ops_py import approx_ops as P
    assert self_ops.__all__ == ['init_lookup_tables', 'approx_gemm_op', 'approx_gemm_baseline_op', 'approx_conv2d_op',
                                'approx_conv2d_baseline_op']
    for n in self_ops.__all__:
        assert callable(getattr(self_ops, n))
    for n in ("approx_gemm_forward", "acc_gemm_forward_fp32", "approx_gemm_backward"):
        assert callable(getattr(approx_ops, n))
    for n in ("lut_appmult", "lut_grad_a", "lut_grad_b", "ApproxGemm", "ApproxGemmBaseline", "AccGemm", "acc_gemm_op"):
        assert hasattr(P, n)


def test_check_input_errors_like_reference():
    import approx_ops
    u8 = lambda *s: torch.zeros(*s, dtype=torch.uint8)
    lut = torch.zeros(17408, dtype=torch.uint16)
    c = torch.zeros(2, 2, dtype=torch.uint32)
    with pytest.raises(RuntimeError, match="a_tensor must be a CUDAtensor"):
        approx_ops.approx_gemm_forward(u8(2, 2), u8(2, 2), c, lut)
    with pytest.raises(RuntimeError, match="gc_tensor must be a CUDAtensor"):
        approx_ops.approx_gemm_backward(torch.zeros(2, 2), u8(2, 2), u8(2, 2), torch.zeros(2, 2), torch.zeros(2, 2),
                                        lut.view(torch.int16), lut.view(torch.int16))
    with pytest.raises(RuntimeError, match="a_tensor must be a CUDAtensor"):
        approx_ops.acc_gemm_forward_fp32(torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2))


def test_conv_op_asserts_like_reference():
    import self_ops
    x = torch.zeros(1, 1, 4, 4)
    w = torch.zeros(1, 1, 3, 3)
    with pytest.raises(AssertionError, match="bias is not supported"):
        self_ops.approx_conv2d_op(x, w, torch.zeros(1), (1, 1), (1, 1), (1, 1), 1)
    with pytest.raises(AssertionError, match="groups is not supported"):
        self_ops.approx_conv2d_op(x, w, None, (1, 1), (1, 1), (1, 1), 2)


@pytest.mark.parametrize("name,bits", [("lut6_vert_trunc_bp2.txt.gz", 6), ("lut7_resub_63_bp8.txt.gz", 7),
                                       ("lut7_vert_trunc_fwdonly.txt.gz", 7)])
def test_table_reader_equals_oracle_parser(oracle, golden_dir, name, bits):
    from self_ops.ops_py import approx_ops as P
    path = os.path.join(golden_dir, name)
    fwd, ga, gb = P.read_lut_file(path, bits)
    f0, a0, b0 = oracle.parse_lut_file(path, bits)
    assert fwd.dtype == np.uint16 and ga.dtype == np.int16 and gb.dtype == np.int16
    assert (fwd == oracle.pack_table(f0, bits, np.uint16)).all()
    assert (ga == oracle.pack_table(a0, bits, np.int16)).all()
    assert (gb == oracle.pack_table(b0, bits, np.int16)).all()


def test_init_lookup_tables_on_cpu_device_and_errors(golden_dir, tmp_path):
    from self_ops.ops_py import approx_ops as P
    P.init_lookup_tables("cpu", os.path.join(golden_dir, "lut6_vert_trunc_bp2.txt.gz"), 6)
    assert P.lut_appmult.dtype == torch.uint16 and P.lut_appmult.shape == (5120,)
    assert P.lut_grad_a.dtype == torch.int16 and P.lut_grad_b.dtype == torch.int16
    with pytest.raises(NotImplementedError):
        P.init_lookup_tables("cpu", "unused", 5)
    bad = tmp_path / "bad.txt"
    bad.write_text("LUT for approximate multiplier:\n0 0\n")
    with pytest.raises(ValueError):
        P.read_lut_file(str(bad), 7)


@pytest.mark.parametrize("bits", [4, 6, 7, 8])
def test_pad_table_places_entries_like_the_reader_and_the_oracle(oracle, bits):
    """The padded layout written by the package's pad_table: entry (a, b) at a * cols + b and zeros everywhere else, i.e.
    what the table reader produces for a file that lists every entry, and what the oracle packs."""
    from self_ops.ops_py import approx_ops as P
    n = 1 << bits
    rng = np.random.default_rng(bits)
    t = rng.integers(0, 65536, (n, n))
    flat = P.pad_table(t, bits, np.uint16)
    rows, cols, elems = P.lut_geometry(bits)
    assert flat.shape == (elems,) and flat.dtype == np.uint16
    for a, b in ((0, 0), (n - 1, n - 1), (3, n - 2), (n - 1, 0)):
        assert flat[a * cols + b] == t[a, b]
    assert flat.astype(np.int64).sum() == t.sum()                       # nothing but the entries is non-zero
    assert (flat == oracle.pack_table(t, bits, np.uint16)).all()
    g = rng.standard_normal((n, n)).astype(np.float32)
    assert (P.pad_table(g, bits, np.float32) == oracle.pack_table(g, bits, np.float32)).all()


def test_layer_level_entry_points_check_arguments_without_touching_a_device():
    """The entry points of the quantised layer on uint8 codes reject bad shapes, null pointers and unknown table lengths
    with an AMR_E* code before anything is launched; the size queries answer 0 for what the kernels do not serve."""
    lib = _lib()
    lib.amr_last_error.restype = ctypes.c_char_p
    vp, i64, i, sz, f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
    lib.amr_quantize_codes_nhwc_u8.argtypes = [vp, vp, vp, f, vp, vp, vp, i, i, i, vp]
    assert lib.amr_quantize_codes_nhwc_u8(None, None, None, 127.0, None, None, None, 2, 0, 4, None) == -1      # no channels
    assert lib.amr_quantize_codes_nhwc_u8(None, None, None, 300.0, None, None, None, 2, 3, 4, None) == -1      # codes must fit a byte
    assert lib.amr_quantize_codes_nhwc_u8(None, None, None, 127.0, None, None, None, 0, 3, 4, None) == 0       # empty batch
    assert lib.amr_quantize_codes_nhwc_u8(None, None, None, 127.0, None, None, None, 2, 3, 4, None) == -1      # null pointers
    lib.amr_quantize_codes_nhwc_relu_u8.argtypes = [vp, vp, vp, f, vp, vp, vp, i, i, i, i, vp]
    assert lib.amr_quantize_codes_nhwc_relu_u8(None, None, None, 127.0, None, None, None, 2, 3, 4, 1, None) == -1  # null pointers
    assert lib.amr_quantize_codes_nhwc_relu_u8(None, None, None, 127.0, None, None, None, 0, 3, 4, 1, None) == 0   # empty batch
    lib.amr_im2col_nhwc_u8.argtypes = [vp, vp, i, i, i, i, i, i, i, i, i, vp]
    assert lib.amr_im2col_nhwc_u8(None, None, 2, 3, 4, 4, 5, 5, 1, 0, 1, None) == -1                            # window larger than the image
    assert lib.amr_im2col_nhwc_u8(None, None, 2, 3, 4, 4, 3, 3, 1, 1, 1, None) == -1                            # null pointers
    lib.amr_lut_conv_forward_dequant_f32.argtypes = [vp, vp, vp, i64, i, i, i, i] + [vp] * 9 + [vp, sz, vp]
    call = lambda elems, M, K, N, L: lib.amr_lut_conv_forward_dequant_f32(None, None, None, elems, M, K, N, L, *([None] * 9), None, 0, None)
    assert call(17408, 10, 4, 4, 3) == -1          # positions must divide M
    assert call(17000, 12, 4, 4, 3) == -2          # not a padded table length
    assert call(17408, 0, 4, 4, 3) == 0            # empty problem
    assert call(17408, 12, 4, 4, 3) == -1          # null pointers
    lib.amr_lut_conv_forward_dequant_workspace_bytes.argtypes = [i64, i, i, i]
    lib.amr_lut_conv_forward_dequant_workspace_bytes.restype = sz
    assert lib.amr_lut_conv_forward_dequant_workspace_bytes(17408, 100, 27, 10) == 100 * 10 * 4
    lib.amr_lut_conv_input_grad_supported.argtypes = [i64, i, i, i, i, i]
    lib.amr_lut_conv_input_grad_workspace_bytes.argtypes = [i64, i, i, i, i, i]
    lib.amr_lut_conv_input_grad_workspace_bytes.restype = sz
    assert lib.amr_lut_conv_input_grad_supported(17408, 512, 64, 32, 32, 64) == 1
    assert lib.amr_lut_conv_input_grad_supported(66306, 512, 64, 32, 32, 64) == 0      # 8-bit table
    assert lib.amr_lut_conv_input_grad_supported(17408, 512, 24, 32, 32, 64) == 0      # channels no multiple of 16
    assert lib.amr_lut_conv_input_grad_workspace_bytes(17408, 512, 24, 32, 32, 64) == 0
    assert lib.amr_lut_conv_input_grad_workspace_bytes(17408, 512, 64, 32, 32, 64) == 256 + 512 * 1024 * 4 + 9 * 64 * 64 * 256
    lib.amr_lut_conv_input_grad_f32.argtypes = [vp] * 4 + [i64] + [vp] * 5 + [i] * 5 + [vp, vp, vp, sz, vp]
    assert lib.amr_lut_conv_input_grad_f32(*([None] * 4), 17408, *([None] * 5), 512, 64, 32, 32, 64, None, None, None, 0, None) == -1
    lib.amr_lut_conv_input_grad_cached_workspace_bytes.argtypes = [i64, i, i, i, i, i]
    lib.amr_lut_conv_input_grad_cached_workspace_bytes.restype = sz
    assert lib.amr_lut_conv_input_grad_cached_workspace_bytes(17408, 512, 64, 32, 32, 64) == 256 + 512 * 1024 * 4
    assert lib.amr_lut_conv_input_grad_cached_workspace_bytes(17408, 512, 24, 32, 32, 64) == 0
    lib.amr_lut_conv_input_grad_cached_f32.argtypes = [vp, ctypes.c_uint64] + [vp] * 4 + [i64] + [vp] * 5 + [i] * 5 + [vp, vp, vp, sz, vp]
    assert lib.amr_lut_conv_input_grad_cached_f32(None, 0, *([None] * 4), 17408, *([None] * 5), 512, 64, 32, 32, 64, None, None, None, 0, None) == -1
    lib.amr_observe_minmax_f32.argtypes = [vp, i64, vp, vp, vp, vp, vp, i] + [f] * 5 + [vp]
    assert lib.amr_observe_minmax_f32(None, 10, None, None, None, None, None, 3, 0.9, 0.1, 127.0, 0.0, 1e-7, None) == -1   # mode
    assert lib.amr_observe_minmax_f32(None, 10, None, None, None, None, None, 7, 0.9, 0.1, 127.0, 0.0, 1e-7, None) == -1   # mode 3 with the ReLU bit
    assert lib.amr_observe_minmax_f32(None, 10, None, None, None, None, None, 8, 0.9, 0.1, 127.0, 0.0, 1e-7, None) == -1   # unknown bit
    assert lib.amr_observe_minmax_f32(None, 10, None, None, None, None, None, 2, 0.9, 0.1, 127.0, 0.0, 1e-7, None) == -1   # null pointers
    lib.amr_lut_conv_forward_implicit_supported.argtypes = [i64, i, i, i, i, i]
    lib.amr_lut_conv_forward_implicit_workspace_bytes.argtypes = [i64, i, i, i, i, i, i, i]
    lib.amr_lut_conv_forward_implicit_workspace_bytes.restype = sz
    assert lib.amr_lut_conv_forward_implicit_supported(17408, 512, 64, 32, 32, 64) == 1
    assert lib.amr_lut_conv_forward_implicit_supported(17408, 512, 24, 32, 32, 64) == 0      # channels no multiple of 16
    assert lib.amr_lut_conv_forward_implicit_supported(66306, 512, 64, 32, 32, 64) == 0      # 8-bit table
    assert lib.amr_lut_conv_forward_implicit_supported(17408, 4, 64, 32, 32, 64) == 0        # too few rows to fill the device without a K split
    assert lib.amr_lut_conv_forward_implicit_supported(17000, 512, 64, 32, 32, 64) == 0      # not a padded table length
    e_bytes = 256 + 2 * 144 * 32768
    assert lib.amr_lut_conv_forward_implicit_workspace_bytes(17408, 512, 64, 32, 32, 64, 0, 0) == e_bytes
    assert lib.amr_lut_conv_forward_implicit_workspace_bytes(17408, 512, 64, 32, 32, 64, 1, 0) == 0
    assert lib.amr_lut_conv_forward_implicit_workspace_bytes(17408, 512, 64, 32, 32, 64, 1, 1) == 512 * 1024 * 64 * 4
    lib.amr_lut_conv_forward_implicit_f32.argtypes = [vp, ctypes.c_uint64, vp, vp, vp, i64, i, i, i, i, i] + [vp] * 10 + [vp, sz, vp]
    icall = lambda elems, B, C: lib.amr_lut_conv_forward_implicit_f32(None, 0, None, None, None, elems, B, C, 32, 32, 64, *([None] * 10), None, 0, None)
    assert icall(17000, 512, 64) == -2             # not a padded table length
    assert icall(17408, 0, 64) == -1               # empty batch is a bad shape here
    assert icall(17408, 512, 24) == -4             # unsupported geometry
    assert icall(17408, 512, 64) == -1             # null pointers
    lib.amr_conv_weight_prepare_f32.argtypes = [vp, vp, vp, f, vp, vp, vp, vp, i, i, i, i, vp]
    assert lib.amr_conv_weight_prepare_f32(*([None] * 3), 127.0, *([None] * 4), 8, 4, 81, 16, None) == -1     # more than 64 taps
    assert lib.amr_conv_weight_prepare_f32(*([None] * 3), 300.0, *([None] * 4), 8, 4, 9, 16, None) == -1      # codes must fit a byte
    assert lib.amr_conv_weight_prepare_f32(*([None] * 3), 127.0, *([None] * 4), 8, 4, 9, 16, None) == -1      # null pointers
    lib.amr_conv_zero_point_grad_workspace_bytes.argtypes = [i, i, i]
    lib.amr_conv_zero_point_grad_workspace_bytes.restype = sz
    assert lib.amr_conv_zero_point_grad_workspace_bytes(0, 10, 10) == 0
    assert lib.amr_conv_zero_point_grad_workspace_bytes(4, 10, 10) == 100 * 4                                 # few images: one segment
    assert lib.amr_conv_zero_point_grad_workspace_bytes(512, 64, 1024) % (65536 * 4) == 0
    lib.amr_conv_zero_point_grad_f32.argtypes = [vp] * 7 + [i, i, i, i, vp, sz, vp]
    assert lib.amr_conv_zero_point_grad_f32(*([None] * 7), 0, 4, 10, 9, None, 0, None) == -1
    assert lib.amr_conv_zero_point_grad_f32(*([None] * 7), 4, 4, 10, 65, None, 0, None) == -1                 # more than 64 taps
    assert lib.amr_conv_zero_point_grad_f32(*([None] * 7), 4, 4, 10, 9, None, 0, None) == -1                  # null pointers
    assert lib.amr_conv_zero_point_grad_parts(1024) == 16 and lib.amr_conv_zero_point_grad_parts(16) == 1 and lib.amr_conv_zero_point_grad_parts(0) == 0
    lib.amr_conv_output_grad_workspace_bytes.argtypes = [i, i, i]
    lib.amr_conv_output_grad_workspace_bytes.restype = sz
    assert lib.amr_conv_output_grad_workspace_bytes(0, 64, 1024) == 0
    assert lib.amr_conv_output_grad_workspace_bytes(512, 64, 1024) == 64 * 64 * 1024 * 4          # 64 segments of 8 images
    assert lib.amr_conv_output_grad_workspace_bytes(512, 512, 16) == lib.amr_conv_zero_point_grad_workspace_bytes(512, 512, 16)
    lib.amr_conv_output_grad_f32.argtypes = [vp] * 8 + [i, i, i, i, vp, sz, vp]
    assert lib.amr_conv_output_grad_f32(*([None] * 8), 0, 64, 16, 9, None, 0, None) == -1
    assert lib.amr_conv_output_grad_f32(*([None] * 8), 4, 64, 16, 9, None, 0, None) == -1                     # null pointers
    lib.amr_conv_weight_grad_f32.argtypes = [vp, vp, i, vp, vp, vp, i, i, i, vp]
    assert lib.amr_conv_weight_grad_f32(None, None, 1, None, None, None, 8, 0, 9, None) == -1
    assert lib.amr_conv_weight_grad_f32(None, None, 0, None, None, None, 8, 4, 9, None) == -1                 # no block of positions
    assert lib.amr_conv_weight_grad_f32(None, None, 1, None, None, None, 8, 4, 9, None) == -1                 # null pointers
    # the decision on a gradient table in host memory
    lib.amr_grad_table_fits_halves.argtypes = [vp, i64]
    small = np.zeros(17408, np.int16); small[:100] = 2048; small[200:300] = -2048
    wide = small.copy(); wide[5] = 6000
    shifted = np.zeros(17408, np.int16); shifted[:129 * 130] = 1500; shifted[7] = 3000; shifted[9] = -500
    assert lib.amr_grad_table_fits_halves(small.ctypes.data, small.size) == 1
    assert lib.amr_grad_table_fits_halves(wide.ctypes.data, wide.size) == 0            # spans more than 4096
    assert lib.amr_grad_table_fits_halves(shifted.ctypes.data, shifted.size) == 1      # fits with an offset that does not swamp the entries
    assert lib.amr_grad_table_fits_halves(small.ctypes.data, 17000) < 0
    # the cache object lives on the host until it is used
    h = vp()
    lib.amr_fwd_cache_create.argtypes = [ctypes.POINTER(vp)]
    lib.amr_fwd_cache_destroy.argtypes = [vp]
    lib.amr_fwd_cache_stats.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(sz)]
    assert lib.amr_fwd_cache_create(ctypes.byref(h)) == 0 and h.value
    hits, misses, held = ctypes.c_uint64(9), ctypes.c_uint64(9), sz(9)
    assert lib.amr_fwd_cache_stats(h, ctypes.byref(hits), ctypes.byref(misses), ctypes.byref(held)) == 0
    assert (hits.value, misses.value, held.value) == (0, 0, 0)
    assert lib.amr_fwd_cache_destroy(h) == 0
