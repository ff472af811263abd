"""GPU parity tests (run on the MI355X box with -m gpu): the HIP path, called through the C ABI of
libamr_lutgemm.so, against the CPU oracle on the same seeded inputs.

Bars: forward bit-exact (uint32); backward within 1e-5 of the float64 sums, relative to the sum of
term magnitudes per output (fp32 summation-order tolerance) and norm-wise relative to the largest
output; STE tables with small-integer gC are bit-exact.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from conftest import PKG

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def lib():
    assert torch.cuda.is_available(), "gpu tests need a device"
    L = ctypes.CDLL(os.path.join(PKG, "libamr_lutgemm.so"))
    vp, i64, i, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    L.amr_last_error.restype = ctypes.c_char_p
    L.amr_lut_gemm_forward.argtypes = [vp, vp, vp, vp, i64, i, i, i, vp]
    L.amr_lut_gemm_forward_ws.argtypes = [vp, vp, vp, vp, i64, i, i, i, vp, sz, vp]
    L.amr_lut_gemm_forward_f32_ws.argtypes = [vp, vp, vp, vp, i64, i, i, i, vp, sz, vp]
    L.amr_lut_gemm_forward_workspace_bytes.argtypes = [i64, i, i, i]
    L.amr_lut_gemm_forward_workspace_bytes.restype = sz
    L.amr_lut_gemm_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i, i, i, vp, sz, vp]
    L.amr_lut_gemm_backward_ex.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i, i, i, i, vp, sz, vp]
    L.amr_lut_gemm_backward_f32tab.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, ctypes.c_float, i, i, i, i, vp, sz, vp]
    L.amr_lut_gemm_backward_f32tab_workspace_bytes.argtypes = [i, i, i]
    L.amr_lut_gemm_backward_f32tab_workspace_bytes.restype = sz
    L.amr_lut_gemm_backward_workspace_bytes.argtypes = [i, i, i]
    L.amr_lut_gemm_backward_workspace_bytes.restype = sz
    L.amr_lut_gemm_backward_workspace_bytes_for.argtypes = [i64, i, i, i]
    L.amr_lut_gemm_backward_workspace_bytes_for.restype = sz
    L.amr_acc_gemm_forward_fp32.argtypes = [vp, vp, vp, i, i, i, vp]
    # mode 2: the expanded-table kernels wherever the shape allows, so that the test sizes (small next to the sizes
    # at which the library would pick them by itself) exercise them; mode 0 / 1 have tests of their own below
    L.amr_set_expanded_table_kernels(2)
    yield L
    L.amr_set_expanded_table_kernels(1)


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def gpu_forward(lib, A, B, flat_u16):
    M, K = A.shape
    N = B.shape[1]
    a, b, l = dev(A), dev(B), dev(flat_u16)
    c = torch.full((M, N), 0xDEADBEEF, dtype=torch.int64, device="cuda").to(torch.int32)  # poison: op must overwrite
    rc = lib.amr_lut_gemm_forward(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, None)
    assert rc == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    return c.cpu().numpy().view(np.uint32)


def gpu_backward(lib, g, A, B, la, lb, own_workspace=True, ga_offset_floats=0):
    M, K = A.shape
    N = B.shape[1]
    gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(la), dev(lb)
    # (ga_offset_floats: gA starts that many floats into its allocation, i.e. aligned to 4 bytes only)
    ga = torch.full((M * K + ga_offset_floats,), float("nan"), device="cuda")[ga_offset_floats:].view(M, K)
    gb = torch.full((K, N), float("nan"), device="cuda")
    need = lib.amr_lut_gemm_backward_workspace_bytes(M, K, N)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda") if own_workspace else None
    rc = lib.amr_lut_gemm_backward(gd.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                   tb.data_ptr(), ta.numel(), M, K, N, ws.data_ptr() if ws is not None else None,
                                   need if ws is not None else 0, None)
    assert rc == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    return ga.cpu().numpy(), gb.cpu().numpy()


def seed_of(*key):
    """Seed of a test case from its parameters: the same in every process (hash() of a str is not)."""
    import zlib
    return zlib.crc32(repr(key).encode())


def rand_case(seed, M, K, N, bits):
    rng = np.random.default_rng(seed)
    n = 1 << bits
    A = rng.integers(0, n, (M, K)).astype(np.uint8)
    B = rng.integers(0, n, (K, N)).astype(np.uint8)
    T = rng.integers(0, 65536, (n, n))
    return rng, A, B, T


FWD_SHAPES = [(1, 1, 1), (3, 5, 7), (9, 27, 10), (64, 64, 64), (33, 130, 65), (128, 576, 64), (257, 100, 129),
              (100, 64, 300), (40, 1152, 128), (1000, 27, 64), (70, 2304, 256), (17, 9, 513)]


@pytest.mark.parametrize("bits", [7, 8, 6, 4])
@pytest.mark.parametrize("shape", FWD_SHAPES)
def test_forward_bit_exact_random_tables(lib, oracle, bits, shape):
    print("forward", bits, shape, flush=True)
    _, A, B, T = rand_case(seed_of(bits, shape), *shape, bits)
    flat = oracle.pack_table(T, bits, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == oracle.forward_c(A, B, flat, bits)).all()


# shapes with M >= 2048, K >= 32 and K % 4 == 0 take the expanded-table forward kernels in the mode the fixture sets
# (K % 16 != 0 moves the last group of codes back; a small M x N grid splits K over workgroups)
BIG_M_SHAPES = [(2048, 512, 64), (2081, 515, 65), (2081, 516, 65), (3000, 27, 10), (4096, 640, 300), (2500, 1153, 128),
                (2500, 1156, 128), (5000, 777, 1), (5000, 776, 1), (2048, 2056, 96), (3100, 520, 33),
                # short K (the expanded-table kernels take K >= 32 when forced, K >= 64 by themselves)
                (2048, 32, 64), (2500, 36, 33), (4096, 64, 512), (2048, 100, 40), (65536, 64, 128)]


@pytest.mark.parametrize("bits", [7, 6, 4, 8])
@pytest.mark.parametrize("shape", BIG_M_SHAPES)
def test_forward_bit_exact_large_m(lib, oracle, bits, shape):
    print("forward large M", bits, shape, flush=True)
    _, A, B, T = rand_case(seed_of(bits, shape, "L"), *shape, bits)
    flat = oracle.pack_table(T, bits, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == oracle.forward_c(A, B, flat, bits)).all()


def test_forward_large_m_small_table_values_masked_codes_and_own_workspace(lib, oracle):
    print("forward large M masked / workspace", flush=True)
    M, K, N = 2600, 532, 70
    rng, A, B, _ = rand_case(99, M, K, N, 7)
    T = oracle.synth_lut(7, 64, rng)                      # max < 16384: packed 16-bit partial sums
    flat = oracle.pack_table(T, 7, np.uint16)
    want = oracle.forward_c(A, B, flat, 7)
    assert (gpu_forward(lib, A, B, flat) == want).all()
    a, b, l = dev(A), dev(B), dev(flat)
    need = lib.amr_lut_gemm_forward_workspace_bytes(l.numel(), M, K, N)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    assert lib.amr_lut_gemm_forward_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, ws.data_ptr(), need, None) == 0
    torch.cuda.synchronize()
    assert (c.cpu().numpy().view(np.uint32) == want).all()
    assert lib.amr_lut_gemm_forward_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, ws.data_ptr(), need - 1, None) == -3
    # masked code 2^b in both operands (zero contribution), rows spread over several workgroups
    A2, B2 = A.copy(), B.copy()
    A2[::7, 3] = 128
    A2[1234, :] = 128
    B2[5, ::3] = 128
    want2 = oracle.forward_c(A2, B2, flat, 7)
    assert (gpu_forward(lib, A2, B2, flat) == want2).all()
    # and the next call without masked codes is clean again
    assert (gpu_forward(lib, A, B, flat) == want).all()


def test_forward_config1_bit_exact_and_exact_multiplier(lib, oracle):
    print("forward config1", flush=True)
    A, B, T, _ = oracle.synth_gemm(4096, 576, 64, bits=7, err=64, seed=0)
    flat = oracle.pack_table(T, 7, np.uint16)
    got = gpu_forward(lib, A, B, flat)
    assert (got == oracle.forward_c(A, B, flat, 7)).all()
    exact = oracle.pack_table(np.arange(128)[:, None] * np.arange(128)[None, :], 7, np.uint16)
    assert (gpu_forward(lib, A, B, exact) == (A.astype(np.int64) @ B.astype(np.int64)).astype(np.uint32)).all()


def test_forward_masked_code_and_unaligned_views(lib, oracle):
    print("forward masked/unaligned", flush=True)
    _, A, B, T = rand_case(77, 50, 37, 70, 7)
    A[:, 3] = 128
    B[5, :] = 128
    flat = oracle.pack_table(T, 7, np.uint16)
    want = oracle.forward_c(A, B, flat, 7)
    assert (gpu_forward(lib, A, B, flat) == want).all()
    # operand pointers at odd byte addresses (a slice of a larger buffer)
    buf_a = torch.zeros(A.size + 3, dtype=torch.uint8, device="cuda")
    buf_b = torch.zeros(B.size + 1, dtype=torch.uint8, device="cuda")
    buf_a[3:] = dev(A).flatten()
    buf_b[1:] = dev(B).flatten()
    l = dev(flat)
    c = torch.zeros(want.shape, dtype=torch.int32, device="cuda")
    rc = lib.amr_lut_gemm_forward(buf_a.data_ptr() + 3, buf_b.data_ptr() + 1, c.data_ptr(), l.data_ptr(), l.numel(), 50, 37, 70, None)
    assert rc == 0
    assert (c.cpu().numpy().view(np.uint32) == want).all()


def test_forward_golden_shipped_tables(lib, oracle, golden_dir):
    print("forward golden", flush=True)
    fwd, _, _ = oracle.parse_lut_file(os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), 7)
    _, A, B, _ = rand_case(5, 300, 200, 96, 7)
    flat = oracle.pack_table(fwd, 7, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == oracle.forward_np(A, B, fwd)).all()
    z = np.load(os.path.join(golden_dir, "lut8_resub_183.npz"))
    _, A, B, _ = rand_case(6, 200, 150, 80, 8)
    flat = oracle.pack_table(z["fwd"], 8, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == oracle.forward_np(A, B, z["fwd"])).all()


# the float32 output of the forward pass = the uint32 sums converted with round-to-nearest-even (what torch's
# .to(float32) does): direct kernels, K split over workgroups (small M), expanded-table kernels, both table widths of the
# packed / unpacked flavours, the masked-code fall-back, sums beyond 2^24 and wrapped sums
@pytest.mark.parametrize("bits,shape,big", [(7, (37, 530, 70), False), (7, (300, 2048, 64), True), (8, (100, 300, 130), True),
                                            (7, (4096, 576, 64), False), (7, (2048, 4608, 96), True), (6, (2100, 600, 33), False),
                                            (7, (2048, 1024, 64), True), (4, (4100, 512, 40), False)])
def test_forward_float_output_is_the_converted_integer_sum(lib, oracle, bits, shape, big):
    print("forward f32", bits, shape, big, flush=True)
    M, K, N = shape
    rng, A, B, _ = rand_case(seed_of(bits, shape, "f32"), M, K, N, bits)
    n = 1 << bits
    T = rng.integers(60000, 65536, (n, n)) if big else rng.integers(0, 300, (n, n))      # big: sums pass 2^24 (and 2^32 for long K)
    flat = oracle.pack_table(T, bits, np.uint16)
    if bits == 7:
        A[::9, 5] = 128            # masked codes: the fall-back kernel stores the floats itself
    want = gpu_forward(lib, A, B, flat)
    assert (want == oracle.forward_c(A, B, flat, bits)).all()
    a, b, l = dev(A), dev(B), dev(flat)
    c = torch.full((M, N), float("nan"), device="cuda")
    need = lib.amr_lut_gemm_forward_workspace_bytes(l.numel(), M, K, N)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    rc = lib.amr_lut_gemm_forward_f32_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, ws.data_ptr(),
                                         need, None)
    assert rc == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    ref = torch.from_numpy(want.astype(np.int64)).to(torch.float32)          # int64 -> float32: round to nearest even
    assert torch.equal(c.cpu(), ref)
    if big:
        assert (want > 2**24).any()


def test_forward_wraparound_and_k_zero(lib, oracle):
    print("forward wrap", flush=True)
    A = np.full((3, 70000), 255, np.uint8)
    B = np.full((70000, 5), 255, np.uint8)
    flat = oracle.pack_table(np.full((256, 256), 65535), 8, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == (70000 * 65535) % 2**32).all()
    assert (gpu_forward(lib, np.zeros((4, 0), np.uint8), np.zeros((0, 6), np.uint8), flat) == 0).all()


def check_backward(oracle, got, g, A, B, la, lb, bits, factor=1.0 / 16):
    gA, gB = got
    a64, b64, absA, absB = oracle.backward_c_f64(g, A, B, la, lb, bits, factor=factor, want_abs=True)
    assert np.isfinite(gA).all() and np.isfinite(gB).all()
    for x, r, ab in ((gA, a64, absA), (gB, b64, absB)):
        err = np.abs(x - r)
        assert np.max(err / np.maximum(ab, 1e-30)) < TOL          # relative to sum of |terms|
        assert np.max(err) <= TOL * np.max(np.abs(r)) + 1e-30      # norm-wise relative


BWD_SHAPES = [(1, 1, 1), (3, 5, 7), (9, 27, 10), (64, 64, 64), (33, 130, 65), (600, 96, 64), (257, 100, 129),
              (1100, 27, 64), (300, 288, 256), (70, 50, 513)]


@pytest.mark.parametrize("bits", [7, 8, 6])
@pytest.mark.parametrize("shape", BWD_SHAPES)
def test_backward_within_tolerance_random_tables(lib, oracle, bits, shape):
    print("backward", bits, shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(bits, shape, "b"), *shape, bits)
    n = 1 << bits
    la = oracle.pack_table(rng.integers(-32768, 32768, (n, n)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(-32768, 32768, (n, n)), bits, np.int16)
    g = rng.standard_normal((shape[0], shape[2])).astype(np.float32)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, bits)


# M >= 1024 takes the expanded-table backward kernels (tables of at most 7 bits)
BWD_BIG_M_SHAPES = [(4096, 8, 64), (4100, 27, 10), (5000, 130, 65), (4096, 64, 300), (4500, 70, 129), (4096, 33, 513), (9000, 5, 200),
                    (1024, 64, 64), (1500, 40, 70), (3000, 130, 65), (1100, 9, 200)]


@pytest.mark.parametrize("bits", [7, 6, 8])
@pytest.mark.parametrize("shape", BWD_BIG_M_SHAPES)
def test_backward_within_tolerance_large_m(lib, oracle, bits, shape):
    print("backward large M", bits, shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(bits, shape, "bL"), *shape, bits)
    n = 1 << bits
    la = oracle.pack_table(rng.integers(-32768, 32768, (n, n)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(-32768, 32768, (n, n)), bits, np.int16)
    g = rng.standard_normal((shape[0], shape[2])).astype(np.float32)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, bits)


# 8-bit tables, M % 256 == 0, M >= 1024 (forced; 2048 by itself), K % 4 == 0, N % 64 == 0: gradB on the expanded table held as int16
# (one to three column tiles, one to 144 k tiles, one and several M splits)
SLAB8_SHAPES = [(2048, 4, 64), (4096, 8, 64), (4096, 64, 128), (8192, 36, 192), (2304, 12, 64), (16384, 576, 64), (32768, 20, 64),
                (1024, 16, 128), (1280, 8, 64)]


@pytest.mark.parametrize("shape", SLAB8_SHAPES)
def test_backward_8bit_int16_slab(lib, oracle, shape):
    print("backward 8-bit int16 slab", shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(shape, "s8"), *shape, 8)
    A[0, :] = 255                                                       # the last code of both operands occurs
    B[:, 0] = 255
    la = oracle.pack_table(rng.integers(-32768, 32768, (256, 256)), 8, np.int16)
    Gb = rng.integers(-32768, 32768, (256, 256))
    Gb[255, 255], Gb[0, 0], Gb[255, 0], Gb[0, 255] = -32768, 32767, 12345, -12345
    lb = oracle.pack_table(Gb, 8, np.int16)
    g = (rng.standard_normal((shape[0], shape[2])) + 0.25).astype(np.float32)
    got = gpu_backward(lib, g, A, B, la, lb)
    check_backward(oracle, got, g, A, B, la, lb, 8)
    old = lib.amr_set_expanded_table_kernels(0)                          # the direct kernels: same sums in another order
    try:
        ref = gpu_backward(lib, g, A, B, la, lb)
    finally:
        lib.amr_set_expanded_table_kernels(old)
    assert np.abs(got[1] - ref[1]).max() <= 1e-5 * np.abs(ref[1]).max()


# 8-bit tables, M >= 512 (forced; 4096 by itself), K % 16 == 0, N % 16 == 0: gradA on the expanded table held as int16, 16 or
# 32 k per tile, one to twelve column tiles, ragged last row block
SLAB8_GA_SHAPES = [(4096, 16, 16), (4096, 64, 64), (4100, 32, 48), (9001, 64, 16), (2148, 144, 160), (33011, 128, 32), (32768, 128, 192),
                   (1024, 16, 64)]


@pytest.mark.parametrize("shape", SLAB8_GA_SHAPES)
def test_backward_8bit_int16_expanded_table_gradA(lib, oracle, shape):
    print("backward 8-bit int16 expanded table, gradA", shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(shape, "a8"), *shape, 8)
    A[0, :] = 255                                                       # the last code of both operands occurs
    A[-1, :] = 128
    B[:, 0] = 255
    Ga = rng.integers(-32768, 32768, (256, 256))
    Ga[255, 255], Ga[0, 0], Ga[255, 0], Ga[0, 255] = -32768, 32767, 12345, -12345
    la = oracle.pack_table(Ga, 8, np.int16)
    lb = oracle.pack_table(rng.integers(-32768, 32768, (256, 256)), 8, np.int16)
    g = (rng.standard_normal((shape[0], shape[2])) + 0.25).astype(np.float32)
    got = gpu_backward(lib, g, A, B, la, lb)
    check_backward(oracle, got, g, A, B, la, lb, 8)
    for off in (0, 1):                                                  # gA aligned to 16 and to 4 bytes
        again = gpu_backward(lib, g, A, B, la, lb, ga_offset_floats=off)
        assert np.array_equal(again[0], got[0])


# 8-bit tables, at most 1024 rows: the k tiles of the direct gradA kernel are its only workgroups, so their depth (16, 20 or 24 k)
# follows the count that fills the CUs in the fewest rounds (256 CUs: K = 4612 -> 20, K = 6142 -> 24); K % 4 != 0 takes the
# scalar stores, a last tile sticking out of K the clamped loads
@pytest.mark.parametrize("kind", ["i16", "f32"])
@pytest.mark.parametrize("shape,L", [((300, 4612, 40), 4), ((130, 6142, 24), 10), ((1024, 4608, 16), 64), ((512, 9220, 8), 0)])
def test_backward_8bit_one_row_block_deep_k_tiles(lib, oracle, kind, shape, L):
    print("backward 8-bit, one row block, deep k tiles", kind, shape, flush=True)
    M, K, N = shape
    rng, A, B, _ = rand_case(seed_of(shape, "deep"), *shape, 8)
    g = rng.standard_normal((M, N)).astype(np.float32)
    if kind == "f32":
        la = oracle.pack_table(rng.standard_normal((256, 256)) * 40 + 3, 8, np.float32)
        lb = oracle.pack_table(rng.standard_normal((256, 256)) * 40 - 5, 8, np.float32)
        got = gpu_backward_f32tab(lib, g, A, B, la, lb, 0.5)
        check_backward(oracle, got, g, A, B, la, lb, 8, factor=np.float32(0.5))
        if L:
            gat = gpu_backward_f32tab(lib, g, A, B, la, lb, 0.5, rows_per_image=L)[0]
            assert np.array_equal(gat.reshape(M // L, K, L).transpose(0, 2, 1).reshape(M, K), got[0])
        return
    la = oracle.pack_table(rng.integers(-32768, 32768, (256, 256)), 8, np.int16)
    lb = oracle.pack_table(rng.integers(-32768, 32768, (256, 256)), 8, np.int16)
    got = gpu_backward(lib, g, A, B, la, lb)
    check_backward(oracle, got, g, A, B, la, lb, 8)
    if L:
        gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(la), dev(lb)
        gat = torch.full((M * K,), float("nan"), device="cuda")
        need = lib.amr_lut_gemm_backward_workspace_bytes(M, K, N)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
        rc = lib.amr_lut_gemm_backward_ex(gd.data_ptr(), a.data_ptr(), b.data_ptr(), gat.data_ptr(), None, ta.data_ptr(), tb.data_ptr(),
                                          ta.numel(), M, K, N, L, ws.data_ptr(), need, None)
        assert rc == 0, lib.amr_last_error()
        torch.cuda.synchronize()
        assert np.array_equal(gat.cpu().numpy().reshape(M // L, K, L).transpose(0, 2, 1).reshape(M, K), got[0])


def test_backward_large_m_masked_codes(lib, oracle):
    print("backward large M masked", flush=True)
    M, K, N = 4300, 40, 70
    rng, A, B, _ = rand_case(123, M, K, N, 7)
    la = oracle.pack_table(rng.integers(-3000, 3000, (128, 128)), 7, np.int16)
    lb = oracle.pack_table(rng.integers(-3000, 3000, (128, 128)), 7, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    A2, B2 = A.copy(), B.copy()
    A2[::5, 7] = 128
    A2[4000, :] = 128
    B2[3, ::2] = 128
    check_backward(oracle, gpu_backward(lib, g, A2, B2, la, lb), g, A2, B2, la, lb, 7)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, 7)


@pytest.mark.parametrize("kind", ["i16", "f32"])
def test_backward_masked_code_fallback_keeps_the_digits_of_a_long_sum(lib, oracle, kind):
    """A masked code sends the whole result to the direct kernels queued behind the expanded-table ones, where one wave adds
    all rows of a k tile.  It adds them in blocks (block sums into a second accumulator), so the result stays within 3e-6 of
    the float64 one norm-wise; one running sum over 32768 rows comes to 1e-5 on gradients with a non-zero mean."""
    print("masked-code fallback at 32768 rows", kind, flush=True)
    M, K, N = 32768, 128, 64
    rng, A, B, _ = rand_case(seed_of("mask", kind), M, K, N, 7)
    A[-1, :] = 128
    A[::7, 3] = 128
    Ga, Gb = rng.integers(-1024, 3073, (128, 128)), rng.integers(-1024, 3073, (128, 128))
    g = (rng.standard_normal((M, N)) + 0.25).astype(np.float32)
    if kind == "i16":
        la, lb = oracle.pack_table(Ga, 7, np.int16), oracle.pack_table(Gb, 7, np.int16)
        got = gpu_backward(lib, g, A, B, la, lb)
    else:
        la, lb = oracle.pack_table(Ga, 7, np.float32), oracle.pack_table(Gb, 7, np.float32)
        got = gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0 / 16)
    check_backward(oracle, got, g, A, B, la, lb, 7)
    a64, b64 = oracle.backward_c_f64(g, A, B, la, lb, 7, factor=1.0 / 16)
    for x, r in ((got[0], a64), (got[1], b64)):
        assert np.abs(x - r).max() <= 3e-6 * np.abs(r).max()


# K % 8 == 0, N % 64 == 0, M % 128 == 0 and M >= 4096: gradB runs on the expanded table held as halves (entries - 1024)
# (N % 32 == 0, K % 16 == 0 and M >= 2048: gradA runs on its own expanded table, 16, 32 or 48 k per workgroup and one to
# six column tiles, also with a ragged last row block)
HALF_SLAB_SHAPES = [(4096, 8, 64), (4224, 24, 128), (8192, 64, 64), (16384, 16, 192), (8200, 48, 96), (9001, 64, 32),
                    (4100, 32, 64), (2148, 144, 160), (5000, 80, 128), (1024, 16, 64), (2048, 48, 128), (1280, 64, 192),
                    # enough tiles for 32 k per workgroup in gradA: whole row blocks; a ragged last one
                    (32768, 128, 64), (33011, 128, 32)]


@pytest.mark.parametrize("bits", [7, 6, 4])
@pytest.mark.parametrize("low", [-1024, -2048])
@pytest.mark.parametrize("shape", HALF_SLAB_SHAPES)
def test_backward_half_slab_tables_inside_the_exact_range(lib, oracle, bits, shape, low):
    print("backward half slab", bits, shape, low, flush=True)
    rng, A, B, _ = rand_case(seed_of(bits, shape, "h"), *shape, bits)
    n = 1 << bits
    # [-1024, 3072]: halves of the entries - 1024; [-2048, 2048]: gradA holds the entries themselves
    Ga, Gb = rng.integers(low, low + 4097, (n, n)), rng.integers(-1024, 3073, (n, n))
    Ga[0, 0], Ga[1, 1], Ga[2, 2], Ga[3, 3] = low, low + 4096, low + 4094, low + 2
    Gb[0, 0], Gb[1, 1], Gb[2, 2], Gb[3, 3] = -1024, 3072, 3070, -1022     # ends of the range; even values beyond +-2048
    la, lb = oracle.pack_table(Ga, bits, np.int16), oracle.pack_table(Gb, bits, np.int16)
    g = (rng.standard_normal((shape[0], shape[2])) + 0.25).astype(np.float32)      # non-zero column sums
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, bits)
    if bits == 7:   # masked codes in both operands: the gated direct kernel takes over
        A2, B2 = A.copy(), B.copy()
        A2[::7, 3] = 128
        A2[-1, :] = 128
        B2[5, ::3] = 128
        check_backward(oracle, gpu_backward(lib, g, A2, B2, la, lb), g, A2, B2, la, lb, bits)


@pytest.mark.parametrize("bits", [7, 6])
def test_backward_half_slab_entry_a_half_cannot_hold(lib, oracle, bits):
    print("backward half slab inexact entry", bits, flush=True)
    M, K, N = 4096, 16, 64
    rng, A, B, _ = rand_case(77 + bits, M, K, N, bits)
    n = 1 << bits
    Ga, Gb = rng.integers(0, 2033, (n, n)), rng.integers(0, 2033, (n, n))
    Gb[5, 9] = 3075            # 3075 - 1024 = 2051 is not a half
    A[100, 3], B[3, 20] = 5, 9  # ... and it is used
    la, lb = oracle.pack_table(Ga, bits, np.int16), oracle.pack_table(Gb, bits, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    g[100, 20] = 1000.0        # make the one product matter
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, bits)
    Gb[5, 9] = -20000
    lb = oracle.pack_table(Gb, bits, np.int16)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, bits)


@pytest.mark.parametrize("shape", [(4096, 64, 64), (8192, 576, 64), (4224, 32, 128)])
@pytest.mark.parametrize("small,big", [((0, 17), 3000), ((0, 17), -3000), ((900, 1101), 3000), ((-40, 41), 2300), ((-40, 41), 6000)])
def test_backward_half_tables_whose_offset_would_swamp_small_entries(lib, oracle, shape, small, big):
    """Tables that do not fit a half as they are (one entry beyond +-2048) while most entries are small next to the offset
    that would make them fit: sum g * (entry - offset) + offset * sum g would then be a small number computed as the
    difference of two large ones.  The per-element bar (error relative to the sum of the true term magnitudes) holds
    for every output, for both gradients, whether the library stores such a table with an offset or steps aside."""
    print("backward, offset against small entries", shape, small, big, flush=True)
    M, K, N = shape
    rng, A, B, _ = rand_case(seed_of(shape, small, big), M, K, N, 7)
    Ga, Gb = rng.integers(small[0], small[1], (128, 128)), rng.integers(small[0], small[1], (128, 128))
    Ga[77, 13] = big
    Gb[13, 77] = big
    A[5, 3], B[3, 9] = 77, 13      # both entries are used once at least
    A[6, 4], B[4, 10] = 13, 77
    la, lb = oracle.pack_table(Ga, 7, np.int16), oracle.pack_table(Gb, 7, np.int16)
    g = (rng.standard_normal((M, N)) + 0.5).astype(np.float32)        # row and column sums of gC well away from zero
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, 7)


@pytest.mark.parametrize("shape", [(4096, 64, 64), (33011, 128, 32), (4100, 32, 64)])
def test_backward_ga_aligned_to_four_bytes_only(lib, oracle, shape):
    """gA one, two and three floats into a 16-byte-aligned allocation: the expanded-table kernel stores 16 bytes at a time
    where it can and must not where it cannot."""
    print("backward, gA not 16-byte aligned", shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(shape, "u"), *shape, 7)
    la = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), 7, np.int16)
    lb = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), 7, np.int16)
    g = rng.standard_normal((shape[0], shape[2])).astype(np.float32)
    want = gpu_backward(lib, g, A, B, la, lb)
    check_backward(oracle, want, g, A, B, la, lb, 7)
    for off in (1, 2, 3):
        got = gpu_backward(lib, g, A, B, la, lb, ga_offset_floats=off)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


def test_backward_config2_difference_tables_and_ste(lib, oracle):
    print("backward config2", flush=True)
    A, B, T, g = oracle.synth_gemm(4096, 576, 64, bits=7, err=64, seed=0)
    Gx, Gy = oracle.gen_bp_lut(T, 8)
    la, lb = oracle.pack_table(Gx, 7, np.int16), oracle.pack_table(Gy, 7, np.int16)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, 7)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb, own_workspace=False), g, A, B, la, lb, 7)
    # STE tables + small integer gC: every partial sum is exact in fp32 -> bit-exact dense matmuls
    Sx, Sy = oracle.ste_tables16(7)
    gi = np.random.default_rng(1).integers(-4, 5, g.shape).astype(np.float32)
    gA, gB = gpu_backward(lib, gi, A, B, oracle.pack_table(Sx, 7, np.int16), oracle.pack_table(Sy, 7, np.int16))
    assert (gA == gi.astype(np.int64) @ B.astype(np.int64).T).all()
    assert (gB == A.astype(np.int64).T @ gi.astype(np.int64)).all()


def test_backward_golden_shipped_tables(lib, oracle, golden_dir):
    print("backward golden", flush=True)
    _, ga, gb = oracle.parse_lut_file(os.path.join(golden_dir, "lut7_evo_081_bp16.txt.gz"), 7)
    rng, A, B, _ = rand_case(8, 500, 144, 128, 7)
    g = rng.standard_normal((500, 128)).astype(np.float32)
    la, lb = oracle.pack_table(ga, 7, np.int16), oracle.pack_table(gb, 7, np.int16)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, 7)
    z = np.load(os.path.join(golden_dir, "lut8_resub_183.npz"))
    rng, A, B, _ = rand_case(9, 300, 100, 70, 8)
    g = rng.standard_normal((300, 70)).astype(np.float32)
    la, lb = oracle.pack_table(z["grad_a"], 8, np.int16), oracle.pack_table(z["grad_b"], 8, np.int16)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, 8)


# ------------------------------------------------------------------------------------------ float32 gradient tables
def gpu_backward_f32tab(lib, g, A, B, la, lb, scale, own_workspace=True, rows_per_image=0):
    M, K = A.shape
    N = B.shape[1]
    gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(np.asarray(la, np.float32)), dev(np.asarray(lb, np.float32))
    ga = torch.full((M, K), float("nan"), device="cuda")
    gb = torch.full((K, N), float("nan"), device="cuda")
    need = lib.amr_lut_gemm_backward_f32tab_workspace_bytes(M, K, N)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda") if own_workspace else None
    rc = lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                          tb.data_ptr(), ta.numel(), scale, M, K, N, rows_per_image,
                                          ws.data_ptr() if ws is not None else None, need if ws is not None else 0, None)
    assert rc == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    return ga.cpu().numpy(), gb.cpu().numpy()


# small and ragged shapes (direct kernels), K below one workgroup's share (idle waves at the band barriers), and
# M >= 1024 (gradB on the fp32 expanded table for tables of at most 7 bits)
# (N % 16 == 0, K % 16 == 0 and M >= 512: gradA on the float32 expanded table, 16 or 32 k per tile, one to ten column tiles, also
# with a ragged last row block)
F32TAB_SHAPES = [(1, 1, 1), (3, 5, 7), (9, 27, 10), (64, 64, 64), (33, 130, 65), (600, 96, 64), (257, 100, 129), (300, 288, 256),
                 (70, 50, 513), (1100, 27, 64), (4096, 8, 64), (4100, 27, 10), (5000, 130, 65), (2048, 48, 128), (1500, 40, 70),
                 (1024, 16, 16), (5000, 80, 48), (4096, 64, 32), (9001, 64, 16), (2148, 144, 160), (16384, 32, 64), (8192, 576, 64),
                 (33011, 128, 32)]


# 8-bit float32 tables, M % 256 == 0, M >= 1024 (forced; 2048 by itself), K % 4 == 0, N % 64 == 0: gradB on the expanded float32
# table (two k per workgroup; one to three column tiles, one and several M splits)
SLAB8F_SHAPES = [(2048, 4, 64), (4096, 64, 128), (8192, 36, 192), (2304, 12, 64), (1024, 16, 128), (16384, 576, 64), (32768, 20, 64)]


@pytest.mark.parametrize("shape", SLAB8F_SHAPES)
def test_backward_8bit_float_table_slab(lib, oracle, shape):
    print("backward 8-bit float32 slab", shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(shape, "s8f"), *shape, 8)
    A[0, :] = 255                                                       # the last code of both operands occurs
    B[:, 0] = 255
    Ga, Gb = rng.standard_normal((256, 256)) * 40 + 3, rng.standard_normal((256, 256)) * 40 - 5
    Gb[255, 255], Gb[0, 0], Gb[255, 0], Gb[0, 255] = -1234.5, 4321.25, 0.125, -0.375
    la, lb = oracle.pack_table(Ga, 8, np.float32), oracle.pack_table(Gb, 8, np.float32)
    g = (rng.standard_normal((shape[0], shape[2])) + 0.25).astype(np.float32)
    got = gpu_backward_f32tab(lib, g, A, B, la, lb, 0.5)
    check_backward(oracle, got, g, A, B, la, lb, 8, factor=np.float32(0.5))
    old = lib.amr_set_expanded_table_kernels(0)                          # the direct kernels: same sums in another order
    try:
        ref = gpu_backward_f32tab(lib, g, A, B, la, lb, 0.5)
    finally:
        lib.amr_set_expanded_table_kernels(old)
    assert np.abs(got[1] - ref[1]).max() <= 1e-5 * np.abs(ref[1]).max()
    # image-major gA (1024 to 8191 rows: gradA with the table expanded in LDS and a kernel of its own that writes gA)
    M, K, N = shape
    L = 256
    gat = gpu_backward_f32tab(lib, g, A, B, la, lb, 0.5, rows_per_image=L)[0]
    assert np.array_equal(gat.reshape(M // L, K, L).transpose(0, 2, 1).reshape(M, K), got[0])


@pytest.mark.parametrize("bits", [7, 8, 6, 4])
@pytest.mark.parametrize("shape", F32TAB_SHAPES)
def test_backward_float_tables_within_tolerance(lib, oracle, bits, shape):
    print("backward float tables", bits, shape, flush=True)
    rng, A, B, _ = rand_case(seed_of(bits, shape, "f"), *shape, bits)
    n = 1 << bits
    la = oracle.pack_table(rng.standard_normal((n, n)) * 40 + 3, bits, np.float32)
    lb = oracle.pack_table(rng.standard_normal((n, n)) * 40 - 5, bits, np.float32)
    g = rng.standard_normal((shape[0], shape[2])).astype(np.float32)
    scale = 0.37
    check_backward(oracle, gpu_backward_f32tab(lib, g, A, B, la, lb, scale), g, A, B, la, lb, bits, factor=np.float32(scale))


@pytest.mark.parametrize("bits", [7, 8])
def test_backward_float_tables_masked_codes_and_both_bands(lib, oracle, bits):
    print("backward float tables, masked codes", bits, flush=True)
    n = 1 << bits
    M, K, N = 4300, 40, 70
    rng, A, B, _ = rand_case(500 + bits, M, K, N, bits)
    la = oracle.pack_table(rng.standard_normal((n, n)) * 10, bits, np.float32)
    lb = oracle.pack_table(rng.standard_normal((n, n)) * 10, bits, np.float32)
    g = rng.standard_normal((M, N)).astype(np.float32)
    if bits < 8:           # masked code 2^b: zero contribution (the pad row / column of the table); a uint8 cannot hold 256
        A[::5, 7] = n
        A[4000, :] = n
        B[3, ::2] = n
    else:                  # an 8-bit float table is staged in two bands of 129 rows: 128 is the last of the first band
        A[::5, 7], A[4000, :], B[3, ::2] = 128, 129, 128
        B[:, 5], B[:, 6] = 129, 128
    A[17, :] = n - 1
    A[18, :] = 0
    check_backward(oracle, gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0), g, A, B, la, lb, bits, factor=1.0)
    check_backward(oracle, gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0, own_workspace=False), g, A, B, la, lb, bits, factor=1.0)


@pytest.mark.parametrize("bits,shape", [(7, (700, 96, 64)), (8, (300, 40, 48)), (7, (4224, 32, 64)), (6, (129, 17, 33))])
def test_backward_float_tables_pointers_aligned_to_four_bytes_only(lib, oracle, bits, shape):
    """Tables, gC, gA and gB at addresses that are multiples of 4 but not of 16: no 128-bit access may be assumed."""
    print("backward float tables, 4-byte aligned pointers", bits, shape, flush=True)
    M, K, N = shape
    n = 1 << bits
    rng, A, B, _ = rand_case(800 + bits + M, M, K, N, bits)
    la = oracle.pack_table(rng.standard_normal((n, n)) * 7, bits, np.float32)
    lb = oracle.pack_table(rng.standard_normal((n, n)) * 7, bits, np.float32)
    g = rng.standard_normal((M, N)).astype(np.float32)

    def shifted(x, fill=None):
        t = torch.empty(x.size + 1, dtype=torch.float32, device="cuda")
        v = t[1:]
        if fill is None:
            v.copy_(torch.from_numpy(np.ascontiguousarray(x).ravel()))
        else:
            v.fill_(fill)
        assert v.data_ptr() % 16 == 4
        return t, v
    keep = []
    ptr = {}
    for name, arr, fill in (("g", g, None), ("ta", la, None), ("tb", lb, None), ("ga", np.empty((M, K), np.float32), float("nan")),
                            ("gb", np.empty((K, N), np.float32), float("nan"))):
        t, v = shifted(arr, fill)
        keep.append(t)
        ptr[name] = v
    a, b = dev(A), dev(B)
    rc = lib.amr_lut_gemm_backward_f32tab(ptr["g"].data_ptr(), a.data_ptr(), b.data_ptr(), ptr["ga"].data_ptr(), ptr["gb"].data_ptr(),
                                          ptr["ta"].data_ptr(), ptr["tb"].data_ptr(), la.size, 0.5, M, K, N, 0, None, 0, None)
    assert rc == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    got = (ptr["ga"].cpu().numpy().reshape(M, K), ptr["gb"].cpu().numpy().reshape(K, N))
    check_backward(oracle, got, g, A, B, la, lb, bits, factor=0.5)


@pytest.mark.parametrize("bits,shape", [(7, (700, 96, 64)), (8, (300, 40, 48)), (7, (4224, 32, 64)), (6, (1290, 17, 33))])
def test_backward_int16_tables_pointers_aligned_to_four_bytes_only(lib, oracle, bits, shape):
    print("backward, 4-byte aligned pointers", bits, shape, flush=True)
    M, K, N = shape
    n = 1 << bits
    rng, A, B, _ = rand_case(900 + bits + M, M, K, N, bits)
    la = oracle.pack_table(rng.integers(-2000, 2000, (n, n)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(-2000, 2000, (n, n)), bits, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    tg = torch.empty(g.size + 1, device="cuda"); vg = tg[1:]; vg.copy_(torch.from_numpy(g.ravel()))
    tga = torch.full((M * K + 1,), float("nan"), device="cuda"); vga = tga[1:]
    tgb = torch.full((K * N + 1,), float("nan"), device="cuda"); vgb = tgb[1:]
    tta = torch.empty(la.size + 2, dtype=torch.int16, device="cuda"); vta = tta[2:]; vta.copy_(torch.from_numpy(la))
    ttb = torch.empty(lb.size + 2, dtype=torch.int16, device="cuda"); vtb = ttb[2:]; vtb.copy_(torch.from_numpy(lb))
    assert vg.data_ptr() % 16 == 4 and vta.data_ptr() % 16 == 4
    a, b = dev(A), dev(B)
    rc = lib.amr_lut_gemm_backward(vg.data_ptr(), a.data_ptr(), b.data_ptr(), vga.data_ptr(), vgb.data_ptr(), vta.data_ptr(),
                                   vtb.data_ptr(), la.size, M, K, N, None, 0, None)
    assert rc == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    check_backward(oracle, (vga.cpu().numpy().reshape(M, K), vgb.cpu().numpy().reshape(K, N)), g, A, B, la, lb, bits)


@pytest.mark.parametrize("bits,shape", [(7, (3000, 64, 64)), (8, (3000, 64, 64)), (7, (300, 200, 40))])
def test_backward_float_tables_deterministic_and_skippable_outputs(lib, oracle, bits, shape):
    print("backward float tables, determinism", bits, shape, flush=True)
    M, K, N = shape
    n = 1 << bits
    rng, A, B, _ = rand_case(1000 + bits + M, M, K, N, bits)
    la = oracle.pack_table(rng.standard_normal((n, n)) * 30, bits, np.float32)
    g = rng.standard_normal((M, N)).astype(np.float32)
    r1 = gpu_backward_f32tab(lib, g, A, B, la, la, 0.25)
    r2 = gpu_backward_f32tab(lib, g, A, B, la, la, 0.25)
    assert (r1[0] == r2[0]).all() and (r1[1] == r2[1]).all()
    gd, a, b, t = dev(g), dev(A), dev(B), dev(la)
    gb = torch.zeros(K, N, device="cuda")
    ga = torch.zeros(M, K, device="cuda")
    assert lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), None, gb.data_ptr(), None, t.data_ptr(),
                                            t.numel(), 0.25, M, K, N, 0, None, 0, None) == 0
    assert lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), None, t.data_ptr(), None,
                                            t.numel(), 0.25, M, K, N, 0, None, 0, None) == 0
    torch.cuda.synchronize()
    assert (gb.cpu().numpy() == r1[1]).all() and (ga.cpu().numpy() == r1[0]).all()


def test_backward_float_tables_expanded_gradA_masked_codes(lib, oracle):
    print("backward float tables, expanded gradA with masked codes", flush=True)
    M, K, N = 4224, 32, 64
    rng, A, B, _ = rand_case(700, M, K, N, 7)
    la = oracle.pack_table(rng.standard_normal((128, 128)) * 10, 7, np.float32)
    lb = oracle.pack_table(rng.standard_normal((128, 128)) * 10, 7, np.float32)
    g = rng.standard_normal((M, N)).astype(np.float32)
    # (queried by shape alone the int16 scratch is sized for an 8-bit table as well, whose expanded table is as large as
    # the float32 one of a 7-bit table; with the table's size given it is half of that)
    assert lib.amr_lut_gemm_backward_f32tab_workspace_bytes(M, K, N) >= lib.amr_lut_gemm_backward_workspace_bytes(M, K, N) > 0
    assert lib.amr_lut_gemm_backward_f32tab_workspace_bytes(M, K, N) > lib.amr_lut_gemm_backward_workspace_bytes_for(129 * 130 + 638, M, K, N) > 0
    check_backward(oracle, gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0), g, A, B, la, lb, 7, factor=1.0)
    A2, B2 = A.copy(), B.copy()
    A2[::7, 3] = 128
    A2[-1, :] = 128
    B2[5, ::3] = 128
    check_backward(oracle, gpu_backward_f32tab(lib, g, A2, B2, la, lb, 1.0), g, A2, B2, la, lb, 7, factor=1.0)
    check_backward(oracle, gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0), g, A, B, la, lb, 7, factor=1.0)     # clean again
    # image-major gA from the expanded-table kernel equals the row-major one
    L = 64
    gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(la), dev(lb)
    gat = torch.full((M // L, K, L), float("nan"), device="cuda")
    assert lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), gat.data_ptr(), None, ta.data_ptr(), tb.data_ptr(),
                                            ta.numel(), 1.0, M, K, N, L, None, 0, None) == 0
    torch.cuda.synchronize()
    assert (gat.cpu().numpy().transpose(0, 2, 1).reshape(M, K) == gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0)[0]).all()


@pytest.mark.parametrize("bits", [7, 8])
def test_backward_float_tables_ste_is_the_dense_product_and_int16_values_agree(lib, oracle, bits):
    print("backward float tables, STE / int16 values", bits, flush=True)
    n = 1 << bits
    M, K, N = 1300, 72, 96
    rng, A, B, _ = rand_case(600 + bits, M, K, N, bits)
    # Gx[a][b] = b, Gy[a][b] = a, scale 1, small integer gC: every partial sum is exact -> the dense products, bit for bit
    Sx = np.broadcast_to(np.arange(n, dtype=np.float32)[None, :], (n, n))
    Sy = np.broadcast_to(np.arange(n, dtype=np.float32)[:, None], (n, n))
    gi = rng.integers(-4, 5, (M, N)).astype(np.float32)
    gA, gB = gpu_backward_f32tab(lib, gi, A, B, oracle.pack_table(Sx, bits, np.float32), oracle.pack_table(Sy, bits, np.float32), 1.0)
    assert (gA == gi.astype(np.int64) @ B.astype(np.int64).T).all()
    assert (gB == A.astype(np.int64).T @ gi.astype(np.int64)).all()
    # a float table holding int16 values with scale 1/16 is the reference's backward pass
    Ga, Gb = rng.integers(-32768, 32768, (n, n)), rng.integers(-32768, 32768, (n, n))
    g = rng.standard_normal((M, N)).astype(np.float32)
    la16, lb16 = oracle.pack_table(Ga, bits, np.int16), oracle.pack_table(Gb, bits, np.int16)
    got = gpu_backward_f32tab(lib, g, A, B, la16.astype(np.float32), lb16.astype(np.float32), 1.0 / 16)
    check_backward(oracle, got, g, A, B, la16, lb16, bits)
    ref = gpu_backward(lib, g, A, B, la16, lb16)
    for x, r in zip(got, ref):
        assert np.max(np.abs(x - r)) <= 2e-5 * np.max(np.abs(r))


def test_backward_float_tables_unrounded_difference_slopes_and_image_major_layout(lib, oracle):
    """The GEMM of BASELINE configs[1] with the float32 difference slopes (half window 8) before their x16 rounding."""
    print("backward float tables, config2 slopes", flush=True)
    A, B, T, g = oracle.synth_gemm(4096, 576, 64, bits=7, err=64, seed=0)
    Gx, Gy = oracle.gen_bp_lut(T, 8, rounded=False)
    assert Gx.dtype == np.float32 and not (Gx * 16 == np.round(Gx * 16)).all()      # really unrounded
    la, lb = oracle.pack_table(Gx, 7, np.float32), oracle.pack_table(Gy, 7, np.float32)
    gA, gB = gpu_backward_f32tab(lib, g, A, B, la, lb, 1.0)
    check_backward(oracle, (gA, gB), g, A, B, la, lb, 7, factor=1.0)
    # image-major gA (the layout col2im takes): [M/L][K][L]
    L = 1024
    M, K = A.shape
    gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(la), dev(lb)
    gat = torch.full((M // L, K, L), float("nan"), device="cuda")
    assert lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), gat.data_ptr(), None, ta.data_ptr(), tb.data_ptr(),
                                            ta.numel(), 1.0, M, K, 64, L, None, 0, None) == 0
    torch.cuda.synchronize()
    assert (gat.cpu().numpy().transpose(0, 2, 1).reshape(M, K) == gA).all()
    # argument checks
    assert lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), gat.data_ptr(), None, ta.data_ptr(), tb.data_ptr(),
                                            ta.numel() - 1, 1.0, M, K, 64, L, None, 0, None) != 0
    assert lib.amr_lut_gemm_backward_f32tab(gd.data_ptr(), a.data_ptr(), b.data_ptr(), gat.data_ptr(), None, ta.data_ptr(), tb.data_ptr(),
                                            ta.numel(), 1.0, M, K, 64, 1000, None, 0, None) != 0


def test_backward_deterministic_and_skippable_outputs(lib, oracle):
    print("backward determinism", flush=True)
    rng, A, B, _ = rand_case(10, 3000, 64, 64, 7)
    la = oracle.pack_table(rng.integers(-3000, 3000, (128, 128)), 7, np.int16)
    g = rng.standard_normal((3000, 64)).astype(np.float32)
    r1 = gpu_backward(lib, g, A, B, la, la)
    r2 = gpu_backward(lib, g, A, B, la, la)
    assert (r1[0] == r2[0]).all() and (r1[1] == r2[1]).all()
    gd, a, b, t = dev(g), dev(A), dev(B), dev(la)
    gb = torch.zeros(64, 64, device="cuda")
    assert lib.amr_lut_gemm_backward(gd.data_ptr(), a.data_ptr(), b.data_ptr(), None, gb.data_ptr(), None, t.data_ptr(),
                                     t.numel(), 3000, 64, 64, None, 0, None) == 0
    torch.cuda.synchronize()
    assert (gb.cpu().numpy() == r1[1]).all()


@pytest.mark.parametrize("shape", [(2048, 512, 64), (4096, 640, 300), (8200, 48, 96), (5000, 130, 65)])
def test_direct_kernels_at_large_m(lib, oracle, shape):
    """Mode 0: the direct gather kernels on shapes that otherwise take the expanded-table kernels."""
    print("direct kernels, large M", shape, flush=True)
    M, K, N = shape
    rng, A, B, T = rand_case(seed_of(shape, "d"), M, K, N, 7)
    flat = oracle.pack_table(T, 7, np.uint16)
    la = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), 7, np.int16)
    lb = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), 7, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    assert lib.amr_set_expanded_table_kernels(0) == 2
    try:
        assert lib.amr_lut_gemm_forward_workspace_bytes(flat.size, M, K, N) == 0
        c0 = gpu_forward(lib, A, B, flat)
        r0 = gpu_backward(lib, g, A, B, la, lb)
    finally:
        lib.amr_set_expanded_table_kernels(2)
    assert (c0 == oracle.forward_c(A, B, flat, 7)).all()
    check_backward(oracle, r0, g, A, B, la, lb, 7)
    assert (gpu_forward(lib, A, B, flat) == c0).all()            # expanded-table kernels: same bits


def test_operands_beyond_2_31_elements(lib, oracle):
    """M * K just above 2^31 (2 GiB of codes, 8 GiB of gA): the kernels that take 32-bit offsets step aside and the rows whose
    offsets need more than 32 bits come out right.  Forward and gA are checked against the oracle on row samples (first rows,
    middle, and the rows beyond offset 2^31); gB, a sum over all rows, against the sum of the two halves of the rows computed
    by launches whose offsets fit 32 bits, within the tolerance measured against the sum of term magnitudes (the same
    launch on |gC| and |table|)."""
    print("M*K > 2^31", flush=True)
    M, K, N, bits = 4194432, 512, 20, 7
    assert M * K > 2**31 and M % 2 == 0
    rng = np.random.default_rng(77)
    gen = torch.Generator(device="cuda").manual_seed(77)
    a = torch.randint(0, 128, (M, K), dtype=torch.uint8, device="cuda", generator=gen)
    B = rng.integers(0, 128, (K, N)).astype(np.uint8)
    T = rng.integers(0, 65536, (128, 128))
    flat = oracle.pack_table(T, bits, np.uint16)
    la = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), bits, np.int16)
    gd = torch.randn((M, N), device="cuda", generator=gen)
    b, l, ta, tb = dev(B), dev(flat), dev(la), dev(lb)
    idx = np.concatenate([np.arange(64), np.arange(M // 2 - 32, M // 2 + 32), np.arange(M - 192, M)])
    assert (idx[-128:] * K >= 2**31).all()
    tidx = torch.from_numpy(idx).cuda()
    A_s, g_s = a[tidx].cpu().numpy(), gd[tidx].cpu().numpy()

    assert lib.amr_lut_gemm_forward_workspace_bytes(l.numel(), M, K, N) == 0
    c = torch.full((M, N), -1, dtype=torch.int32, device="cuda")
    assert lib.amr_lut_gemm_forward(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, None) == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    assert (c[tidx].cpu().numpy().view(np.uint32) == oracle.forward_c(A_s, B, flat, bits)).all()
    del c

    def backward(gc, codes, table_b, rows, want_a):
        ga = torch.full((rows, K), float("nan"), device="cuda") if want_a else None
        gb = torch.full((K, N), float("nan"), device="cuda")
        need = lib.amr_lut_gemm_backward_workspace_bytes(rows, K, N)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
        rc = lib.amr_lut_gemm_backward(gc.data_ptr(), codes.data_ptr(), b.data_ptr(), ga.data_ptr() if want_a else None, gb.data_ptr(),
                                       ta.data_ptr(), table_b.data_ptr(), ta.numel(), rows, K, N, ws.data_ptr(), need, None)
        assert rc == 0, lib.amr_last_error()
        torch.cuda.synchronize()
        return ga, gb

    ga, gb = backward(gd, a, tb, M, True)
    a64, _, absA, _ = oracle.backward_c_f64(g_s, A_s, B, la, lb, bits, want_abs=True)
    err = np.abs(ga[tidx].cpu().numpy() - a64)
    assert np.max(err / np.maximum(absA, 1e-30)) < TOL
    assert bool(torch.isfinite(ga).all())
    del ga
    h = M // 2
    _, gb0 = backward(gd[:h], a[:h], tb, h, False)
    _, gb1 = backward(gd[h:], a[h:], tb, h, False)
    _, gb_abs = backward(gd.abs(), a, dev(np.abs(lb)), M, False)
    err = (gb.double() - (gb0.double() + gb1.double())).abs()
    assert float((err / gb_abs.double().clamp_min(1e-30)).max()) < 2 * TOL
    assert bool(torch.isfinite(gb).all()) and float(gb_abs.min()) > 0


def test_row_counts_beyond_65535_row_blocks(lib, oracle):
    """More row blocks than a grid may have workgroups along y (65535): the direct kernels fold their tile grid into x."""
    print("row blocks > 65535", flush=True)
    # 64 rows per workgroup in the forward kernel for N > 128 and in the fp32 GEMM: 65538 row blocks
    M, K, N = 4194432, 8, 130
    rng, A, B, T = rand_case(31, M, K, N, 7)
    flat = oracle.pack_table(T, 7, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == oracle.forward_c(A, B, flat, 7)).all()
    a, b = dev(A.astype(np.float32)), dev(B.astype(np.float32))
    c = torch.full((M, N), float("nan"), device="cuda")
    assert lib.amr_acc_gemm_forward_fp32(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, K, N, None) == 0, lib.amr_last_error()
    torch.cuda.synchronize()
    assert torch.equal(c.cpu(), torch.from_numpy(A.astype(np.float32) @ B.astype(np.float32)))     # small integers: exact
    del a, b, c
    # 512 rows per workgroup in the direct gradA kernel, 128 in the forward kernel for N <= 64: 65537 and 262145 row blocks
    M, K, N = 33554496, 3, 2
    rng, A, B, T = rand_case(32, M, K, N, 7)
    flat = oracle.pack_table(T, 7, np.uint16)
    assert (gpu_forward(lib, A, B, flat) == oracle.forward_c(A, B, flat, 7)).all()
    la = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), 7, np.int16)
    lb = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), 7, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    check_backward(oracle, gpu_backward(lib, g, A, B, la, lb), g, A, B, la, lb, 7)


def _seeded_case(seed):
    """A pseudo-random problem: bit width, shape (half of them with the divisibilities the expanded-table kernels want),
    table value range and kernel-selection mode all drawn from the seed."""
    rng = np.random.default_rng(1000 + seed)
    bits = int(rng.choice([7, 7, 7, 8, 6, 4]))
    M = int(np.exp(rng.uniform(0, np.log(7000))))
    K = int(np.exp(rng.uniform(0, np.log(1400))))
    N = int(np.exp(rng.uniform(0, np.log(320))))
    if rng.random() < 0.5:
        M, K, N = max(1024, M // 128 * 128 + int(rng.choice([0, 0, 5]))), max(16, K // 16 * 16), max(32, N // 32 * 32)
    lo, hi = [(-2048, 2049), (-1024, 3073), (-32768, 32768), (0, 4081)][int(rng.integers(0, 4))]
    mode = int(rng.choice([1, 2, 2]))
    return rng, bits, max(M, 1), max(K, 1), max(N, 1), lo, hi, mode


@pytest.mark.parametrize("seed", range(48))
def test_seeded_random_problems(lib, oracle, seed):
    """Forward bit-exact and both backward entry points within tolerance on 48 problems drawn from seeds."""
    rng, bits, M, K, N, lo, hi, mode = _seeded_case(seed)
    print("seeded problem", seed, bits, (M, K, N), (lo, hi), "mode", mode, flush=True)
    n = 1 << bits
    A = rng.integers(0, n, (M, K)).astype(np.uint8)
    B = rng.integers(0, n, (K, N)).astype(np.uint8)
    if bits < 8 and seed % 5 == 0:                       # the masked code 2^b here and there
        A[rng.integers(0, M), rng.integers(0, K)] = n
        B[rng.integers(0, K), rng.integers(0, N)] = n
    flat = oracle.pack_table(rng.integers(0, 65536 if seed % 2 else 16384, (n, n)), bits, np.uint16)
    la = oracle.pack_table(rng.integers(lo, hi, (n, n)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(lo, hi, (n, n)), bits, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    assert lib.amr_set_expanded_table_kernels(mode) == 2
    try:
        c = gpu_forward(lib, A, B, flat)
        r16 = gpu_backward(lib, g, A, B, la, lb)
        fa, fb = (la.astype(np.float32) * np.float32(0.37)), (lb.astype(np.float32) * np.float32(-1.3))
        r32 = gpu_backward_f32tab(lib, g, A, B, fa, fb, 0.5)
    finally:
        lib.amr_set_expanded_table_kernels(2)
    assert (c == oracle.forward_c(A, B, flat, bits)).all()
    check_backward(oracle, r16, g, A, B, la, lb, bits)
    check_backward(oracle, r32, g, A, B, fa, fb, bits, factor=0.5)


def test_default_mode_picks_kernels_by_problem_size(lib, oracle):
    print("kernel selection by size", flush=True)
    assert lib.amr_set_expanded_table_kernels(1) == 2
    try:
        # configs[1]-sized GEMM: too small for the expanded forward table to pay; a conv2_x-sized one is not
        assert lib.amr_lut_gemm_forward_workspace_bytes(17408, 4096, 576, 64) == 0
        assert lib.amr_lut_gemm_forward_workspace_bytes(17408, 262144, 576, 64) == 256 + 2 * 144 * 32768
        rng, A, B, T = rand_case(5, 4096, 576, 64, 7)
        flat = oracle.pack_table(T, 7, np.uint16)
        assert (gpu_forward(lib, A, B, flat) == oracle.forward_c(A, B, flat, 7)).all()
    finally:
        lib.amr_set_expanded_table_kernels(2)


@pytest.mark.parametrize("bits", [7, 8])
def test_calls_can_be_recorded_into_a_device_graph(lib, oracle, bits):
    """Forward and backward with caller-provided scratch, recorded once into a graph and replayed with new operand
    contents (with eager work and synchronisations in between): every replay equals the eager result."""
    print("graph capture", bits, flush=True)
    M, K, N = 4096, 576, 64
    rng, A, B, T = rand_case(31, M, K, N, bits)
    T = oracle.synth_lut(bits, 64, rng)
    flat = oracle.pack_table(T, bits, np.uint16)
    Gx, Gy = oracle.gen_bp_lut(T, 8)
    la, lb = oracle.pack_table(Gx, bits, np.int16), oracle.pack_table(Gy, bits, np.int16)
    a, b, l, ta, tb = dev(A), dev(B), dev(flat), dev(la), dev(lb)
    g = torch.randn(M, N, device="cuda")
    c = torch.zeros(M, N, dtype=torch.int32, device="cuda")
    ga, gb = torch.zeros(M, K, device="cuda"), torch.zeros(K, N, device="cuda")
    need_f = lib.amr_lut_gemm_forward_workspace_bytes(l.numel(), M, K, N)
    need_b = lib.amr_lut_gemm_backward_workspace_bytes(M, K, N)
    assert need_f > 0 and need_b > 0
    ws_f = torch.empty(need_f, dtype=torch.uint8, device="cuda")
    ws_b = torch.empty(need_b, dtype=torch.uint8, device="cuda")

    def run(stream):
        sp = ctypes.c_void_p(stream.cuda_stream)
        assert lib.amr_lut_gemm_forward_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N,
                                           ws_f.data_ptr(), need_f, sp) == 0, lib.amr_last_error()
        assert lib.amr_lut_gemm_backward(g.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                         tb.data_ptr(), ta.numel(), M, K, N, ws_b.data_ptr(), need_b, sp) == 0, lib.amr_last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(side)                                   # warm-up: one-time attribute calls happen outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(torch.cuda.current_stream())
    for rep in range(3):
        a.copy_(torch.randint(0, 1 << bits, (M, K), dtype=torch.uint8, device="cuda"))
        if rep == 1 and bits == 7:
            a[5, 7] = 128                           # a masked code: the gated fall-back kernels do the work in this replay
        g.copy_(torch.randn(M, N, device="cuda"))
        c.zero_(); ga.zero_(); gb.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = (c.clone(), ga.clone(), gb.clone())
        c.zero_(); ga.zero_(); gb.zero_()
        run(torch.cuda.current_stream())
        torch.cuda.synchronize()
        assert torch.equal(got[0], c) and torch.equal(got[1], ga) and torch.equal(got[2], gb), f"replay {rep} differs from the eager call"
        assert (c.cpu().numpy().view(np.uint32) == oracle.forward_c(a.cpu().numpy(), B, flat, bits)).all()


def test_two_host_threads_on_two_streams_equal_the_serial_results(lib, oracle):
    """Two host threads of one process call forward and backward at the same time, each on a stream of its own and without
    passing scratch (the library's own per-stream buffers): every result equals the one the same call gives alone."""
    import threading
    print("two threads, two streams", flush=True)
    problems = []
    for seed, (M, K, N), bits in ((41, (8192, 576, 64), 7), (42, (4096, 1152, 128), 8)):       # (one 7-bit and one 8-bit problem)
        rng, A, B, T = rand_case(seed, M, K, N, bits)
        T = oracle.synth_lut(bits, 64, rng)
        Gx, Gy = oracle.gen_bp_lut(T, 8)
        t = dict(M=M, K=K, N=N, a=dev(A), b=dev(B), l=dev(oracle.pack_table(T, bits, np.uint16)), ta=dev(oracle.pack_table(Gx, bits, np.int16)),
                 tb=dev(oracle.pack_table(Gy, bits, np.int16)), g=dev(rng.standard_normal((M, N)).astype(np.float32)),
                 c=torch.zeros((M, N), dtype=torch.int32, device="cuda"), ga=torch.zeros((M, K), device="cuda"),
                 gb=torch.zeros((K, N), device="cuda"), stream=torch.cuda.Stream())
        problems.append(t)

    def run(t, stream_ptr, reps):
        for _ in range(reps):
            rc = lib.amr_lut_gemm_forward(t["a"].data_ptr(), t["b"].data_ptr(), t["c"].data_ptr(), t["l"].data_ptr(), t["l"].numel(),
                                          t["M"], t["K"], t["N"], stream_ptr)
            assert rc == 0, lib.amr_last_error()
            rc = lib.amr_lut_gemm_backward(t["g"].data_ptr(), t["a"].data_ptr(), t["b"].data_ptr(), t["ga"].data_ptr(), t["gb"].data_ptr(),
                                           t["ta"].data_ptr(), t["tb"].data_ptr(), t["ta"].numel(), t["M"], t["K"], t["N"], None, 0, stream_ptr)
            assert rc == 0, lib.amr_last_error()

    serial = []
    for t in problems:                     # each problem alone, on the default stream
        run(t, None, 1)
        torch.cuda.synchronize()
        serial.append((t["c"].clone(), t["ga"].clone(), t["gb"].clone()))
        t["c"].zero_(); t["ga"].zero_(); t["gb"].zero_()
    torch.cuda.synchronize()
    errors = []

    def worker(t):
        try:
            run(t, ctypes.c_void_p(t["stream"].cuda_stream), 20)
        except BaseException as e:        # noqa: BLE001 -- handed to the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(t,)) for t in problems]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for t, (c, ga, gb) in zip(problems, serial):
        assert torch.equal(t["c"], c) and torch.equal(t["ga"], ga) and torch.equal(t["gb"], gb)


def test_accgemm_matches_torch(lib):
    print("accgemm", flush=True)
    torch.manual_seed(0)
    for (M, K, N) in [(1, 1, 1), (65, 33, 70), (256, 576, 64)]:
        a = torch.randint(-4, 5, (M, K), device="cuda").float()
        b = torch.randint(-4, 5, (K, N), device="cuda").float()
        c = torch.full((M, N), float("nan"), device="cuda")
        assert lib.amr_acc_gemm_forward_fp32(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, K, N, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(c, a @ b)


# ---------------------------------------------------------------- full-size, size-independent properties
def test_full_size_resnet_layer_properties(lib, oracle):
    """conv2_x at batch 256 (M=262144, K=576, N=64): too big for the CPU oracle in seconds, so check
    properties: exact-multiplier table == torch integer matmul; linearity in the table; row-subset
    agreement with the oracle; STE backward == dense matmul on integer gC."""
    print("full size", flush=True)
    M, K, N = 262144, 576, 64
    gen = torch.Generator(device="cuda").manual_seed(0)
    a = torch.randint(0, 128, (M, K), dtype=torch.uint8, device="cuda", generator=gen)
    b = torch.randint(0, 128, (K, N), dtype=torch.uint8, device="cuda", generator=gen)
    rng = np.random.default_rng(0)
    T1 = oracle.synth_lut(7, 64, rng)
    Tx = np.arange(128)[:, None] * np.arange(128)[None, :]

    def fwd(T):
        l = dev(oracle.pack_table(T, 7, np.uint16))
        c = torch.empty((M, N), dtype=torch.int32, device="cuda")
        assert lib.amr_lut_gemm_forward(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, None) == 0
        torch.cuda.synchronize()
        return c

    cx = fwd(Tx)
    want = (a.double() @ b.double()).to(torch.int32)          # < 2^53, exact
    assert torch.equal(cx, want)
    c1 = fwd(T1)
    assert torch.equal(fwd(T1 + Tx), c1 + cx)                  # linearity in the table
    rows = np.r_[0:64, 131000:131064, M - 64:M]
    sub = oracle.forward_c(a[rows].cpu().numpy(), b.cpu().numpy(), oracle.pack_table(T1, 7, np.uint16), 7)
    assert (c1[rows].cpu().numpy().view(np.uint32) == sub).all()
    # STE backward, integer gC in {-1,0,1}: sums are exact in fp32 (|gB| <= 262144*127 < 2^25 needs care -> use sparse gC)
    g = (torch.rand((M, N), device="cuda", generator=gen) < 0.05).float() * torch.randint(-1, 2, (M, N), device="cuda", generator=gen).float()
    Sx, Sy = oracle.ste_tables16(7)
    ta, tb = dev(oracle.pack_table(Sx, 7, np.int16)), dev(oracle.pack_table(Sy, 7, np.int16))
    ga = torch.empty((M, K), device="cuda")
    gb = torch.empty((K, N), device="cuda")
    assert lib.amr_lut_gemm_backward(g.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                     tb.data_ptr(), ta.numel(), M, K, N, None, 0, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(ga.double(), g.double() @ b.double().t())
    assert torch.equal(gb.double(), a.double().t() @ g.double())


# The GEMM shapes of the benchmark step (ResNet-18 / CIFAR at batch 256) and of the training-step configuration (batch 512:
# M doubled), in the library's own kernel selection.
RESNET18_B256_SHAPES = [(262144, 27, 64), (262144, 576, 64), (65536, 576, 128), (65536, 1152, 128), (65536, 64, 128),
                        (16384, 1152, 256), (16384, 2304, 256), (16384, 128, 256), (4096, 2304, 512), (4096, 4608, 512),
                        (4096, 256, 512), (256, 512, 10)]
RESNET18_B512_SHAPES = [(2 * M, K, N) for M, K, N in RESNET18_B256_SHAPES]
VGG16_B128_SHAPES = [(131072, 27, 64), (131072, 576, 64), (32768, 576, 128), (32768, 1152, 128), (8192, 1152, 256), (8192, 2304, 256),
                     (2048, 2304, 512), (2048, 4608, 512), (512, 4608, 512), (128, 512, 10)]


def check_full_size_layer(lib, oracle, kind, bits, shape):
    """One full-size layer with a gradient on EVERY row (gC ~ N(0,1)), in the library's own kernel selection.  Every output
    row of the forward pass and of gA depends on its own row of A / gC only: those are checked against the oracle on a
    sample of rows spread over all row blocks.  gB is a sum over all rows: the whole of it is checked against the oracle's
    row-streaming float64 sums, per element relative to the sum of term magnitudes and norm-wise.  gA must be finite
    everywhere."""
    M, K, N = shape
    n = 1 << bits
    gen = torch.Generator(device="cuda").manual_seed(M + K + N + bits)
    rng = np.random.default_rng(M + 3 * K + 7 * N + bits)
    T = oracle.synth_lut(bits, 64 if bits == 7 else 256, rng)
    hw = 8 if bits == 7 else 16
    if kind == "f32":
        Gx, Gy = oracle.gen_bp_lut(T, hw, rounded=False)
        la, lb, factor = oracle.pack_table(Gx, bits, np.float32), oracle.pack_table(Gy, bits, np.float32), 1.0
    else:
        Gx, Gy = oracle.gen_bp_lut(T, hw)
        la, lb, factor = oracle.pack_table(Gx, bits, np.int16), oracle.pack_table(Gy, bits, np.int16), 1.0 / 16
    flat = oracle.pack_table(T, bits, np.uint16)
    a = torch.randint(0, n, (M, K), dtype=torch.uint8, device="cuda", generator=gen)
    b = torch.randint(0, n, (K, N), dtype=torch.uint8, device="cuda", generator=gen)
    rows = np.unique(np.r_[0:96, np.arange(37, M, max(M // 1200, 1)), M // 2 - 70:M // 2 + 70, M - 96:M].clip(0, M - 1))
    rows_t = torch.from_numpy(rows).cuda()
    g = torch.randn((M, N), device="cuda", generator=gen)
    c = torch.empty((M, N), dtype=torch.int32, device="cuda")
    ga = torch.full((M, K), float("nan"), device="cuda")
    gb = torch.full((K, N), float("nan"), device="cuda")
    l, ta, tb = dev(flat), dev(la), dev(lb)
    assert lib.amr_set_expanded_table_kernels(1) == 2
    try:
        assert lib.amr_lut_gemm_forward(a.data_ptr(), b.data_ptr(), c.data_ptr(), l.data_ptr(), l.numel(), M, K, N, None) == 0
        if kind == "f32":
            rc = lib.amr_lut_gemm_backward_f32tab(g.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                                  tb.data_ptr(), ta.numel(), 1.0, M, K, N, 0, None, 0, None)
        else:
            rc = lib.amr_lut_gemm_backward(g.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                           tb.data_ptr(), ta.numel(), M, K, N, None, 0, None)
        assert rc == 0, lib.amr_last_error()
        torch.cuda.synchronize()
    finally:
        lib.amr_set_expanded_table_kernels(2)
    An, Bn, gn = a.cpu().numpy(), b.cpu().numpy(), g.cpu().numpy()
    As, gs = An[rows], gn[rows]
    assert (c[rows_t].cpu().numpy().view(np.uint32) == oracle.forward_c(As, Bn, flat, bits)).all()
    assert bool(torch.isfinite(ga).all())
    a64, _, absA, _ = oracle.backward_c_f64(gs, As, Bn, la, lb, bits, factor=factor, want_abs=True)
    err = np.abs(ga[rows_t].cpu().numpy() - a64)
    assert np.max(err / np.maximum(absA, 1e-30)) < TOL
    assert np.max(err) <= TOL * np.max(np.abs(a64))
    b64, absB = oracle.gradB_c_f64_rows(gn, An, Bn, lb, bits, factor=factor)
    err = np.abs(gb.cpu().numpy() - b64)
    assert np.max(err / np.maximum(absB, 1e-30)) < TOL
    assert np.max(err) <= TOL * np.max(np.abs(b64))


@pytest.mark.parametrize("shape", RESNET18_B256_SHAPES + RESNET18_B512_SHAPES)
def test_benchmark_shapes_dense_gradients_against_oracle(lib, oracle, shape):
    print("benchmark shape, dense gC", shape, flush=True)
    check_full_size_layer(lib, oracle, "i16", 7, shape)


@pytest.mark.parametrize("kind,bits,shape", [("f32", 7, s) for s in RESNET18_B256_SHAPES] + [("i16", 8, s) for s in VGG16_B128_SHAPES] +
                         [("f32", 8, s) for s in VGG16_B128_SHAPES])
def test_benchmark_shapes_other_table_formats_dense_gradients(lib, oracle, kind, bits, shape):
    """The same check for the other two workloads of the benchmark: float32 gradient tables on the ResNet-18 shapes (7 bit)
    and the VGG-16 shapes at batch 128 with 8-bit tables, int16 and float32 gradient tables (unrounded difference slopes,
    half window 8 / 16)."""
    print("benchmark shape, dense gC", kind, bits, shape, flush=True)
    check_full_size_layer(lib, oracle, kind, bits, shape)


def test_rows_without_gradient_give_exact_zeros(lib, oracle):
    """gC non-zero on a sample of rows only: every other row of gA is exactly zero (no cross-row leakage), conv2_x size."""
    print("rows without gradient", flush=True)
    M, K, N = 262144, 576, 64
    gen = torch.Generator(device="cuda").manual_seed(5)
    rng = np.random.default_rng(5)
    T = oracle.synth_lut(7, 64, rng)
    Gx, Gy = oracle.gen_bp_lut(T, 8)
    ta, tb = dev(oracle.pack_table(Gx, 7, np.int16)), dev(oracle.pack_table(Gy, 7, np.int16))
    a = torch.randint(0, 128, (M, K), dtype=torch.uint8, device="cuda", generator=gen)
    b = torch.randint(0, 128, (K, N), dtype=torch.uint8, device="cuda", generator=gen)
    rows_t = torch.from_numpy(np.unique(np.r_[0:96, np.arange(37, M, 170), M - 96:M])).cuda()
    g = torch.zeros((M, N), device="cuda")
    g[rows_t] = torch.randn((len(rows_t), N), device="cuda", generator=gen)
    ga = torch.full((M, K), float("nan"), device="cuda")
    gb = torch.full((K, N), float("nan"), device="cuda")
    assert lib.amr_set_expanded_table_kernels(1) == 2
    try:
        assert lib.amr_lut_gemm_backward(g.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                         tb.data_ptr(), ta.numel(), M, K, N, None, 0, None) == 0, lib.amr_last_error()
        torch.cuda.synchronize()
    finally:
        lib.amr_set_expanded_table_kernels(2)
    mask = torch.ones(M, dtype=torch.bool, device="cuda")
    mask[rows_t] = False
    assert (ga[mask] == 0).all()
    assert bool((ga[rows_t] != 0).any())
