"""Pins the CPU oracle (oracle/) before anything is compared against it.

Reference-held data: the look-up-table files under app_mults/ (committed copies in tests/golden/).
Closed forms: exact-multiplier table -> integer matmul; STE tables -> dense matmuls; masked code
2^b -> zero contribution; brute-force triple loops on tiny shapes; linearity in the table.
"""
import gzip
import json
import os

import numpy as np
import pytest


# ------------------------------------------------------------------------------- geometry / format
def test_geometry_lengths_quoted_by_reference(oracle):
    # approx_mult.h:17-19 (7-bit: 129*130+638), :24-25 (8-bit), :28-30 (4-bit), :33-35 (6-bit)
    assert oracle.geometry(7) == (129, 130, 17408)
    assert oracle.geometry(8) == (257, 258, 66306)
    assert oracle.geometry(4) == (17, 18, 1024)
    assert oracle.geometry(6) == (65, 66, 5120)
    for b in (4, 6, 7):
        assert oracle.geometry(b)[2] % (256 * 4) == 0   # 256 threads x 4-element loads (approx_gemm_forward.cu:84-87)
    with pytest.raises(NotImplementedError):
        oracle.geometry(5)


def test_parser_against_shipped_7bit_file(oracle, golden_dir):
    path = os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz")
    lines = gzip.open(path, "rt").read().splitlines()
    # header positions of this file: lines 20, 16405, 32790 (1-based) of 49174
    assert len(lines) == 49174
    assert lines[19].startswith(oracle.HEADER_FWD)
    assert lines[16404].startswith(oracle.HEADER_GA)
    assert lines[32789].startswith(oracle.HEADER_GB)
    fwd, ga, gb = oracle.parse_lut_file(path, 7)
    assert fwd[0, 0] == 88 and fwd[0, 4] == 88           # first data lines "0 0 88" ... "0 4 88"
    # spot-check every 997th data line of each section against the parsed tables
    for start, tab in ((20, fwd), (16405, ga), (32790, gb)):
        for ln in range(start, start + 16384, 997):
            a, b, v = map(int, lines[ln].split())
            assert tab[a, b] == v
    flat = oracle.pack_table(fwd, 7, np.uint16)
    assert flat.shape == (17408,) and flat[5 * 130 + 7] == fwd[5, 7]
    assert flat[128 * 130:].sum() == 0 and flat.reshape(-1)[:129 * 130].reshape(129, 130)[:, 128:].sum() == 0
    assert (oracle.unpack_table(flat, 7) == fwd).all()


def test_parser_header_after_junk_lines(oracle, golden_dir):
    # plain _lutfp.txt: ABC warnings + INFO lines first; gradient sections absent -> stay zero
    path = os.path.join(golden_dir, "lut7_vert_trunc_fwdonly.txt.gz")
    lines = gzip.open(path, "rt").read().splitlines()
    hdr = [i for i, l in enumerate(lines) if l.startswith(oracle.HEADER_FWD)]
    assert len(hdr) == 1 and hdr[0] > 0
    fwd, ga, gb = oracle.parse_lut_file(path, 7)
    a, b, v = map(int, lines[hdr[0] + 1 + 127 * 128 + 127].split())
    assert (a, b) == (127, 127) and fwd[127, 127] == v
    assert not ga.any() and not gb.any()


@pytest.mark.parametrize("name,bits,hw", [("lut6_vert_trunc_bp2.txt.gz", 6, 2), ("lut7_resub_63_bp8.txt.gz", 7, 8),
                                          ("lut7_evo_081_bp16.txt.gz", 7, 16)])
def test_gen_bp_lut_reproduces_shipped_gradient_tables(oracle, golden_dir, name, bits, hw):
    fwd, ga, gb = oracle.parse_lut_file(os.path.join(golden_dir, name), bits)
    a16, b16 = oracle.gen_bp_lut(fwd, hw)
    assert (a16 == ga).all() and (b16 == gb).all()


def test_gen_bp_lut_8bit_fixture(oracle, golden_dir):
    z = np.load(os.path.join(golden_dir, "lut8_resub_183.npz"))
    a16, b16 = oracle.gen_bp_lut(z["fwd"], int(z["half_window"]))
    assert (a16 == z["grad_a"]).all() and (b16 == z["grad_b"]).all()


def test_manifest_lists_every_fixture(golden_dir):
    man = json.load(open(os.path.join(golden_dir, "manifest.json")))
    for name in man:
        assert os.path.exists(os.path.join(golden_dir, name))


# ------------------------------------------------------------------------------------ forward math
def _rand_case(rng, M, K, N, bits):
    n = 1 << bits
    A = rng.integers(0, n, (M, K)).astype(np.uint8)
    B = rng.integers(0, n, (K, N)).astype(np.uint8)
    T = rng.integers(0, 65536, (n, n)).astype(np.int64)
    return A, B, T


def test_forward_np_is_the_triple_loop(oracle):
    rng = np.random.default_rng(1)
    A, B, T = _rand_case(rng, 5, 7, 3, 4)
    want = np.zeros((5, 3), np.int64)
    for m in range(5):
        for n in range(3):
            for k in range(7):
                want[m, n] += T[A[m, k], B[k, n]]
    assert (oracle.forward_np(A, B, T) == want.astype(np.uint32)).all()


@pytest.mark.parametrize("bits", [4, 6, 7, 8])
@pytest.mark.parametrize("shape", [(1, 1, 1), (9, 27, 10), (64, 64, 64), (33, 130, 65)])
def test_forward_c_equals_numpy(oracle, bits, shape):
    rng = np.random.default_rng(hash((bits, shape)) % 2**32)
    A, B, T = _rand_case(rng, *shape, bits)
    flat = oracle.pack_table(T, bits, np.uint16)
    assert (oracle.forward_c(A, B, flat, bits) == oracle.forward_np(A, B, T)).all()


@pytest.mark.parametrize("bits", [7, 8])
def test_forward_exact_multiplier_reduces_to_integer_matmul(oracle, bits):
    rng = np.random.default_rng(3)
    n = 1 << bits
    A, B, _ = _rand_case(rng, 40, 100, 24, bits)
    T = np.arange(n)[:, None] * np.arange(n)[None, :]
    want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.uint32)
    assert (oracle.forward_c(A, B, oracle.pack_table(T, bits, np.uint16), bits) == want).all()


def test_forward_asymmetric_table_catches_transposed_operands(oracle):
    # T[a][b] = a only: C[m,n] = sum_k A[m,k]; swapping the roles of a and b would give sum_k B[k,n]
    rng = np.random.default_rng(4)
    A, B, _ = _rand_case(rng, 6, 11, 5, 7)
    T = np.broadcast_to(np.arange(128)[:, None], (128, 128))
    got = oracle.forward_c(A, B, oracle.pack_table(T, 7, np.uint16), 7)
    assert (got == A.astype(np.int64).sum(1, keepdims=True)).all()


def test_forward_masked_code_contributes_zero(oracle):
    # code 2^b indexes the zero pad row / column (approx_mult.h:40)
    rng = np.random.default_rng(5)
    A, B, T = _rand_case(rng, 8, 16, 8, 7)
    flat = oracle.pack_table(T, 7, np.uint16)
    A2, B2 = A.copy(), B.copy()
    A2[:, 3] = 128
    B2[5, :] = 128
    want = oracle.forward_np(np.delete(A, [3, 5], 1), np.delete(B, [3, 5], 0), T)
    assert (oracle.forward_c(A2, B2, flat, 7) == want).all()


def test_forward_wraps_modulo_2_32(oracle):
    A = np.full((2, 70000), 255, np.uint8)
    B = np.full((70000, 2), 255, np.uint8)
    T = np.full((256, 256), 65535, np.int64)
    got = oracle.forward_c(A, B, oracle.pack_table(T, 8, np.uint16), 8)
    assert (got == (70000 * 65535) % 2**32).all()


def test_forward_linear_in_table(oracle):
    rng = np.random.default_rng(6)
    A, B, T1 = _rand_case(rng, 12, 20, 9, 6)
    T1 //= 2
    T2 = rng.integers(0, 32768, (64, 64))
    f = lambda T: oracle.forward_c(A, B, oracle.pack_table(T, 6, np.uint16), 6).astype(np.int64)
    assert (f(T1 + T2) == f(T1) + f(T2)).all()


# ----------------------------------------------------------------------------------- backward math
def test_backward_np_is_the_triple_loop(oracle):
    rng = np.random.default_rng(7)
    A, B, _ = _rand_case(rng, 4, 6, 5, 4)
    Ga = rng.integers(-300, 300, (16, 16))
    Gb = rng.integers(-300, 300, (16, 16))
    g = rng.standard_normal((4, 5)).astype(np.float32)
    gA = np.zeros((4, 6))
    gB = np.zeros((6, 5))
    for m in range(4):
        for k in range(6):
            for n in range(5):
                gA[m, k] += float(g[m, n]) * Ga[A[m, k], B[k, n]] / 16
                gB[k, n] += Gb[A[m, k], B[k, n]] * float(g[m, n]) / 16
    a, b = oracle.backward_np(g, A, B, Ga, Gb)
    np.testing.assert_allclose(a, gA, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(b, gB, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("bits", [6, 7, 8])
def test_backward_c_f64_equals_numpy(oracle, bits):
    rng = np.random.default_rng(8 + bits)
    n = 1 << bits
    A, B, _ = _rand_case(rng, 19, 31, 13, bits)
    Ga = rng.integers(-4000, 4000, (n, n))
    Gb = rng.integers(-4000, 4000, (n, n))
    g = rng.standard_normal((19, 13)).astype(np.float32)
    a, b = oracle.backward_c_f64(g, A, B, oracle.pack_table(Ga, bits, np.int16), oracle.pack_table(Gb, bits, np.int16), bits)
    an, bn = oracle.backward_np(g, A, B, Ga, Gb)
    np.testing.assert_allclose(a, an, rtol=1e-12, atol=1e-9)
    np.testing.assert_allclose(b, bn, rtol=1e-12, atol=1e-9)


@pytest.mark.parametrize("bits,shape", [(7, (301, 19, 13)), (8, (64, 33, 70)), (6, (1000, 8, 5))])
def test_row_streaming_gradB_equals_brute_force_and_ste_matmul(oracle, bits, shape):
    # the loop order used for full-size layers: against the numpy brute force (asymmetric random table: catches a / b swapped),
    # its |terms| sums against the same brute force on absolute values, and STE tables against the dense integer product
    M, K, N = shape
    rng = np.random.default_rng(80 + bits)
    n = 1 << bits
    A, B, _ = _rand_case(rng, M, K, N, bits)
    Gb = rng.integers(-4000, 4000, (n, n))
    g = rng.standard_normal((M, N)).astype(np.float32)
    lb = oracle.pack_table(Gb, bits, np.int16)
    b, ab = oracle.gradB_c_f64_rows(g, A, B, lb, bits)
    _, bn = oracle.backward_np(g, A, B, Gb, Gb)
    _, abn = oracle.backward_np(np.abs(g), A, B, np.abs(Gb), np.abs(Gb))
    np.testing.assert_allclose(b, bn, rtol=1e-12, atol=1e-9)
    np.testing.assert_allclose(ab, abn, rtol=1e-12, atol=1e-9)
    gi = rng.integers(-8, 9, (M, N)).astype(np.float32)
    _, Gy = oracle.ste_tables16(bits)
    bs, _ = oracle.gradB_c_f64_rows(gi, A, B, oracle.pack_table(Gy, bits, np.int16), bits)
    assert (bs == A.astype(np.int64).T @ gi.astype(np.int64)).all()


def test_backward_ste_tables_reduce_to_dense_matmuls_bit_exact(oracle):
    # the author's known-answer idea (approx_ops.py:81-86): Gx = 16 b, Gy = 16 a  =>  gA = gC B^T, gB = A^T gC.
    # With small integer gC every fp32 partial sum is exact, so the fp32 oracle must match bit for bit.
    rng = np.random.default_rng(9)
    A, B, _ = _rand_case(rng, 50, 40, 30, 7)
    g = rng.integers(-8, 9, (50, 30)).astype(np.float32)
    Gx, Gy = oracle.ste_tables16(7)
    la, lb = oracle.pack_table(Gx, 7, np.int16), oracle.pack_table(Gy, 7, np.int16)
    a32, b32 = oracle.backward_c_f32(g, A, B, la, lb, 7)
    a64, b64 = oracle.backward_c_f64(g, A, B, la, lb, 7)
    wantA = g.astype(np.int64) @ B.astype(np.int64).T
    wantB = A.astype(np.int64).T @ g.astype(np.int64)
    assert (a32 == wantA).all() and (b32 == wantB).all()
    assert (a64 == wantA).all() and (b64 == wantB).all()


def test_backward_f32_reference_order_close_to_f64(oracle):
    A, B, T, g = oracle.synth_gemm(300, 96, 64, bits=7, err=64, seed=2)
    Gx, Gy = oracle.gen_bp_lut(T, 8)
    la, lb = oracle.pack_table(Gx, 7, np.int16), oracle.pack_table(Gy, 7, np.int16)
    a32, b32 = oracle.backward_c_f32(g, A, B, la, lb, 7)
    a64, b64, absA, absB = oracle.backward_c_f64(g, A, B, la, lb, 7, want_abs=True)
    assert np.max(np.abs(a32 - a64) / absA) < 1e-5
    assert np.max(np.abs(b32 - b64) / absB) < 1e-5


def test_accgemm_oracle(oracle):
    rng = np.random.default_rng(10)
    A = rng.integers(-5, 6, (17, 33)).astype(np.float32)
    B = rng.integers(-5, 6, (33, 9)).astype(np.float32)
    assert (oracle.accgemm_c(A, B) == A @ B).all()


# ---------------------------------------------------------------------------------------- conv glue
def test_conv_oracle_equals_torch_conv2d_with_exact_multiplier(oracle):
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(11)
    T = np.arange(128)[:, None] * np.arange(128)[None, :]
    for (s, p, d, kh) in [(1, 1, 1, 3), (2, 1, 1, 3), (1, 0, 1, 1), (2, 0, 1, 1), (1, 2, 2, 3)]:
        x = rng.integers(0, 128, (2, 3, 9, 9)).astype(np.uint8)
        w = rng.integers(0, 128, (4, 3, kh, kh)).astype(np.uint8)
        got = oracle.conv2d_lut_np(x, w, T, s, p, d)
        want = F.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(w.astype(np.float64)), stride=s, padding=p, dilation=d)
        assert (got.astype(np.int64) == want.numpy().astype(np.int64)).all()
