"""TEST INFRASTRUCTURE ONLY -- NumPy/C restatement of the reference LUT-GEMM path.

This module is the checker for the HIP kernels and the host code.  It may be imported only by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``; the product
package never imports it and has no CPU fallback.

Every function names the reference lines it restates.  What pins each function (so that a dropped
term, a transposed operand or a wrong index fails a test) is listed next to it; the tests are in
``tests/test_oracle.py``.

Parity status: every function below is pinned either by data files shipped in the reference
(``app_mults/**``, committed as fixtures under ``tests/golden/``) or by a closed form that reduces to a
NumPy/torch library routine.  None is "parity unpinned".  The one thing no CPU check can pin is the
exact fp32 rounding sequence of the reference's CUDA backward sums; the contract there is a
tolerance (1e-5 relative), judged against the float64 sums of ``backward_f64``.
"""
from __future__ import annotations

import ctypes
import gzip
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

FACTOR = 1.0 / 16.0  # self_ops/src/approx_mult.h:41
HEADER_FWD = "LUT for approximate multiplier:"
HEADER_GA = "LUT for the gradient of the approximate multiplier w.r.t. the first operand:"
HEADER_GB = "LUT for the gradient of the approximate multiplier w.r.t. the second operand:"


# ----------------------------------------------------------------------------------------------
# Table geometry (self_ops/src/approx_mult.h:12-40, mirrored at self_ops/ops_py/approx_ops.py:21-41)
# Pinned by: lengths 17408 / 66306 / 1024 / 5120 quoted in the reference comments and divisibility
# by 256 threads x 4 elements for the <8-bit cases (approx_gemm_forward.cu:84-87).
# ----------------------------------------------------------------------------------------------
_TAIL = {7: 638, 8: 0, 4: 718, 6: 830}


def geometry(bits: int):
    """Return (rows, cols, elem_num) of the padded 1-D table for a bit-width."""
    if bits not in _TAIL:
        raise NotImplementedError(f"quantization_bit = {bits} is not supported")
    maxval = (1 << bits) - 1
    rows, cols = maxval + 2, maxval + 3
    return rows, cols, rows * cols + _TAIL[bits]


def pack_table(table2d: np.ndarray, bits: int, dtype) -> np.ndarray:
    """Place a (2^b, 2^b) table at index a*cols+b of a zero 1-D array of length elem_num
    (self_ops/ops_py/approx_ops.py:51-53,70-77)."""
    rows, cols, elems = geometry(bits)
    n = 1 << bits
    assert table2d.shape == (n, n)
    out = np.zeros(elems, dtype=dtype)
    idx = (np.arange(n)[:, None] * cols + np.arange(n)[None, :]).ravel()
    out[idx] = table2d.astype(dtype).ravel()
    return out


def unpack_table(flat: np.ndarray, bits: int) -> np.ndarray:
    rows, cols, elems = geometry(bits)
    n = 1 << bits
    assert flat.shape == (elems,)
    return flat[: rows * cols].reshape(rows, cols)[:n, :n].copy()


# ----------------------------------------------------------------------------------------------
# Text file format (self_ops/ops_py/approx_ops.py:54-79): a 4-state machine keyed on three header
# strings; every other line before the first header is skipped; data lines are "a b value".
# Pinned by: the shipped files (tests/golden/*.txt.gz) -- spot values at known lines, 2^(2b) entries
# per section, header positions that differ between files.
# ----------------------------------------------------------------------------------------------
def _open_text(path):
    if path.endswith(".gz"):
        return gzip.open(path, "rt")
    return open(path, "r")


def parse_lut_file(path: str, bits: int):
    """Line-by-line restatement of the reference parser.  Returns three (2^b, 2^b) int64 arrays
    (forward, grad wrt first operand, grad wrt second operand); sections absent from the file stay 0."""
    n = 1 << bits
    tabs = {"load_appmult": np.zeros((n, n), np.int64), "load_grad_a": np.zeros((n, n), np.int64),
            "load_grad_b": np.zeros((n, n), np.int64)}
    state = "init"
    with _open_text(path) as f:
        for line in f:
            if line.startswith(HEADER_FWD):
                state = "load_appmult"
                continue
            elif line.startswith(HEADER_GA):
                state = "load_grad_a"
                continue
            elif line.startswith(HEADER_GB):
                state = "load_grad_b"
                continue
            elif state == "init":
                continue
            a, b, res = line.split()
            tabs[state][int(a), int(b)] = int(res)
    return tabs["load_appmult"], tabs["load_grad_a"], tabs["load_grad_b"]


# ----------------------------------------------------------------------------------------------
# Gradient tables (scripts/gen_bp_lut.py:7-62 smoothing + central difference, :172-183 x16 rounding)
# Pinned by: the shipped (forward section -> gradient sections) pairs inside every "+bp" file.
# ----------------------------------------------------------------------------------------------
def gen_bp_lut(fwd: np.ndarray, half_ws: int, rounded: bool = True):
    """Literal (loop-for-loop) restatement; float32 arithmetic exactly as NumPy does it there.
    Returns (grad_a16, grad_b16) as int64 = round(16 * slope); with rounded=False the float32 slopes themselves
    (the values the reference's script holds just before its x16 rounding, gen_bp_lut.py:172-183)."""
    lut = fwd.astype(np.float32)
    R, Cn = lut.shape
    smooth_a = np.zeros((R, Cn), np.float32)
    smooth_b = np.zeros((R, Cn), np.float32)
    for b in range(Cn):          # gen_bp_lut.py:36-45
        for a in range(R):
            smooth_a[a][b] = np.mean(lut[max(0, a - half_ws):min(R, a + half_ws + 1), b])
    for a in range(R):           # gen_bp_lut.py:7-16
        for b in range(Cn):
            smooth_b[a][b] = np.mean(lut[a][max(0, b - half_ws):min(Cn, b + half_ws + 1)])
    grad_a = np.zeros((R, Cn), np.float32)
    grad_b = np.zeros((R, Cn), np.float32)
    assert half_ws >= 1
    for b in range(Cn):          # gen_bp_lut.py:48-62
        for a in range(R):
            if half_ws + 1 <= a <= R - 1 - half_ws - 1:
                grad_a[a][b] = (smooth_a[a + 1][b] - smooth_a[a - 1][b]) / 2
            else:
                # the reference indexes lut[0:R][b], i.e. ROW b, not column b (gen_bp_lut.py:58-59)
                grad_a[a][b] = (np.max(lut[0:R][b]) - np.min(lut[0:R][b])) / R
    for a in range(R):           # gen_bp_lut.py:19-33
        for b in range(Cn):
            if half_ws + 1 <= b <= Cn - 1 - half_ws - 1:
                grad_b[a][b] = (smooth_b[a][b + 1] - smooth_b[a][b - 1]) / 2
            else:
                grad_b[a][b] = (np.max(lut[a][0:Cn]) - np.min(lut[a][0:Cn])) / Cn
    if not rounded:
        return grad_a, grad_b
    ga16 = np.round(grad_a * np.float32(16.0)).astype(np.int64)
    gb16 = np.round(grad_b * np.float32(16.0)).astype(np.int64)
    return ga16, gb16


# ----------------------------------------------------------------------------------------------
# GEMM arithmetic in NumPy (brute force; small shapes) -- these pin the C oracle below.
# ----------------------------------------------------------------------------------------------
def forward_np(A: np.ndarray, B: np.ndarray, fwd2d: np.ndarray) -> np.ndarray:
    """C[m,n] = sum_k T[A[m,k], B[k,n]] in int64, returned modulo 2^32 as uint32
    (self_ops/src/approx_gemm_forward.cu:200, uint32 accumulator :111)."""
    T = np.asarray(fwd2d, np.int64)
    M, K = A.shape
    N = B.shape[1]
    C = np.zeros((M, N), np.int64)
    for k in range(K):
        C += T[A[:, k].astype(np.int64)[:, None], B[k, :].astype(np.int64)[None, :]]
    return (C & 0xFFFFFFFF).astype(np.uint32)


def backward_np(gC, A, B, ga2d, gb2d, factor=FACTOR):
    """float64 sums: gA[m,k] = f*sum_n gC[m,n]*Ga[A[m,k],B[k,n]], gB[k,n] = f*sum_m Gb[A[m,k],B[k,n]]*gC[m,n]
    (self_ops/src/approx_gemm_backward.cu:220,240 and :454,474)."""
    Ga = np.asarray(ga2d, np.float64)
    Gb = np.asarray(gb2d, np.float64)
    g = np.asarray(gC, np.float64)
    M, K = A.shape
    N = B.shape[1]
    gA = np.zeros((M, K))
    gB = np.zeros((K, N))
    Ai = A.astype(np.int64)
    Bi = B.astype(np.int64)
    for k in range(K):
        ta = Ga[Ai[:, k][:, None], Bi[k, :][None, :]]      # [M, N]
        tb = Gb[Ai[:, k][:, None], Bi[k, :][None, :]]
        gA[:, k] = (g * ta).sum(axis=1)
        gB[k, :] = (tb * g).sum(axis=0)
    return gA * factor, gB * factor


# ----------------------------------------------------------------------------------------------
# im2col glue (self_ops/ops_py/approx_ops.py:545-571) as explicit index arithmetic.
# Pinned by: with the exact-multiplier table the result must equal torch conv2d on integer tensors.
# ----------------------------------------------------------------------------------------------
def im2col_np(x: np.ndarray, kh: int, kw: int, stride: int, padding: int, dilation: int) -> np.ndarray:
    """x [B,C,H,W] -> [B*oh*ow, C*kh*kw]; K index = c*kh*kw + i*kw + j; padding pixels hold code 0."""
    Bn, Cc, H, W = x.shape
    oh = (H + 2 * padding - dilation * (kh - 1) - 1) // stride + 1
    ow = (W + 2 * padding - dilation * (kw - 1) - 1) // stride + 1
    xp = np.zeros((Bn, Cc, H + 2 * padding, W + 2 * padding), x.dtype)
    xp[:, :, padding:padding + H, padding:padding + W] = x
    out = np.zeros((Bn, oh * ow, Cc * kh * kw), x.dtype)
    for c in range(Cc):
        for i in range(kh):
            for j in range(kw):
                patch = xp[:, c, i * dilation: i * dilation + stride * (oh - 1) + 1: stride,
                           j * dilation: j * dilation + stride * (ow - 1) + 1: stride]
                out[:, :, c * kh * kw + i * kw + j] = patch.reshape(Bn, oh * ow)
    return out.reshape(Bn * oh * ow, Cc * kh * kw), oh, ow


def conv2d_lut_np(x_codes, w_codes, fwd2d, stride=1, padding=0, dilation=1):
    """approx_conv2d_op forward on integer code arrays; returns uint32 [B, outC, oh, ow]."""
    outC, _, kh, kw = w_codes.shape
    Bn = x_codes.shape[0]
    cols, oh, ow = im2col_np(x_codes, kh, kw, stride, padding, dilation)
    Wm = w_codes.reshape(outC, -1).T
    Cm = forward_np(cols, Wm, fwd2d)
    return Cm.reshape(Bn, oh * ow, outC).transpose(0, 2, 1).reshape(Bn, outC, oh, ow)


# ----------------------------------------------------------------------------------------------
# Synthetic workloads of the benchmark configurations (seeded, numpy PCG64; drawn in this order).
# ----------------------------------------------------------------------------------------------
def synth_lut(bits: int, err: int, rng: np.random.Generator) -> np.ndarray:
    n = 1 << bits
    a = np.arange(n, dtype=np.int64)
    E = rng.integers(-err, err + 1, size=(n, n))
    return np.clip(a[:, None] * a[None, :] + E, 0, 65535)


def synth_gemm(M, K, N, bits=7, err=64, seed=0):
    rng = np.random.default_rng(seed)
    A = rng.integers(0, 1 << bits, size=(M, K), dtype=np.uint8 if bits <= 8 else np.uint16).astype(np.uint8)
    B = rng.integers(0, 1 << bits, size=(K, N)).astype(np.uint8)
    T = synth_lut(bits, err, rng)
    gC = rng.standard_normal((M, N)).astype(np.float32)
    return A, B, T, gC


def ste_tables16(bits: int):
    """Gx16[a][b] = 16*b, Gy16[a][b] = 16*a -- the author's own known-answer idea
    (self_ops/ops_py/approx_ops.py:81-86)."""
    n = 1 << bits
    a = np.arange(n, dtype=np.int64)
    return np.broadcast_to(16 * a[None, :], (n, n)).copy(), np.broadcast_to(16 * a[:, None], (n, n)).copy()


# ----------------------------------------------------------------------------------------------
# C oracle (oracle/lutgemm_oracle.c) loader
# ----------------------------------------------------------------------------------------------
_LIB = None


def build_c_oracle(force: bool = False) -> str:
    so = os.path.join(_HERE, "_build", "liblutgemm_oracle.so")
    src = os.path.join(_HERE, "lutgemm_oracle.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return so


def c_lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "_build", "liblutgemm_oracle.so")
        if not os.path.exists(so):
            build_c_oracle()
        _LIB = ctypes.CDLL(so)
        _LIB.oracle_num_threads.restype = ctypes.c_int
    return _LIB


def _p(arr):
    return arr.ctypes.data_as(ctypes.c_void_p)


def forward_c(A, B, lut_flat_u16, bits):
    rows, cols, elems = geometry(bits)
    A = np.ascontiguousarray(A, np.uint8)
    B = np.ascontiguousarray(B, np.uint8)
    lut = np.ascontiguousarray(lut_flat_u16, np.uint16)
    assert lut.shape == (elems,)
    M, K = A.shape
    N = B.shape[1]
    C = np.empty((M, N), np.uint32)
    c_lib().oracle_lutgemm_forward(_p(A), _p(B), _p(C), _p(lut), ctypes.c_int(cols),
                                   ctypes.c_int(M), ctypes.c_int(K), ctypes.c_int(N))
    return C


def backward_c_f32(gC, A, B, lutA_i16, lutB_i16, bits, factor=FACTOR):
    rows, cols, elems = geometry(bits)
    gC = np.ascontiguousarray(gC, np.float32)
    A = np.ascontiguousarray(A, np.uint8)
    B = np.ascontiguousarray(B, np.uint8)
    la = np.ascontiguousarray(lutA_i16, np.int16)
    lb = np.ascontiguousarray(lutB_i16, np.int16)
    M, K = A.shape
    N = B.shape[1]
    gA = np.empty((M, K), np.float32)
    gB = np.empty((K, N), np.float32)
    c_lib().oracle_lutgemm_backward_f32(_p(gC), _p(A), _p(B), _p(gA), _p(gB), _p(la), _p(lb), ctypes.c_int(cols),
                                        ctypes.c_float(factor), ctypes.c_int(M), ctypes.c_int(K), ctypes.c_int(N))
    return gA, gB


def backward_c_f64(gC, A, B, lutA_flat, lutB_flat, bits, factor=FACTOR, want_abs=False):
    """Tables are flat padded arrays of any numeric dtype (int16 x16 tables, or fp32 slope tables)."""
    rows, cols, elems = geometry(bits)
    gC = np.ascontiguousarray(gC, np.float32)
    A = np.ascontiguousarray(A, np.uint8)
    B = np.ascontiguousarray(B, np.uint8)
    la = np.ascontiguousarray(lutA_flat, np.float64)
    lb = np.ascontiguousarray(lutB_flat, np.float64)
    M, K = A.shape
    N = B.shape[1]
    gA = np.empty((M, K), np.float64)
    gB = np.empty((K, N), np.float64)
    aA = np.empty((M, K), np.float64) if want_abs else None
    aB = np.empty((K, N), np.float64) if want_abs else None
    c_lib().oracle_lutgemm_backward_f64(_p(gC), _p(A), _p(B), _p(gA), _p(gB),
                                        _p(aA) if want_abs else None, _p(aB) if want_abs else None,
                                        _p(la), _p(lb), ctypes.c_int(cols), ctypes.c_double(factor),
                                        ctypes.c_int(M), ctypes.c_int(K), ctypes.c_int(N))
    if want_abs:
        return gA, gB, aA, aB
    return gA, gB


def gradB_c_f64_rows(gC, A, B, lutB_flat, bits, factor=FACTOR):
    """gB and the sums of |terms| of gB in float64 for layers with very many rows (row-streaming loop order)."""
    rows, cols, elems = geometry(bits)
    gC = np.ascontiguousarray(gC, np.float32)
    A = np.ascontiguousarray(A, np.uint8)
    B = np.ascontiguousarray(B, np.uint8)
    lb = np.ascontiguousarray(lutB_flat, np.float64)
    M, K = A.shape
    N = B.shape[1]
    gB = np.empty((K, N), np.float64)
    aB = np.empty((K, N), np.float64)
    c_lib().oracle_lutgemm_gradB_f64_rows(_p(gC), _p(A), _p(B), _p(gB), _p(aB), _p(lb), ctypes.c_int(cols),
                                          ctypes.c_double(factor), ctypes.c_int(M), ctypes.c_int(K), ctypes.c_int(N))
    return gB, aB


def accgemm_c(A, B):
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M, K = A.shape
    N = B.shape[1]
    C = np.empty((M, N), np.float32)
    c_lib().oracle_accgemm_forward_f32(_p(A), _p(B), _p(C), ctypes.c_int(M), ctypes.c_int(K), ctypes.c_int(N))
    return C
