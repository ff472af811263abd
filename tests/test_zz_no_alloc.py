"""amr_lut_gemm_backward_static -- the backward entry point that allocates nothing (its scratch is a device array inside
the library) -- against amr_lut_gemm_backward_ex with a caller workspace, through the C ABI.  Collected last on purpose:
a failure here must not hide the other tests."""
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
    L.amr_lut_gemm_backward_ex.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i, i, i, i, vp, sz, vp]
    L.amr_lut_gemm_backward_static.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i, i, i, i, vp]
    L.amr_lut_gemm_backward_workspace_bytes.argtypes = [i, i, i]
    L.amr_lut_gemm_backward_workspace_bytes.restype = sz
    L.amr_static_scratch_bytes.restype = sz
    L.amr_library_resources.argtypes = [ctypes.POINTER(sz), ctypes.POINTER(i)]
    L.amr_library_resources.restype = None
    return L


def library_resources(lib):
    b, n = ctypes.c_size_t(0), ctypes.c_int(0)
    lib.amr_library_resources(ctypes.byref(b), ctypes.byref(n))
    return b.value, n.value


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def both_ways(lib, oracle, seed, M, K, N, bits, rows_per_image=0, lo=-1024, hi=3073, same_kernels=True):
    """One problem through both entry points: identical bits where both run the same kernels (same order of additions),
    and the new entry point's results within tolerance of the float64 oracle."""
    rng = np.random.default_rng(seed)
    n = 1 << bits
    A = rng.integers(0, n, (M, K)).astype(np.uint8)
    B = rng.integers(0, n, (K, N)).astype(np.uint8)
    la = oracle.pack_table(rng.integers(lo, hi, (n, n)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(lo, hi, (n, n)), bits, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(la), dev(lb)
    ga_shape = (M // rows_per_image, K, rows_per_image) if rows_per_image else (M, K)
    out = []
    for static in (False, True):
        ga = torch.full(ga_shape, float("nan"), device="cuda")
        gb = torch.full((K, N), float("nan"), device="cuda")
        if static:
            rc = lib.amr_lut_gemm_backward_static(gd.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                                  tb.data_ptr(), ta.numel(), M, K, N, rows_per_image, None)
        else:
            need = lib.amr_lut_gemm_backward_workspace_bytes(M, K, N)
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
            rc = lib.amr_lut_gemm_backward_ex(gd.data_ptr(), a.data_ptr(), b.data_ptr(), ga.data_ptr(), gb.data_ptr(), ta.data_ptr(),
                                              tb.data_ptr(), ta.numel(), M, K, N, rows_per_image, ws.data_ptr(), need, None)
        assert rc == 0, lib.amr_last_error()
        torch.cuda.synchronize()
        out.append((ga, gb))
    (ga0, gb0), (ga1, gb1) = out
    # (same_kernels False: the array held fewer M splits of gB or no expanded table of gradA, so the additions ran in another order)
    assert not same_kernels or (torch.equal(gb0, gb1) and torch.equal(ga0, ga1))
    a64, b64, absA, absB = oracle.backward_c_f64(g, A, B, la, lb, bits, want_abs=True)
    gA = ga1.cpu().numpy()
    if rows_per_image:
        gA = gA.transpose(0, 2, 1).reshape(M, K)
    for x, r, ab in ((gA, a64, absA), (gb1.cpu().numpy(), b64, absB)):
        err = np.abs(x - r)
        assert np.max(err / np.maximum(ab, 1e-30)) < TOL
        assert np.max(err) <= TOL * np.max(np.abs(r)) + 1e-30


def test_static_scratch_backward_two_calls_in_a_row(lib, oracle):
    print("static scratch: two calls", flush=True)
    assert lib.amr_static_scratch_bytes() == 32 << 20
    # expanded-table kernels of both gradients (scratch: flags, partial sums over the M splits, expanded table) ...
    both_ways(lib, oracle, 1, 8192, 576, 64, 7)
    # ... then a smaller problem on the same scratch, which still holds the first call's flags, sums and table
    both_ways(lib, oracle, 2, 2048, 64, 32, 7)
    # direct kernels (8-bit table), ragged shape, image-major gA, a table that needs no offset
    both_ways(lib, oracle, 3, 1500, 40, 70, 8)
    both_ways(lib, oracle, 4, 4096, 48, 64, 6, rows_per_image=256, lo=-2048, hi=2049)
    both_ways(lib, oracle, 5, 300, 27, 10, 7)
    # 8-bit table, 2048 rows: gradA with the table expanded in LDS (scratch: partial results per column tile), gradB on the
    # int16 slab; row-major and image-major gA
    both_ways(lib, oracle, 7, 2048, 16, 128, 8, lo=-32768, hi=32768)
    both_ways(lib, oracle, 8, 2048, 12, 64, 8, rows_per_image=256, lo=-32768, hi=32768)


def test_static_scratch_backward_steps_aside_or_rejects_beyond_its_size(lib, oracle):
    print("static scratch: limits", flush=True)
    # the expanded table of gradA (K * N * 256 B = 64 MB) does not fit 32 MiB: gradA runs on the direct kernel, results as before
    assert lib.amr_lut_gemm_backward_workspace_bytes(4096, 1024, 256) > lib.amr_static_scratch_bytes()
    both_ways(lib, oracle, 6, 4096, 1024, 256, 7, same_kernels=False)
    # the column sums of gC of the half-slab gradB kernel (64 x N floats) alone beyond the array: rejected before anything is launched
    t = torch.zeros(64, device="cuda")
    tab = torch.zeros(17408, dtype=torch.int16, device="cuda")
    rc = lib.amr_lut_gemm_backward_static(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), tab.data_ptr(),
                                          tab.data_ptr(), 17408, 1024, 8, 131072 + 64, 0, None)
    assert rc == -3 and b"static scratch" in lib.amr_last_error()


def test_static_scratch_backward_runs_the_largest_benchmark_layer(lib, oracle):
    """4096 x 4608 x 512 on 7-bit tables (the widest convolution of the ResNet-18 step): one set of partial sums of gB is
    9.4 MB and the expanded table of gradA 604 MB; the array holds three M splits and no table, and the results are still
    those of the float64 sums."""
    print("static scratch: 4096 x 4608 x 512", flush=True)
    both_ways(lib, oracle, 9, 4096, 4608, 512, 7, same_kernels=False)


def test_static_scratch_backward_allocates_nothing_and_can_be_captured(lib, oracle):
    """On a stream the library has never seen (the library's own scratch is per stream), the call changes the device's free
    memory by nothing; recorded into a HIP
    graph (after an uncaptured call), every replay gives the eager result."""
    print("static scratch: no allocation, graph capture", flush=True)
    rng = np.random.default_rng(11)
    M, K, N, bits = 4096, 64, 64, 7
    A, B = rng.integers(0, 128, (M, K)).astype(np.uint8), rng.integers(0, 128, (K, N)).astype(np.uint8)
    la = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), bits, np.int16)
    lb = oracle.pack_table(rng.integers(-1024, 3073, (128, 128)), bits, np.int16)
    g = rng.standard_normal((M, N)).astype(np.float32)
    gd, a, b, ta, tb = dev(g), dev(A), dev(B), dev(la), dev(lb)
    ga, gb = torch.empty((M, K), device="cuda"), torch.empty((K, N), device="cuda")
    ga_g, gb_g = torch.empty_like(ga), torch.empty_like(gb)

    def call(out_a, out_b, stream):
        rc = lib.amr_lut_gemm_backward_static(gd.data_ptr(), a.data_ptr(), b.data_ptr(), out_a.data_ptr(), out_b.data_ptr(), ta.data_ptr(),
                                              tb.data_ptr(), ta.numel(), M, K, N, 0, ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, lib.amr_last_error()

    fresh = torch.cuda.Stream()
    taken_before = library_resources(lib)
    call(ga, gb, fresh)                             # (the runtime sets up the stream's queue and the kernels' code on first use)
    fresh.synchronize()
    ga.fill_(float("nan"))
    gb.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    call(ga, gb, fresh)
    fresh.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point changed the device's free memory"
    assert library_resources(lib) == taken_before, "the static entry point took scratch or a side stream from the runtime"
    # (the same call through the entry point with library-owned scratch does take some for that stream: the check above can fail)
    ws_call = lib.amr_lut_gemm_backward_ex(gd.data_ptr(), a.data_ptr(), b.data_ptr(), ga_g.data_ptr(), gb_g.data_ptr(), ta.data_ptr(),
                                           tb.data_ptr(), ta.numel(), M, K, N, 0, None, 0, ctypes.c_void_p(fresh.cuda_stream))
    assert ws_call == 0, lib.amr_last_error()
    fresh.synchronize()
    assert library_resources(lib)[0] > taken_before[0]
    a64, b64 = oracle.backward_c_f64(g, A, B, la, lb, bits)
    assert np.abs(ga.cpu().numpy() - a64).max() <= TOL * np.abs(a64).max()
    assert np.abs(gb.cpu().numpy() - b64).max() <= TOL * np.abs(b64).max()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(ga_g, gb_g, side)                      # uncaptured call: one-time attribute calls happen outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(ga_g, gb_g, torch.cuda.current_stream())
    for replay in range(3):
        ga_g.fill_(float("nan"))
        gb_g.fill_(float("nan"))
        torch.cuda.synchronize()                    # eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ga_g, ga) and torch.equal(gb_g, gb), f"replay {replay} differs from the eager call"
