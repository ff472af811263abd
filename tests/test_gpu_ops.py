"""GPU tests of the Python operator layer (approx_ops module + self_ops autograd Functions), written
the way a user of the reference would call them."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(golden_dir):
    import self_ops
    from self_ops.ops_py import approx_ops as P
    P.init_lookup_tables(torch.device("cuda"), os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), 7)
    return self_ops, P


def test_native_module_checks_dtype_shape_contiguity(ops):
    import approx_ops
    print("native checks", flush=True)
    d = "cuda"
    a = torch.zeros(4, 6, dtype=torch.uint8, device=d)
    b = torch.zeros(6, 8, dtype=torch.uint8, device=d)
    c = torch.zeros(4, 8, dtype=torch.uint32, device=d)
    lut = torch.zeros(17408, dtype=torch.uint16, device=d)
    approx_ops.approx_gemm_forward(a, b, c, lut)
    with pytest.raises(RuntimeError, match="b_tensor must be contiguous"):
        approx_ops.approx_gemm_forward(a, torch.zeros(8, 6, dtype=torch.uint8, device=d).t(), c, lut)
    with pytest.raises(RuntimeError, match="a_tensor must be of type"):
        approx_ops.approx_gemm_forward(a.float(), b, c, lut)
    with pytest.raises(RuntimeError, match="c_tensor's shape should be 4 x 8"):
        approx_ops.approx_gemm_forward(a, b, torch.zeros(4, 9, dtype=torch.uint32, device=d), lut)
    with pytest.raises(RuntimeError, match="b_tensor's shape should be"):
        approx_ops.approx_gemm_forward(a, torch.zeros(5, 8, dtype=torch.uint8, device=d), c, lut)
    with pytest.raises(RuntimeError, match="QUANTIZATION_BIT"):
        approx_ops.approx_gemm_forward(a, b, c, lut[:17000].contiguous())
    with pytest.raises(RuntimeError, match="lut_appmult_tensor must be a CUDAtensor"):
        approx_ops.approx_gemm_forward(a, b, c, lut.cpu())


def test_gemm_op_forward_and_backward_against_oracle(ops, oracle, golden_dir):
    self_ops, P = ops
    print("gemm op", flush=True)
    fwd, ga, gb = oracle.parse_lut_file(os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), 7)
    rng = np.random.default_rng(0)
    A = rng.integers(0, 128, (200, 72)).astype(np.uint8)
    B = rng.integers(0, 128, (72, 48)).astype(np.uint8)
    a = torch.tensor(A, dtype=torch.float32, device="cuda", requires_grad=True)
    bt = torch.tensor(B.T.copy(), dtype=torch.float32, device="cuda", requires_grad=True)   # weight arrives as a .t() view
    out = self_ops.approx_gemm_op(a, bt.t())
    assert out.dtype == torch.float32
    assert (out.detach().cpu().numpy() == oracle.forward_np(A, B, fwd).astype(np.float32)).all()
    g = torch.randn(200, 48, device="cuda")
    out.backward(g)
    a64, b64 = oracle.backward_np(g.cpu().numpy(), A, B, ga, gb)
    np.testing.assert_allclose(a.grad.cpu().numpy(), a64, rtol=0, atol=1e-5 * np.abs(a64).max())
    np.testing.assert_allclose(bt.grad.cpu().numpy().T, b64, rtol=0, atol=1e-5 * np.abs(b64).max())


def test_gemm_and_conv_ops_with_float_gradient_tables(ops, oracle, golden_dir):
    """Float32 gradient tables installed with set_lookup_tables: slopes themselves, no 1/16."""
    self_ops, P = ops
    print("gemm / conv op, float gradient tables", flush=True)
    fwd, _, _ = oracle.parse_lut_file(os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), 7)
    Gx, Gy = oracle.gen_bp_lut(fwd, 8, rounded=False)
    saved = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
    try:
        P.set_lookup_tables("cuda", oracle.pack_table(fwd, 7, np.uint16), oracle.pack_table(Gx, 7, np.float32),
                            oracle.pack_table(Gy, 7, np.float32))
        assert P.lut_grad_a.dtype == torch.float32 and P.lut_grad_b.dtype == torch.float32
        rng = np.random.default_rng(3)
        A = rng.integers(0, 128, (200, 72)).astype(np.uint8)
        B = rng.integers(0, 128, (72, 48)).astype(np.uint8)
        a = torch.tensor(A, dtype=torch.float32, device="cuda", requires_grad=True)
        b = torch.tensor(B, dtype=torch.float32, device="cuda", requires_grad=True)
        out = self_ops.approx_gemm_op(a, b)
        g = torch.randn(200, 48, device="cuda")
        out.backward(g)
        a64, b64 = oracle.backward_np(g.cpu().numpy(), A, B, Gx, Gy, factor=1.0)
        np.testing.assert_allclose(a.grad.cpu().numpy(), a64, rtol=0, atol=1e-5 * np.abs(a64).max())
        np.testing.assert_allclose(b.grad.cpu().numpy(), b64, rtol=0, atol=1e-5 * np.abs(b64).max())
        # the convolution on the same tables: its gradients are those of the GEMM of its im2col matrix
        x = torch.tensor(rng.integers(0, 128, (2, 3, 9, 9)), dtype=torch.float32, device="cuda", requires_grad=True)
        w = torch.tensor(rng.integers(0, 128, (5, 3, 3, 3)), dtype=torch.float32, device="cuda", requires_grad=True)
        y = self_ops.approx_conv2d_op(x, w, None, (1, 1), (1, 1), (1, 1), 1)
        gy = torch.randn_like(y)
        y.backward(gy)
        cols, oh, ow = oracle.im2col_np(x.detach().cpu().numpy().astype(np.uint8), 3, 3, 1, 1, 1)
        Wm = w.detach().cpu().numpy().astype(np.uint8).reshape(5, -1).T.copy()
        gm = gy.permute(0, 2, 3, 1).reshape(-1, 5).cpu().numpy()
        ga64, gb64 = oracle.backward_np(gm, cols, Wm, Gx, Gy, factor=1.0)
        np.testing.assert_allclose(w.grad.cpu().numpy().reshape(5, -1).T, gb64, rtol=0, atol=1e-5 * np.abs(gb64).max())
        fold = F.fold(torch.tensor(ga64.reshape(2, oh * ow, -1).transpose(0, 2, 1).copy()), (9, 9), (3, 3), padding=1)
        np.testing.assert_allclose(x.grad.cpu().numpy(), fold.numpy(), rtol=0, atol=1e-5 * float(fold.abs().max()))
        import approx_ops
        with pytest.raises(RuntimeError, match="grad_scale needs float32"):
            approx_ops.approx_gemm_backward(g, a.detach().to(torch.uint8), b.detach().to(torch.uint8), torch.empty_like(a),
                                            torch.empty_like(b), saved[1], saved[2], grad_scale=0.5)
    finally:
        P.lut_appmult, P.lut_grad_a, P.lut_grad_b = saved


def test_baseline_op_uses_dense_ste_gradients(ops):
    self_ops, P = ops
    print("baseline op", flush=True)
    a = torch.randint(0, 128, (50, 30), device="cuda").float().requires_grad_()
    b = torch.randint(0, 128, (30, 20), device="cuda").float().requires_grad_()
    out = self_ops.approx_gemm_baseline_op(a, b)
    ref = self_ops.approx_gemm_op(a.detach(), b.detach())
    assert torch.equal(out, ref)
    g = torch.randn(50, 20, device="cuda")
    out.backward(g)
    # dense fp32 matmuls; only the BLAS summation order may differ
    torch.testing.assert_close(a.grad, g @ b.detach().t(), rtol=1e-5, atol=1e-3)
    torch.testing.assert_close(b.grad, a.detach().t() @ g, rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("stride,padding,dilation,k", [(1, 1, 1, 3), (2, 1, 1, 3), (1, 0, 1, 1), (2, 0, 1, 1), (1, 2, 2, 3)])
def test_conv_op_equals_conv2d_with_exact_multiplier(ops, oracle, stride, padding, dilation, k):
    self_ops, P = ops
    print("conv op", stride, padding, dilation, k, flush=True)
    keep = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
    try:
        n = np.arange(128)
        Sx, Sy = oracle.ste_tables16(7)
        P.set_lookup_tables("cuda", oracle.pack_table(n[:, None] * n[None, :], 7, np.uint16),
                            oracle.pack_table(Sx, 7, np.int16), oracle.pack_table(Sy, 7, np.int16))
        x = torch.randint(0, 128, (3, 5, 10, 10), device="cuda").float().requires_grad_()
        w = torch.randint(0, 128, (7, 5, k, k), device="cuda").float().requires_grad_()
        args = dict(bias=None, stride=(stride, stride), padding=(padding, padding), dilation=(dilation, dilation), groups=1)
        y = self_ops.approx_conv2d_op(x, w, **args)
        x2, w2 = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
        y2 = F.conv2d(x2, w2, **args)
        assert torch.equal(y, y2)                                    # integers < 2^24: exact in fp32
        g = torch.randint(-2, 3, y.shape, device="cuda").float()
        y.backward(g)
        y2.backward(g)
        assert torch.equal(x.grad, x2.grad) and torch.equal(w.grad, w2.grad)
        yb = self_ops.approx_conv2d_baseline_op(x.detach(), w.detach(), **args)
        assert torch.equal(yb, y2.detach())
    finally:
        P.lut_appmult, P.lut_grad_a, P.lut_grad_b = keep


def test_conv_op_against_oracle_with_shipped_table(ops, oracle, golden_dir):
    self_ops, P = ops
    print("conv oracle", flush=True)
    fwd, _, _ = oracle.parse_lut_file(os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), 7)
    rng = np.random.default_rng(3)
    x = rng.integers(0, 128, (2, 4, 8, 8)).astype(np.uint8)
    w = rng.integers(0, 128, (6, 4, 3, 3)).astype(np.uint8)
    y = self_ops.approx_conv2d_op(torch.tensor(x, device="cuda").float(), torch.tensor(w, device="cuda").float(), None,
                                  (1, 1), (1, 1), (1, 1), 1)
    want = oracle.conv2d_lut_np(x, w, fwd, 1, 1, 1)     # padding pixels are code 0 and LUT[0][w] != 0 for this table
    assert (y.cpu().numpy() == want.astype(np.float32)).all()


@pytest.mark.parametrize("shape,k,stride,padding,dilation", [
    ((3, 5, 10, 10), 3, 1, 1, 1),      # K = 45: byte stores
    ((2, 4, 9, 7), 3, 2, 1, 1),        # K = 36, odd image, M not a multiple of 64
    ((2, 8, 12, 12), 1, 2, 0, 1),      # 1x1 stride-2 downsample
    ((1, 3, 16, 16), 7, 2, 3, 1),      # stem-like 7x7
    ((2, 6, 11, 11), 3, 1, 2, 2),      # dilation
    ((1, 130, 6, 6), 3, 1, 1, 1),      # K = 1170 > one 512-column tile, not a multiple of 4
    ((2, 64, 8, 8), 3, 1, 1, 1),       # K = 576: two column tiles, 32-bit stores
])
def test_im2col_codes_against_oracle(ops, oracle, shape, k, stride, padding, dilation):
    import approx_ops
    print("im2col", shape, k, stride, padding, dilation, flush=True)
    rng = np.random.default_rng(11)
    x = rng.integers(0, 256, shape).astype(np.uint8)
    want, oh, ow = oracle.im2col_np(x, k, k, stride, padding, dilation)
    a = torch.full(want.shape, 77, dtype=torch.uint8, device="cuda")
    approx_ops.im2col_codes(torch.tensor(x, device="cuda").float(), a, (k, k), stride, padding, dilation)
    assert (a.cpu().numpy() == want).all()
    # the same matrix the reference's pad + unfold + transpose + reshape + cast produces
    xt = torch.tensor(x, device="cuda").float()
    cols = F.unfold(F.pad(xt, (padding,) * 4), kernel_size=(k, k), dilation=dilation, stride=stride)
    assert torch.equal(a, cols.transpose(1, 2).reshape(-1, want.shape[1]).to(torch.uint8))


@pytest.mark.parametrize("shape,k,stride,padding,dilation", [
    ((3, 5, 10, 10), 3, 1, 1, 1), ((2, 4, 9, 7), 3, 2, 1, 1), ((2, 8, 12, 12), 1, 2, 0, 1), ((1, 3, 16, 16), 7, 2, 3, 1),
    ((2, 6, 11, 11), 3, 1, 2, 2), ((2, 64, 8, 8), 3, 1, 1, 1), ((4, 16, 32, 32), 3, 1, 1, 1)])
def test_col2im_equals_fold(ops, shape, k, stride, padding, dilation):
    import approx_ops
    print("col2im", shape, k, stride, padding, dilation, flush=True)
    Bn, C, H, W = shape
    oh = (H + 2 * padding - dilation * (k - 1) - 1) // stride + 1
    ow = (W + 2 * padding - dilation * (k - 1) - 1) // stride + 1
    g = torch.Generator(device="cuda").manual_seed(1)
    cols = torch.randn(Bn, C * k * k, oh * ow, device="cuda", generator=g)
    x = torch.full(shape, float("nan"), device="cuda")
    approx_ops.col2im(cols, x, (k, k), stride, padding, dilation)
    want = F.fold(cols.double(), (H, W), (k, k), dilation=dilation, padding=padding, stride=stride)
    torch.testing.assert_close(x.double(), want, rtol=0, atol=1e-6 * float(want.abs().max()))
    # integer-valued windows: every order of the sums gives the same bits
    ci = torch.randint(-8, 9, cols.shape, device="cuda", generator=g).float()
    approx_ops.col2im(ci, x, (k, k), stride, padding, dilation)
    assert torch.equal(x, F.fold(ci, (H, W), (k, k), dilation=dilation, padding=padding, stride=stride))


def test_im2col_codes_rejects_wrong_shapes(ops):
    import approx_ops
    x = torch.zeros(2, 3, 8, 8, device="cuda")
    with pytest.raises(RuntimeError, match="a_tensor's shape should be 128 x 27"):
        approx_ops.im2col_codes(x, torch.zeros(128, 28, dtype=torch.uint8, device="cuda"), (3, 3), 1, 1, 1)
    with pytest.raises(RuntimeError, match="x_tensor must be of type"):
        approx_ops.im2col_codes(x.half(), torch.zeros(128, 27, dtype=torch.uint8, device="cuda"), (3, 3), 1, 1, 1)
    with pytest.raises(RuntimeError, match="empty convolution output"):
        approx_ops.im2col_codes(x, torch.zeros(0, 3 * 81, dtype=torch.uint8, device="cuda"), (9, 9), 1, 0, 1)


@pytest.mark.parametrize("M,K,N,L", [(192, 40, 24, 64), (150, 33, 10, 25), (4096, 64, 64, 1024), (6, 5, 3, 1),
                                     # expanded-table gradA: 16 k per workgroup; 32 k per workgroup with images of 64, 16 and 4
                                     # rows, the last with a ragged row block; images of 2 rows (no 16-byte stores)
                                     (8192, 32, 32, 1024), (9216, 48, 64, 256), (32768, 128, 32, 64), (32768, 128, 64, 16),
                                     (33012, 128, 32, 4), (33010, 128, 32, 2), (4100, 32, 64, 4)])
def test_backward_image_major_ga_equals_row_major(ops, oracle, golden_dir, M, K, N, L):
    import approx_ops
    self_ops, P = ops
    print("gA layout", M, K, N, L, flush=True)
    rng = np.random.default_rng(5)
    a = torch.tensor(rng.integers(0, 128, (M, K)).astype(np.uint8), device="cuda")
    b = torch.tensor(rng.integers(0, 128, (K, N)).astype(np.uint8), device="cuda")
    g = torch.tensor(rng.standard_normal((M, N)).astype(np.float32), device="cuda")
    ga, gb = torch.empty(M, K, device="cuda"), torch.empty(K, N, device="cuda")
    approx_ops.approx_gemm_backward(g, a, b, ga, gb, P.lut_grad_a, P.lut_grad_b)
    ga_t, gb2 = torch.full((M // L, K, L), float("nan"), device="cuda"), torch.empty(K, N, device="cuda")
    approx_ops.approx_gemm_backward(g, a, b, ga_t, gb2, P.lut_grad_a, P.lut_grad_b, ga_rows_per_image=L)
    assert torch.equal(ga_t, ga.view(M // L, L, K).transpose(1, 2))      # same sums, other addresses
    assert torch.equal(gb2, gb)
    with pytest.raises(RuntimeError, match="must divide"):
        approx_ops.approx_gemm_backward(g, a, b, ga_t, gb2, P.lut_grad_a, P.lut_grad_b, ga_rows_per_image=M + 1)


@pytest.mark.parametrize("shape,cout,k,stride,padding,dilation", [
    ((4, 16, 12, 12), 24, 3, 1, 1, 1), ((3, 8, 9, 9), 5, 3, 2, 1, 1), ((2, 12, 8, 8), 16, 1, 2, 0, 1),
    ((2, 6, 10, 10), 7, 3, 1, 2, 2), ((64, 16, 8, 8), 64, 3, 1, 1, 1)])
def test_conv_op_matches_reference_composition(ops, oracle, golden_dir, shape, cout, k, stride, padding, dilation):
    """The one-pass convolution against pad + unfold + transpose + GEMM op, the composition the reference uses
    (approx_ops.py:545-571), forward and both gradients, and against the float64 oracle."""
    self_ops, P = ops
    print("conv fused", shape, cout, k, stride, padding, dilation, flush=True)
    fwd, ga, gb = oracle.parse_lut_file(os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), 7)
    rng = np.random.default_rng(9)
    xn = rng.integers(0, 128, shape).astype(np.uint8)
    wn = rng.integers(0, 128, (cout, shape[1], k, k)).astype(np.uint8)
    args = (None, (stride, stride), (padding, padding), (dilation, dilation), 1)
    x = torch.tensor(xn, device="cuda").float().requires_grad_()
    w = torch.tensor(wn, device="cuda").float().requires_grad_()
    x2, w2 = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    y = self_ops.approx_conv2d_op(x, w, *args)
    y2 = P.approx_conv2d_unfold_op(x2, w2, *args)
    assert torch.equal(y, y2) and y.stride() == y2.stride()
    g = torch.randn(y.shape, device="cuda")
    y.backward(g)
    y2.backward(g)
    assert torch.equal(w.grad, w2.grad)
    # fold adds the same per-window terms in a different order than the transposed copy + fold does: not bitwise
    torch.testing.assert_close(x.grad, x2.grad, rtol=0, atol=1e-5 * float(x2.grad.abs().max()))
    if np.prod(shape) <= 4096:
        cols, oh, ow = oracle.im2col_np(xn, k, k, stride, padding, dilation)
        gc = g.permute(0, 2, 3, 1).reshape(-1, cout).cpu().numpy()
        a64, b64 = oracle.backward_np(gc, cols, wn.reshape(cout, -1).T, ga, gb)
        np.testing.assert_allclose(w.grad.reshape(cout, -1).t().cpu().numpy(), b64, rtol=0, atol=1e-5 * np.abs(b64).max())
        gx = F.fold(torch.tensor(a64, dtype=torch.float64).view(shape[0], oh * ow, -1).transpose(1, 2), shape[2:], (k, k),
                    dilation=dilation, padding=padding, stride=stride).numpy()
        np.testing.assert_allclose(x.grad.cpu().numpy(), gx, rtol=0, atol=1e-5 * np.abs(gx).max())
    # straight-through variant: same forward, gradients of the exact convolution of the codes
    xb, wb = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    xb2, wb2 = x.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    yb = self_ops.approx_conv2d_baseline_op(xb, wb, *args)
    yb2 = P.approx_conv2d_baseline_unfold_op(xb2, wb2, *args)
    assert torch.equal(yb, y2)
    yb.backward(g)
    yb2.backward(g)
    torch.testing.assert_close(xb.grad, xb2.grad, rtol=1e-4, atol=1e-4 * float(xb2.grad.abs().max()))
    torch.testing.assert_close(wb.grad, wb2.grad, rtol=1e-4, atol=1e-4 * float(wb2.grad.abs().max()))


def test_conv_op_skips_the_gradient_nobody_needs(ops):
    """Images in front of the first layer need no gradient: only the weight gradient is computed then (and equals
    the one computed together with the input gradient)."""
    self_ops, P = ops
    x = torch.randint(0, 128, (4, 3, 12, 12), device="cuda").float()
    w = torch.randint(0, 128, (8, 3, 3, 3), device="cuda").float().requires_grad_()
    args = (None, (1, 1), (1, 1), (1, 1), 1)
    g = torch.randn(4, 8, 12, 12, device="cuda")
    self_ops.approx_conv2d_op(x, w, *args).backward(g)
    x2, w2 = x.clone().requires_grad_(), w.detach().clone().requires_grad_()
    self_ops.approx_conv2d_op(x2, w2, *args).backward(g)
    assert torch.equal(w.grad, w2.grad) and x2.grad is not None
    w3 = w.detach().clone()
    x3 = x.clone().requires_grad_()
    self_ops.approx_conv2d_op(x3, w3, *args).backward(g)
    assert torch.equal(x3.grad, x2.grad)


def test_conv_op_rejects_bias_and_groups(ops):
    self_ops, P = ops
    x, w = torch.zeros(1, 2, 4, 4, device="cuda"), torch.zeros(2, 2, 3, 3, device="cuda")
    with pytest.raises(AssertionError, match="bias is not supported"):
        self_ops.approx_conv2d_op(x, w, torch.zeros(2, device="cuda"), (1, 1), (1, 1), (1, 1), 1)
    with pytest.raises(AssertionError, match="groups is not supported"):
        self_ops.approx_conv2d_op(x, w, None, (1, 1), (1, 1), (1, 1), 2)


@pytest.mark.parametrize("shape", [(7,), (4, 3, 5, 5), (64, 16, 32, 32), (1023,), (2, 1026)])
def test_fused_quantiser_equals_torch_expression(ops, shape):
    """The one-pass quantiser against the operator chain the reference composes (app_layers.py:147-160):
    bit-identical codes and gradients, including values that land exactly on .5 and outside the range."""
    import app_layers
    print("quantiser", shape, flush=True)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = (torch.randn(shape, device="cuda", generator=g) * 3).requires_grad_()
    with torch.no_grad():
        x.view(-1)[::5] = (torch.arange(x.numel(), device="cuda")[::5] % 200 - 30).float() * 0.05 + 0.025   # ties after scaling
        # non-finite inputs: torch.clamp hands a NaN on, and q - q.detach() + round(q) makes a NaN of an infinite q
        x.view(-1)[1], x.view(-1)[x.numel() // 2], x.view(-1)[-2] = float("nan"), float("inf"), float("-inf")
    scale, zp = torch.tensor([0.05], device="cuda"), torch.tensor([-17.0], device="cuda")
    x2 = x.detach().clone().requires_grad_()
    y = app_layers._to_codes(x, scale, zp, 127.0)
    y2 = app_layers._to_codes_torch(x2, scale, zp, 127.0)
    assert torch.equal(torch.isnan(y), torch.isnan(y2)) and int(torch.isnan(y).sum()) == 3
    assert torch.equal(torch.nan_to_num(y, nan=-1.0), torch.nan_to_num(y2, nan=-1.0))
    assert torch.nan_to_num(y, nan=0.0).min() >= 0 and torch.nan_to_num(y, nan=0.0).max() <= 127
    gy = torch.randn(shape, device="cuda", generator=g)
    y.backward(gy)
    y2.backward(gy)
    assert torch.equal(torch.nan_to_num(x.grad, nan=-7.0), torch.nan_to_num(x2.grad, nan=-7.0))
    assert (x.grad == 0).any() and (x.grad != 0).any()
    # non-contiguous input
    if len(shape) == 4:
        xt = x.detach().transpose(1, 3)
        assert torch.equal(torch.nan_to_num(app_layers._to_codes(xt, scale, zp, 127.0), nan=-1.0),
                           torch.nan_to_num(app_layers._to_codes_torch(xt, scale, zp, 127.0), nan=-1.0))


def test_acc_gemm_op(ops):
    self_ops, P = ops
    a = torch.randn(70, 40, device="cuda", requires_grad=True)
    b = torch.randn(40, 30, device="cuda", requires_grad=True)
    y = P.acc_gemm_op(a, b)
    torch.testing.assert_close(y, a @ b, rtol=1e-4, atol=1e-4)
    y.sum().backward()
    torch.testing.assert_close(a.grad, torch.ones(70, 30, device="cuda") @ b.detach().t())


def test_approx_conv_layer_equals_fake_quant_conv_with_exact_multiplier(ops, oracle):
    """With the exact-multiplier table the four-term expression of ApproxConv2d is the convolution of
    the fake-quantised tensors (reference app_layers.py:175-183), up to fp32 rounding."""
    import app_layers as L
    self_ops, P = ops
    print("layer exact", flush=True)
    keep = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
    try:
        n = np.arange(128)
        Sx, Sy = oracle.ste_tables16(7)
        P.set_lookup_tables("cuda", oracle.pack_table(n[:, None] * n[None, :], 7, np.uint16),
                            oracle.pack_table(Sx, 7, np.int16), oracle.pack_table(Sy, 7, np.int16))
        torch.manual_seed(0)
        layer = L.ApproxConv2d(5, 7, 3, stride=1, padding=1, bias=True, a_bits=7, w_bits=7).cuda().train()
        x = torch.randn(4, 5, 12, 12, device="cuda", requires_grad=True)
        y = layer(x)
        s_a, z_a, s_w, z_w = layer.activation_scale, layer.activation_zp_neg, layer.weight_scale, layer.weight_zp_neg
        xq = (L._to_codes(x.detach(), s_a, z_a, 127.0) + z_a) * s_a
        wq = (L._to_codes(layer.weight.detach(), s_w, z_w, 127.0) + z_w) * s_w
        # a padding pixel contributes 0 to each of the four terms (code 0 times anything is 0 for the exact
        # multiplier; the zero-point convolutions are zero padded), i.e. it is a real zero
        ref = F.conv2d(xq, wq, layer.bias, padding=1)
        torch.testing.assert_close(y, ref, rtol=1e-4, atol=1e-4)
        y.square().mean().backward()
        assert x.grad is not None and layer.weight.grad is not None and torch.isfinite(layer.weight.grad).all()
        # the factorised zero-point terms equal the reference's three full convolutions, values and gradients
        layer.eval()                                   # freeze the observers: both forms see the same scales
        grads = []
        outs = []
        for fused, literal in ((True, False), (False, False), (False, True)):   # one-pass kernel, torch operators, literal
            x.grad = None
            layer.weight.grad = None
            layer.bias.grad = None
            layer.fused_dequant, layer.reference_zero_point_terms = fused, literal
            out = layer(x)
            out.square().mean().backward()
            outs.append(out.detach())
            grads.append((x.grad.clone(), layer.weight.grad.clone(), layer.bias.grad.clone()))
        assert outs[0].is_contiguous()
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])   # integer-valued terms below 2^24: bit-identical
        for k in (1, 2):
            for a, b in zip(grads[0], grads[k]):
                torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)
    finally:
        P.lut_appmult, P.lut_grad_a, P.lut_grad_b = keep


def test_two_training_forwards_before_one_backward_keep_their_own_scales(ops):
    """A layer called twice in training mode before backward (shared layer, two-view losses): the second call moves the
    observers, and the graph of the first call must still use the scale and zero point it was built with -- the reference
    binds new tensors on every forward (app_layers.py:154-160).  Checked against the same computation with every
    quantisation step written in torch operators."""
    import app_layers as L
    print("two forwards, one backward", flush=True)
    torch.manual_seed(3)
    fused = L.ApproxConv2d(5, 12, 3, padding=1, bias=True, a_bits=7, w_bits=7).cuda().train()
    plain = L.ApproxConv2d(5, 12, 3, padding=1, bias=True, a_bits=7, w_bits=7).cuda().train()
    plain.load_state_dict(fused.state_dict())
    plain.fused_dequant = False
    plain.quantize_v2 = lambda x, s, z, q: L._to_codes_torch(x, s, z, q)       # torch operators all the way
    plain.activation_observer.fused_mode = None
    plain.weight_observer.fused_mode = None
    x1 = torch.randn(4, 5, 9, 9, device="cuda")
    x2 = torch.randn(4, 5, 9, 9, device="cuda") * 3 + 1                        # a different range: the second call moves the scale
    res = []
    for layer in (fused, plain):
        a, b = x1.clone().requires_grad_(), x2.clone().requires_grad_()
        y1 = layer(a)
        s_first = layer.activation_scale.clone()
        y2 = layer(b)
        assert not torch.equal(layer.activation_scale, s_first)
        (y1.square().mean() + y2.square().mean()).backward()
        res.append((y1.detach(), y2.detach(), a.grad, b.grad, layer.weight.grad, layer.bias.grad))
    for u, v in zip(*res):
        torch.testing.assert_close(u, v, rtol=1e-4, atol=1e-6 * float(v.abs().max()) + 1e-12)


def test_synthetic_training_steps_reduce_loss(ops, golden_dir):
    """prepare -> calibrate -> a few optimiser steps of a small quantised net on one fixed batch."""
    import app_layers as L
    import app_train as T
    print("train steps", flush=True)
    torch.manual_seed(1)
    net = torch.nn.Sequential(torch.nn.Conv2d(3, 8, 3, padding=1, bias=False), torch.nn.BatchNorm2d(8), torch.nn.ReLU(),
                              torch.nn.Conv2d(8, 16, 3, stride=2, padding=1, bias=False), torch.nn.BatchNorm2d(16), torch.nn.ReLU(),
                              torch.nn.AdaptiveAvgPool2d(1), torch.nn.Flatten(), torch.nn.Linear(16, 10)).cuda()
    net = L.prepare(net, inplace=True, a_bits=7, w_bits=7)
    xs, ys = T.synthetic_batches(1, 64, torch.device("cuda"))
    T.calibrate(net, xs)
    opt = torch.optim.Adam(net.parameters(), lr=1e-2)
    losses = [float(l) for l in T.train_steps(net, opt, xs * 12, ys * 12)]
    assert all(np.isfinite(losses)) and losses[-1] < losses[0]


def test_resnet18_batch512_training_step_expanded_kernels_agree_with_direct_kernels(ops):
    """The training-step configuration (ResNet-18, batch 512, SGD, the shipped 7-bit table with its gradient tables): one
    step -- forward, cross-entropy, backward, update -- of the same model state on the same batch, once with the library's own
    kernel selection and once with the direct gather kernels only (the formulation the oracle tests pin shape by shape).
    The forward pass is integer arithmetic, so the logits are bit-identical; every parameter gradient agrees norm-wise to
    1e-5 (the two differ in summation order only, through 20 layers of backward)."""
    import copy
    import approx_ops
    import app_train as T
    print("resnet18 batch 512 step", flush=True)
    dev = torch.device("cuda")
    torch.manual_seed(7)
    base = T.build_model("resnet18", 7, False, dev)
    xs, ys = T.synthetic_batches(2, 512, dev, seed=3)
    T.calibrate(base, xs[:1])
    results = []
    for mode in (1, 0):
        model = copy.deepcopy(base)
        opt = torch.optim.SGD(model.parameters(), lr=1e-2, momentum=0.9)
        prev = approx_ops._lib.amr_set_expanded_table_kernels(mode)
        try:
            model.train()
            opt.zero_grad()
            logits = model(xs[1])
            loss = torch.nn.functional.cross_entropy(logits, ys[1])
            loss.backward()
            grads = {n: p.grad.detach().clone() for n, p in model.named_parameters()}
            opt.step()
            torch.cuda.synchronize()
        finally:
            approx_ops._lib.amr_set_expanded_table_kernels(prev)
        results.append((logits.detach(), grads, {n: p.detach().clone() for n, p in model.named_parameters()}))
    (l1, g1, p1), (l0, g0, p0) = results
    assert torch.equal(l1, l0) and bool(torch.isfinite(l1).all())
    assert len(g1) > 60
    for n in g0:
        ref = g0[n].double()
        assert float((g1[n].double() - ref).norm()) <= 1e-5 * float(ref.norm()) + 1e-30, n
        assert float(ref.norm()) > 0, n
        assert float((p1[n].double() - p0[n].double()).norm()) <= 1e-5 * float(p0[n].double().norm()) + 1e-30, n


def test_training_harness_cli_with_float_gradient_tables(ops, golden_dir, tmp_path, capsys):
    """The command-line harness end to end on a small batch, with the file's int16 tables and with float32 slopes."""
    import gzip
    import shutil
    import app_train as T
    from self_ops.ops_py import approx_ops as P
    print("train harness cli", flush=True)
    lut = tmp_path / "lut7.txt"
    with gzip.open(os.path.join(golden_dir, "lut7_resub_63_bp8.txt.gz"), "rb") as f, open(lut, "wb") as o:
        shutil.copyfileobj(f, o)
    saved = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
    try:
        for extra, dtype in ([], torch.int16), (["--float-grad-window", "8"], torch.float32):
            T.main(["--lut", str(lut), "--bits", "7", "--batch", "32", "--steps", "2", "--optimizer", "sgd"] + extra)
            assert P.lut_grad_a.dtype == dtype
            out = capsys.readouterr().out
            assert "img/s" in out and "nan" not in out.lower()
    finally:
        P.lut_appmult, P.lut_grad_a, P.lut_grad_b = saved


def test_approx_linear_equals_fake_quant_linear_with_exact_multiplier(ops, oracle):
    """With LUT[a][b] = a*b the table classifier computes the same function as the fake-quantised one (the reference's
    QuantLinear, app_layers.py:101-111), values and gradients, up to fp32 rounding of the scaling."""
    import app_layers
    self_ops, P = ops
    keep = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
    try:
        n = np.arange(128)
        Sx, Sy = oracle.ste_tables16(7)
        P.set_lookup_tables("cuda", oracle.pack_table(n[:, None] * n[None, :], 7, np.uint16),
                            oracle.pack_table(Sx, 7, np.int16), oracle.pack_table(Sy, 7, np.int16))
        torch.manual_seed(0)
        ref = app_layers.QuantLinear(96, 10, bias=True, a_bits=7, w_bits=7).cuda()
        lin = app_layers.ApproxLinear(96, 10, bias=True, a_bits=7, w_bits=7).cuda()
        lin.load_state_dict(ref.state_dict())
        x = torch.randn(33, 96, device="cuda")
        x1, x2 = x.clone().requires_grad_(), x.clone().requires_grad_()
        ref.train(); lin.train()
        y1, y2 = ref(x1), lin(x2)
        torch.testing.assert_close(y2, y1, rtol=1e-4, atol=1e-4 * float(y1.detach().abs().max()))
        g = torch.randn_like(y1)
        y1.backward(g); y2.backward(g)
        torch.testing.assert_close(x2.grad, x1.grad, rtol=1e-3, atol=1e-4 * float(x1.grad.abs().max()))
        torch.testing.assert_close(lin.weight.grad, ref.weight.grad, rtol=1e-3, atol=1e-4 * float(ref.weight.grad.abs().max()))
        torch.testing.assert_close(lin.bias.grad, ref.bias.grad)
        net = app_layers.prepare(torch.nn.Sequential(torch.nn.Linear(8, 4)), a_bits=7, w_bits=7, approx_linear=True)
        assert isinstance(net[0], app_layers.ApproxLinear)
    finally:
        P.lut_appmult, P.lut_grad_a, P.lut_grad_b = keep


@pytest.mark.parametrize("cin,cout,k,stride,padding,hw,bias", [(6, 40, 3, 2, 1, 9, True), (16, 33, 1, 2, 0, 8, False), (3, 64, 3, 1, 1, 32, True)])
def test_one_pass_dequantisation_equals_torch_operators(ops, golden_dir, cin, cout, k, stride, padding, hw, bias):
    """ApproxConv2d with the shipped table: zero-point terms and scaling in one pass (contiguous NCHW result) against the
    same expression in torch operators, on shapes whose channel and position counts are no multiples of the 32 x 32 tile."""
    import app_layers as L
    print("dequant", cin, cout, k, stride, padding, hw, bias, flush=True)
    torch.manual_seed(1)
    layer = L.ApproxConv2d(cin, cout, k, stride=stride, padding=padding, bias=bias, a_bits=7, w_bits=7).cuda().train()
    x = torch.randn(5, cin, hw, hw, device="cuda", requires_grad=True)
    layer(x)                                        # observers see data once
    layer.eval()
    res = []
    for fused in (True, False):
        layer.fused_dequant = fused
        layer.zero_grad()
        x.grad = None
        y = layer(x)
        y.square().mean().backward()
        res.append((y.detach(), x.grad.clone(), layer.weight.grad.clone(), None if not bias else layer.bias.grad.clone()))
    assert res[0][0].is_contiguous() and torch.equal(res[0][0], res[1][0])
    for a, b in zip(res[0][1:], res[1][1:]):
        if a is not None:
            torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-6 * float(b.abs().max()) + 1e-12)


@pytest.mark.parametrize("qmax_on_device", [False, True])
@pytest.mark.parametrize("kind", ["ema", "extremes"])
def test_one_launch_observer_update_equals_tensor_expressions(ops, kind, qmax_on_device):
    """Range tracking + scale + zero point in one launch against the reference's tensor expressions
    (app_layers.py:21-53, :154-160) over several batches: the same bits in every buffer."""
    import app_layers as L
    make = (lambda: L.MovingAverageMinMaxObserver("L", None)) if kind == "ema" else (lambda: L.MinMaxObserver("L", None))
    fused, plain = make().cuda(), make().cuda()
    plain.fused_mode = None                                   # tensor expressions
    qmax, eps = torch.tensor(127.0), torch.tensor(torch.finfo(torch.float32).eps)
    if qmax_on_device:                                        # the pooling quantisers hold it as a device buffer: true division
        qmax, eps = qmax.cuda(), eps.cuda()
    sc, zp = torch.ones(1, device="cuda"), torch.zeros(1, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(4)
    for step in range(6):
        x = torch.randn(64, 33, device="cuda", generator=g) * (1 + step) + 0.3 * step
        s1, z1 = L._observe(fused, x, qmax, eps, sc, zp)
        s2, z2 = L._observe(plain, x, qmax, eps, None, None)
        assert s1.data_ptr() != sc.data_ptr() and float(sc) == 1.0 and float(zp) == 0.0   # new tensors: graphs of earlier passes keep theirs
        assert torch.equal(s1.reshape(1), s2.reshape(1)) and torch.equal(z1.reshape(1), z2.reshape(1)), step
        assert torch.equal(fused.min_val.reshape(1), plain.min_val.reshape(1)) and torch.equal(fused.max_val.reshape(1), plain.max_val.reshape(1))
    # a NaN in the data reaches the range, the scale and the zero point, as it does through torch.min / torch.max
    x = torch.randn(40, device="cuda", generator=g)
    x[3] = float("nan")
    s1, z1 = L._observe(fused, x, qmax, eps, sc, zp)
    s2, z2 = L._observe(plain, x, qmax, eps, None, None)
    assert bool(torch.isnan(s1).all()) and bool(torch.isnan(s2).all()) and bool(torch.isnan(z1).all()) and bool(torch.isnan(z2).all())
    assert bool(torch.isnan(fused.min_val).all()) and bool(torch.isnan(plain.min_val).all())
    x = torch.zeros(8, device="cuda")                         # constant input: scale falls back to eps
    fused2, plain2 = make().cuda(), make().cuda()
    plain2.fused_mode = None
    s1, z1 = L._observe(fused2, x, qmax, eps, sc, zp)
    s2, z2 = L._observe(plain2, x, qmax, eps, None, None)
    assert torch.equal(s1.reshape(1), s2.reshape(1)) and torch.equal(z1.reshape(1), z2.reshape(1))


@pytest.mark.parametrize("n", [1, 5, 4097, 3 * 64 * 32 * 32 + 3, 33554432 + 17])
def test_one_launch_extremes_and_observer_update(ops, n):
    """amr_observe_minmax_f32 against torch.aminmax + the observer's tensor expressions: every workgroup count, ragged tails,
    unaligned data, a NaN in the last element, three calls in a row on one state (the last ticket puts the counter back)."""
    import approx_ops
    print("observe minmax", n, flush=True)
    g = torch.Generator(device="cuda").manual_seed(6)
    base = torch.randn(n + 1, device="cuda", generator=g)
    state = torch.zeros(approx_ops.MINMAX_STATE_WORDS, dtype=torch.int32, device="cuda")
    lo, hi, sc, zp = (torch.zeros(1, device="cuda") for _ in range(4))
    lo2, hi2, sc2, zp2 = (torch.zeros(1, device="cuda") for _ in range(4))
    eps = float(torch.finfo(torch.float32).eps)
    for call, (x, mode) in enumerate(((base[:n], 0), (base[1:] * 3 - 1, 2), (base[:n] * 0.5 + 2, 1))):
        x = x if call != 1 else x.clone()[:n]                     # (call 0: 16-byte aligned view; call 1: a fresh tensor)
        if call == 0 and n > 1:
            x = base[1:n + 1]                                     # 4-byte aligned only
        approx_ops.observe_minmax(x.contiguous(), state, lo, hi, sc, zp, mode, 0.1, 127.0, eps)
        want_lo, want_hi = torch.aminmax(x)
        approx_ops.observer_update(want_lo.reshape(1), want_hi.reshape(1), lo2, hi2, sc2, zp2, mode, 0.1, 127.0, eps)
        for a, b in ((lo, lo2), (hi, hi2), (sc, sc2), (zp, zp2)):
            assert torch.equal(a, b), (call, float(a), float(b))
        assert int(state[0]) == 0
    x = base[:n].clone()
    x[-1] = float("nan")
    approx_ops.observe_minmax(x, state, lo, hi, sc, zp, 0, 0.1, 127.0, eps)
    assert all(bool(torch.isnan(t).all()) for t in (lo, hi, sc, zp)) and int(state[0]) == 0


def test_bench_captured_codes_cover_every_benchmark_layer(ops):
    """bench.py --codes captured: one forward pass of the package's ResNet-18 yields operand codes for each of the 12
    benchmark GEMM shapes (here at batch 4), uint8 below 2^7, and post-ReLU activations pile up on one code."""
    import bench
    _, P = ops
    print("captured codes", flush=True)
    tables = tuple(t.cpu().numpy() for t in (P.lut_appmult, P.lut_grad_a, P.lut_grad_b))
    seen = bench.capture_codes(torch, torch.device("cuda"), 7, tables, "resnet18", 4)
    for name, cnt, M, K, N in bench.RESNET18_B256:
        a, b = seen[(M // 64, K, N)]
        assert a.dtype == torch.uint8 and b.dtype == torch.uint8 and a.is_contiguous() and b.is_contiguous(), name
        assert int(a.max()) < 128 and int(b.max()) < 128, name
    a, _ = seen[(4096, 576, 64)]                      # conv2_x: its input went through a ReLU (and the padding adds zeros)
    assert float(torch.bincount(a.flatten().int(), minlength=128).max()) / a.numel() > 0.25
