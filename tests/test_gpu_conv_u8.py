"""GPU tests of the quantised LUT convolution on uint8 codes: the pixel-major quantiser, the tap-major im2col, the fused
input-gradient pass, the output-gradient pass with row sums and the layer operator built from them, each against the
unfused composition (float32 code tensors and torch operators) and against the CPU oracle."""
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


def out_size(h, w, k, s, p, d):
    return (h + 2 * p - d * (k - 1) - 1) // s + 1, (w + 2 * p - d * (k - 1) - 1) // s + 1


@pytest.mark.parametrize("shape", [(4, 3, 5, 5), (2, 16, 8, 8), (3, 64, 32, 32), (2, 528, 4, 4), (1, 20, 3, 7), (130, 32, 1, 1)])
def test_pixel_major_quantiser_equals_float_quantiser(ops, shape):
    """Codes, in-range mask and channel sums of the uint8 quantiser against the float32 quantiser and its backward
    (themselves pinned against the torch expression of the reference's quantize_v2): same codes at every element, the mask
    is where the straight-through gradient passes, the sums are the codes added over the channels."""
    import app_layers
    import approx_ops
    print("quantiser nhwc", shape, flush=True)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(shape, device="cuda", generator=g) * 3
    x.view(-1)[::5] = (torch.arange(x.numel(), device="cuda")[::5] % 200 - 30).float() * 0.05 + 0.025      # ties after scaling
    x.view(-1)[1], x.view(-1)[x.numel() // 2], x.view(-1)[-2] = float("nan"), float("inf"), float("-inf")
    scale, zp = torch.tensor([0.05], device="cuda"), torch.tensor([-17.0], device="cuda")
    bn, c, h, w = shape
    codes = torch.full((bn * h * w, c), 255, dtype=torch.uint8, device="cuda")
    inside = torch.full(shape, 7, dtype=torch.uint8, device="cuda")
    xs = torch.full((bn * h * w,), float("nan"), device="cuda")
    approx_ops.quantize_codes_nhwc(x, scale, zp, 127.0, codes, inside, xs)
    xr = x.clone().requires_grad_()
    want = app_layers._to_codes(xr, scale, zp, 127.0)
    want.backward(torch.ones_like(want))
    finite = ~torch.isnan(want.detach())
    want_u8 = torch.where(finite, want.detach(), torch.zeros_like(want)).to(torch.uint8)       # a NaN: code 0 (documented)
    got = codes.view(bn, h, w, c).permute(0, 3, 1, 2)
    assert torch.equal(got, want_u8)
    passes = torch.nan_to_num(xr.grad, nan=0.0) != 0
    assert torch.equal(inside.bool(), passes)
    assert int((~finite).sum()) == 3 and not inside.bool()[~finite].any()
    assert torch.equal(xs.view(bn, h, w), want_u8.float().sum(dim=1))


@pytest.mark.parametrize("shape,k,stride,padding,dilation", [
    ((3, 5, 10, 10), 3, 1, 1, 1), ((2, 4, 9, 7), 3, 2, 1, 1), ((2, 16, 12, 12), 1, 2, 0, 1), ((1, 3, 16, 16), 7, 2, 3, 1),
    ((2, 6, 11, 11), 3, 1, 2, 2), ((2, 64, 8, 8), 3, 1, 1, 1), ((3, 32, 16, 16), 3, 2, 1, 1), ((2, 48, 5, 5), 1, 1, 0, 1)])
def test_tap_major_im2col_against_oracle(ops, oracle, shape, k, stride, padding, dilation):
    """The uint8 im2col of pixel-major codes against the oracle's window matrix (reference column order c*kh*kw + tap),
    columns permuted to the tap-major order."""
    import approx_ops
    print("im2col nhwc", shape, k, stride, padding, dilation, flush=True)
    rng = np.random.default_rng(12)
    x = rng.integers(0, 256, shape).astype(np.uint8)
    bn, c, h, w = shape
    want, oh, ow = oracle.im2col_np(x, k, k, stride, padding, dilation)
    want = want.reshape(-1, c, k * k).transpose(0, 2, 1).reshape(-1, k * k * c)
    codes = torch.tensor(x, device="cuda").permute(0, 2, 3, 1).reshape(bn * h * w, c).contiguous()
    a = torch.full(want.shape, 77, dtype=torch.uint8, device="cuda")
    approx_ops.im2col_nhwc(codes, a, shape, (k, k), stride, padding, dilation)
    assert (a.cpu().numpy() == want).all()


@pytest.mark.parametrize("shape,k,stride,padding,dilation", [((200, 32, 61, 67), 3, 1, 1, 1), ((9, 3, 260, 300), 5, 1, 2, 1), ((300, 16, 131, 127), 3, 2, 1, 1)])
def test_tap_major_im2col_over_several_slabs_of_rows(ops, shape, k, stride, padding, dilation):
    """Window matrices of more than 2^22 pieces are written slab by slab (slab borders in the middle of an image line and of
    an image): against torch's unfold of the same codes, columns permuted to the tap-major order."""
    import approx_ops
    print("im2col nhwc, several slabs", shape, k, stride, padding, dilation, flush=True)
    bn, c, h, w = shape
    oh, ow = out_size(h, w, k, stride, padding, dilation)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randint(0, 256, shape, device="cuda", generator=g, dtype=torch.int32)
    pieces = bn * oh * ow * k * k * (c // 16 if c % 16 == 0 else c)
    assert pieces > 2 * (1 << 22)
    codes = x.permute(0, 2, 3, 1).reshape(bn * h * w, c).to(torch.uint8).contiguous()
    a = torch.full((bn * oh * ow, k * k * c), 77, dtype=torch.uint8, device="cuda")
    approx_ops.im2col_nhwc(codes, a, shape, (k, k), stride, padding, dilation)
    cols = F.unfold(x.float(), (k, k), dilation=dilation, padding=padding, stride=stride)          # [B, c*k*k, L]
    want = cols.view(bn, c, k * k, oh * ow).permute(0, 3, 2, 1).reshape(bn * oh * ow, k * k * c).to(torch.uint8)
    assert torch.equal(a, want)


@pytest.mark.parametrize("shape,k,stride,padding,dilation", [
    ((3, 5, 10, 10), 3, 1, 1, 1), ((2, 4, 9, 7), 3, 2, 1, 1), ((2, 8, 12, 12), 1, 2, 0, 1), ((1, 3, 16, 16), 7, 2, 3, 1),
    ((2, 6, 11, 11), 3, 1, 2, 2), ((2, 64, 8, 8), 3, 1, 1, 1), ((4, 16, 32, 32), 3, 1, 1, 1), ((2, 32, 6, 6), 1, 1, 0, 1),
    # stride 2 on even images: the kernel that owns the 2 x 2 pixels of an output position
    ((3, 5, 10, 6), 3, 2, 1, 1), ((2, 64, 32, 32), 3, 2, 1, 1), ((5, 7, 2, 2), 3, 2, 1, 1), ((3, 64, 32, 32), 1, 2, 0, 1),
    ((2, 3, 2, 4), 1, 2, 0, 1), ((2, 4, 8, 8), 3, 2, 1, 2)])
def test_fused_input_gradient_equals_fold_plus_torch_operators(ops, shape, k, stride, padding, dilation):
    """gx = inside ? (fold(cols) + z_w * fold of the row sums spread over the taps) / scale : 0 against torch's fold in
    float64; with cols = None the kernel finishes a tensor that already holds fold(cols)."""
    import approx_ops
    print("input gradient", shape, k, stride, padding, dilation, flush=True)
    bn, c, h, w = shape
    oh, ow = out_size(h, w, k, stride, padding, dilation)
    g = torch.Generator(device="cuda").manual_seed(2)
    cols_tap = torch.randn(bn, k * k * c, oh * ow, device="cuda", generator=g)               # tap-major k
    t = torch.randn(bn * oh * ow, device="cuda", generator=g)
    inside = (torch.rand(shape, device="cuda", generator=g) < 0.8).to(torch.uint8)
    zw, scale = torch.tensor([-61.0], device="cuda"), torch.tensor([0.037], device="cuda")
    gx = torch.full(shape, float("nan"), device="cuda")
    approx_ops.conv_input_grad(cols_tap, t, zw, inside, scale, gx, (k, k), stride, padding, dilation)
    cols_ref = cols_tap.view(bn, k * k, c, oh * ow).transpose(1, 2).reshape(bn, c * k * k, oh * ow).double()
    fold = lambda cc: F.fold(cc, (h, w), (k, k), dilation=dilation, padding=padding, stride=stride)
    t_cols = t.double().view(bn, 1, oh * ow).expand(bn, k * k, oh * ow)
    want = (fold(cols_ref) + zw.double() * fold(t_cols)) / scale.double() * inside.double()
    torch.testing.assert_close(gx.double(), want, rtol=0, atol=2e-6 * float(want.abs().max()))
    assert (gx[inside == 0] == 0).all()
    # finishing in place what a convolution-shaped gradA left
    raw = fold(cols_ref).float().contiguous()
    approx_ops.conv_input_grad(None, t, zw, inside, scale, raw, (k, k), stride, padding, dilation)
    torch.testing.assert_close(raw.double(), want, rtol=0, atol=2e-6 * float(want.abs().max()))


@pytest.mark.parametrize("bn,n,hw", [(3, 40, (5, 7)), (2, 64, (16, 16)), (130, 10, (1, 1)), (1, 33, (9, 9)), (4, 128, (8, 8))])
def test_output_gradient_rows_with_row_sums(ops, bn, n, hw):
    import approx_ops
    print("dequant backward rowsum", bn, n, hw, flush=True)
    g = torch.randn(bn, n, *hw, device="cuda")
    sa, sw = torch.tensor([0.031], device="cuda"), torch.tensor([0.0077], device="cuda")
    L = hw[0] * hw[1]
    rows = torch.full((bn * L, n), float("nan"), device="cuda")
    rows2 = torch.full((bn * L, n), float("nan"), device="cuda")
    t = torch.full((bn * L,), float("nan"), device="cuda")
    approx_ops.conv_dequant_backward_rowsum(g, sa, sw, rows, t)
    approx_ops.conv_dequant_backward(g, sa, sw, rows2)
    assert torch.equal(rows, rows2)
    assert torch.equal(rows, ((sa * sw) * g).permute(0, 2, 3, 1).reshape(bn * L, n))
    want = rows.double().sum(dim=1)
    torch.testing.assert_close(t.double(), want, rtol=0, atol=1e-6 * float(rows.abs().sum(dim=1).max()))


@pytest.mark.parametrize("cin,cout,k,stride,padding,dilation,hw,bias", [
    (16, 24, 3, 1, 1, 1, 12, True),        # 3x3 same-size convolution, 16-byte code runs
    (5, 7, 3, 1, 1, 1, 9, True),           # channel count that takes the byte path
    (32, 40, 1, 1, 0, 1, 8, False),        # 1x1: the codes are the operand matrix
    (16, 33, 1, 2, 0, 1, 8, False),        # 1x1 stride-2 shortcut
    (6, 40, 3, 2, 1, 1, 9, True),          # 3x3 stride 2
    (8, 12, 3, 1, 2, 2, 10, True),         # dilation
    (3, 64, 3, 1, 1, 1, 32, True),         # first layer of the network
])
def test_uint8_layer_path_equals_float_code_path_and_oracle(ops, oracle, golden_dir, cin, cout, k, stride, padding, dilation, hw, bias):
    """ApproxConv2d on the uint8 path (one operator, no float32 code tensor) against the same layer on float32 code
    tensors and torch operators: identical outputs, gradients to summation order; and the output against the four-term
    expression of the reference (app_layers.py:175-183) evaluated with the oracle's LUT convolution in float64."""
    import app_layers as L
    self_ops, P = ops
    print("uint8 layer path", cin, cout, k, stride, padding, dilation, hw, flush=True)
    torch.manual_seed(7)
    layer = L.ApproxConv2d(cin, cout, k, stride=stride, padding=padding, dilation=dilation, bias=bias, a_bits=7, w_bits=7).cuda().train()
    x = torch.randn(4, cin, hw, hw, device="cuda") * 2 + 0.3
    layer(x)                                          # one training pass sets the ranges
    layer.eval()                                      # frozen observers: both paths see the same scales
    gy = None
    res = []
    for fused, fused_w in ((True, True), (False, True), (True, False)):
        layer.fused_layer, layer.fused_weight_side = fused, fused_w
        xi = x.clone().requires_grad_()
        layer.zero_grad()
        y = layer(xi)
        if gy is None:
            gy = torch.randn_like(y)
        y.backward(gy)
        res.append((y.detach(), xi.grad, layer.weight.grad.clone(), layer.bias.grad.clone() if bias else None))
    layer.fused_layer = False
    assert layer._takes_uint8_path(x) is False
    layer.fused_layer = True
    assert layer._takes_uint8_path(x) is True
    # (weight side in one launch each way, weight side in torch operators) against the float32 code path
    for other in (res[0], res[2]):
        assert other[0].is_contiguous() and torch.equal(other[0], res[1][0])
        for a, b in zip(other[1:], res[1][1:]):
            if a is not None:
                torch.testing.assert_close(a, b, rtol=1e-5, atol=2e-6 * float(b.abs().max()))
    # the reference's expression with the oracle's LUT convolution
    s_a, z_a, s_w, z_w = (float(t) for t in (layer.activation_scale, layer.activation_zp_neg, layer.weight_scale, layer.weight_zp_neg))
    xc = L._to_codes_torch(x, layer.activation_scale, layer.activation_zp_neg, 127.0)
    wc = L._to_codes_torch(layer.weight.detach(), layer.weight_scale, layer.weight_zp_neg, 127.0)
    fwd2d = oracle.unpack_table(P.lut_appmult.cpu().numpy(), 7)
    am = oracle.conv2d_lut_np(xc.cpu().numpy().astype(np.uint8), wc.cpu().numpy().astype(np.uint8), fwd2d, stride, padding, dilation)
    conv = lambda a, b: F.conv2d(a.double(), b.double(), stride=stride, padding=padding, dilation=dilation)
    total = (torch.tensor(am.astype(np.float64), device="cuda") + conv(xc, torch.full_like(wc, z_w)) + conv(torch.full_like(xc, z_a), wc)
             + conv(torch.full_like(xc, z_a), torch.full_like(wc, z_w)))
    want = s_a * s_w * total + (layer.bias.detach().double().view(1, -1, 1, 1) if bias else 0.0)
    torch.testing.assert_close(res[0][0].double(), want, rtol=1e-5, atol=1e-5 * float(want.abs().max()))


@pytest.mark.parametrize("n,c,k,hw,stride,padding,dilation", [
    (24, 16, 3, (12, 12), 1, 1, 1), (7, 5, 3, (9, 7), 2, 1, 1), (40, 32, 1, (8, 8), 1, 0, 1), (64, 3, 7, (20, 20), 2, 3, 1),
    (12, 300, 3, (6, 6), 1, 2, 2), (512, 512, 3, (4, 4), 1, 1, 1)])
def test_weight_side_in_one_launch_each_way(ops, n, c, k, hw, stride, padding, dilation):
    """conv_weight_prepare against the torch operators it replaces (codes, tap-major operand, in-range mask, response to an
    all-ones image: integer valued, so exact), conv_batch_sum_scaled against a float64 sum, and conv_weight_grad against
    autograd through those operators in float64."""
    import approx_ops
    import app_layers as L
    print("weight side", n, c, k, hw, stride, padding, dilation, flush=True)
    g = torch.Generator(device="cuda").manual_seed(n * 131 + c)
    w = torch.randn(n, c, k, k, device="cuda", generator=g) * 0.2
    scale = torch.tensor([0.0041], device="cuda")
    zpn = torch.tensor([-57.0], device="cuda")                  # some weights fall outside the code range on both sides
    qmax = 127.0
    ones = torch.ones(1, 1, *hw, device="cuda")
    tapmask = F.unfold(ones, (k, k), dilation=dilation, padding=padding, stride=stride)[0].contiguous()
    T, Lp = tapmask.shape
    bt = torch.empty(T * c, n, dtype=torch.uint8, device="cuda")
    inside = torch.empty(n, c, k, k, dtype=torch.uint8, device="cuda")
    wresp = torch.empty(n, Lp, device="cuda")
    approx_ops.conv_weight_prepare(w, scale, zpn, qmax, tapmask, bt, inside, wresp)
    q = w / scale - zpn
    codes = torch.clamp(torch.round(q), 0, qmax)
    assert torch.equal(codes, L._to_codes_torch(w, scale, zpn, torch.tensor(qmax, device="cuda")))
    assert torch.equal(bt, codes.permute(2, 3, 1, 0).reshape(T * c, n).to(torch.uint8))
    r = torch.round(q)
    assert torch.equal(inside.bool(), (r >= 0) & (r <= qmax))
    assert 0 < int(inside.sum()) < inside.numel()
    want_resp = F.conv2d(torch.ones(1, c, *hw, device="cuda", dtype=torch.float64), codes.double(), stride=stride, padding=padding, dilation=dilation)
    assert torch.equal(wresp.double().view(-1), want_resp.view(-1))
    # gradient of the zero-point term: batch sum with the three scalars, folded onto the taps
    bn = 37
    gout = torch.randn(bn, n, Lp, device="cuda", generator=g)
    z_a, s_a, s_w = (torch.tensor([v], device="cuda") for v in (-3.0, 0.013, 0.0041))
    gwr = torch.empty(n, Lp, device="cuda")
    gz = torch.empty(approx_ops.conv_zero_point_grad_parts(Lp), n, T, device="cuda")
    approx_ops.conv_zero_point_grad(gout, z_a, s_a, s_w, tapmask, gz, gwr)
    want = (z_a * (s_a * s_w)).double() * gout.double().sum(dim=0)
    torch.testing.assert_close(gwr.double(), want, rtol=1e-5, atol=1e-6 * float(want.abs().max()))
    want_z = want @ tapmask.double().t()
    torch.testing.assert_close(gz.double().sum(dim=0), want_z, rtol=1e-5, atol=1e-6 * float(want.abs().sum(dim=1).max()))
    gz2 = torch.empty_like(gz)
    approx_ops.conv_zero_point_grad(gout, z_a, s_a, s_w, tapmask, gz2)          # (without the optional output)
    assert torch.equal(gz, gz2)
    # weight gradient: autograd through codes -> (operand gradient, response) in float64
    gbt = torch.randn(T * c, n, device="cuda", generator=g)
    gw = torch.empty_like(w)
    approx_ops.conv_weight_grad(gbt, gz, inside, scale, gw)
    wd = w.double().requires_grad_()
    qd = wd / scale.double() - zpn.double()
    cd = torch.clamp(qd - qd.detach() + torch.round(q).double(), 0, qmax)
    resp = cd.sum(dim=1).reshape(n, T) @ tapmask.double()
    loss = (cd.permute(2, 3, 1, 0).reshape(T * c, n) * gbt.double()).sum() + (resp * gwr.double()).sum()
    loss.backward()
    torch.testing.assert_close(gw.double(), wd.grad, rtol=1e-5, atol=2e-6 * float(wd.grad.abs().max()))


def test_zero_point_gradient_of_a_large_batch_and_ragged_sizes(ops):
    import approx_ops
    g = torch.Generator(device="cuda").manual_seed(5)
    one = lambda v: torch.tensor([v], device="cuda")
    for bn, n, L, T in ((512, 64, 1024, 9), (3, 2, 5, 1), (130, 6, 683, 4), (9, 1, 7, 64), (64, 512, 16, 9), (40, 3, 2500, 49)):
        print("zero-point gradient", bn, n, L, T, flush=True)
        x = torch.randn(bn, n, L, device="cuda", generator=g)
        mask = (torch.rand(T, L, device="cuda", generator=g) < 0.8).float()
        gwr = torch.empty(n, L, device="cuda")
        parts = approx_ops.conv_zero_point_grad_parts(L)
        assert parts == (L + 63) // 64
        gz = torch.empty(parts, n, T, device="cuda")
        approx_ops.conv_zero_point_grad(x, one(2.0), one(0.5), one(3.0), mask, gz, gwr)
        want = 3.0 * x.double().sum(dim=0)
        torch.testing.assert_close(gwr.double(), want, rtol=1e-5, atol=1e-6 * float(want.abs().max()))
        torch.testing.assert_close(gz.double().sum(dim=0), want @ mask.double().t(), rtol=1e-5, atol=1e-6 * float(want.abs().sum(dim=1).max()))
        again = torch.empty_like(gz)
        approx_ops.conv_zero_point_grad(x, one(2.0), one(0.5), one(3.0), mask, again)
        assert torch.equal(gz, again)                       # fixed summation order


@pytest.mark.parametrize("bn,n,hw,T", [(37, 64, (32, 32), 9), (16, 128, (16, 16), 9), (9, 40, (16, 8), 1), (64, 32, (16, 16), 49),
                                       (5, 64, (32, 32), 9), (12, 256, (16, 16), 9), (20, 64, (8, 8), 9), (3, 7, (5, 5), 4)])
def test_output_gradient_side_in_one_call(ops, bn, n, hw, T):
    """conv_output_grad (rows + row sums + zero-point gradient on the taps; the batch sums come out of the rows kernel where
    positions are a multiple of 128 and there are at most 128 channels) against the two separate calls: identical rows and
    row sums, tap sums to summation order and against float64."""
    import approx_ops
    print("output gradient side", bn, n, hw, T, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(bn * 7 + n)
    L = hw[0] * hw[1]
    g = torch.randn(bn, n, *hw, device="cuda", generator=gen)
    mask = (torch.rand(T, L, device="cuda", generator=gen) < 0.8).float()
    z_a, s_a, s_w = (torch.tensor([v], device="cuda") for v in (-3.0, 0.013, 0.0041))
    rows0, t0 = torch.empty(bn * L, n, device="cuda"), torch.empty(bn * L, device="cuda")
    approx_ops.conv_dequant_backward_rowsum(g, s_a, s_w, rows0, t0)
    parts = approx_ops.conv_zero_point_grad_parts(L)
    gz0 = torch.empty(parts, n, T, device="cuda")
    approx_ops.conv_zero_point_grad(g, z_a, s_a, s_w, mask, gz0)
    rows1, t1 = torch.full_like(rows0, float("nan")), torch.full_like(t0, float("nan"))
    gz1 = torch.full_like(gz0, float("nan"))
    approx_ops.conv_output_grad(g, z_a, s_a, s_w, mask, rows1, t1, gz1)
    assert torch.equal(rows1, rows0) and torch.equal(t1, t0)
    want = ((z_a * (s_a * s_w)).double() * g.double().sum(dim=0).view(n, L)) @ mask.double().t()
    bound = 1e-6 * float((g.double().sum(dim=0).abs().view(n, L).sum(dim=1)).max()) * abs(float(z_a * s_a * s_w)) + 1e-12
    torch.testing.assert_close(gz1.double().sum(dim=0), want, rtol=1e-5, atol=bound)
    torch.testing.assert_close(gz1.sum(dim=0), gz0.sum(dim=0), rtol=1e-5, atol=bound)
    again = torch.empty_like(gz1)
    approx_ops.conv_output_grad(g, z_a, s_a, s_w, mask, torch.empty_like(rows0), torch.empty_like(t0), again)
    assert torch.equal(again, gz1)                          # fixed summation order
    # rows and row sums alone
    rows2, t2 = torch.full_like(rows0, float("nan")), torch.full_like(t0, float("nan"))
    approx_ops.conv_output_grad(g, None, s_a, s_w, None, rows2, t2, None)
    assert torch.equal(rows2, rows0) and torch.equal(t2, t0)


@pytest.mark.parametrize("cin,cout,k,stride,padding,hw,bn", [(16, 24, 3, 1, 1, 12, 4), (64, 64, 3, 1, 1, 16, 16), (5, 7, 3, 2, 1, 9, 3), (32, 40, 1, 1, 0, 8, 4)])
def test_relu_folded_into_the_layers_quantiser(ops, cin, cout, k, stride, padding, hw, bn):
    """ApproxConv2d with pre_relu on x against the same layer on relu(x): identical observer state, quantisation parameters
    and outputs; identical input gradients (the in-range mask carries the ReLU's mask) and weight gradients -- on the uint8
    path in training and evaluation mode, and on the float-code path (where the layer applies the ReLU as an operator)."""
    import copy
    import approx_ops
    import app_layers as L
    print("relu fold", cin, cout, k, stride, padding, hw, bn, flush=True)
    torch.manual_seed(11)
    plain = L.ApproxConv2d(cin, cout, k, stride=stride, padding=padding, bias=False, a_bits=7, w_bits=7).cuda().train()
    fold = copy.deepcopy(plain)
    fold.pre_relu = True
    x = torch.randn(bn, cin, hw, hw, device="cuda") * 2 - 0.2
    x.view(-1)[::7] = 0.0                                           # exact zeros: the ReLU passes no gradient there
    gy = None
    for mode in ("train", "train", "eval", "float"):
        if mode == "eval":
            plain.eval(); fold.eval()
        if mode == "float":
            plain.fused_layer = fold.fused_layer = False
        xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
        plain.zero_grad(); fold.zero_grad()
        ya = plain(F.relu(xa))
        yb = fold(xb)
        if gy is None:
            gy = torch.randn_like(ya)
        ya.backward(gy); yb.backward(gy)
        for name in ("activation_scale", "activation_zp_neg", "weight_scale", "weight_zp_neg"):
            assert torch.equal(getattr(plain, name), getattr(fold, name)), (mode, name)
        assert torch.equal(plain.activation_observer.min_val, fold.activation_observer.min_val)
        assert torch.equal(plain.activation_observer.max_val, fold.activation_observer.max_val)
        assert float(fold.activation_observer.min_val) >= 0.0
        assert torch.equal(ya, yb), mode
        assert torch.equal(xa.grad, xb.grad), mode
        assert (xb.grad[x <= 0] == 0).all()
        torch.testing.assert_close(fold.weight.grad, plain.weight.grad, rtol=0, atol=0)
    # the observer and quantiser entry points by themselves
    big = torch.randn(3, 8, 33, 31, device="cuda") - 0.5
    state = torch.zeros(approx_ops.MINMAX_STATE_WORDS, dtype=torch.int32, device="cuda")
    lo, hi, sc, zp = (torch.zeros(1, device="cuda") for _ in range(4))
    approx_ops.observe_minmax(big, state, lo, hi, sc, zp, 0, 0.1, 127.0, 1e-7, relu=True)
    assert float(lo) == 0.0 and float(hi) == float(big.max())
    neg = -torch.rand(1000, device="cuda") - 1.0
    approx_ops.observe_minmax(neg, state, lo, hi, sc, zp, 0, 0.1, 127.0, 1e-7, relu=True)
    assert float(lo) == 0.0 and float(hi) == 0.0


def test_uint8_layer_path_first_layer_needs_no_input_gradient(ops):
    import app_layers as L
    torch.manual_seed(1)
    layer = L.ApproxConv2d(3, 16, 3, padding=1, bias=False, a_bits=7, w_bits=7).cuda().train()
    x = torch.randn(2, 3, 8, 8, device="cuda")
    y = layer(x)
    y.square().mean().backward()
    assert layer.weight.grad is not None and torch.isfinite(layer.weight.grad).all()


@pytest.mark.parametrize("bits,bn,L,K,N,masked,bias", [
    (7, 8, 1024, 576, 64, False, True),      # expanded-table kernel stores the activation itself
    (7, 8, 1024, 576, 64, True, True),       # a masked code 128: the gated direct kernel and the gated dequantisation do the work
    (7, 32, 64, 64, 40, False, False),       # ragged column tile
    (7, 16, 256, 2304, 256, False, True),    # K split over workgroups: sums meet in memory, second pass
    (7, 3, 25, 45, 10, False, True),         # small: direct kernel + second pass
    (7, 2050, 1, 64, 32, False, True),       # one position per image, rows not a multiple of the wave's 64
    (8, 8, 1024, 288, 64, False, True),      # 8-bit expanded-table kernel
    (6, 4, 1024, 72, 32, False, False),      # narrower table
])
def test_forward_with_dequantising_store_equals_gemm_then_dequantisation(ops, oracle, bits, bn, L, K, N, masked, bias):
    """amr_lut_conv_forward_dequant_f32 through the module function, against approx_gemm_forward (float32 sums, themselves
    checked bit-exact against the oracle here) followed by conv_dequant: identical bits for every shape and kernel choice."""
    import approx_ops
    print("forward + dequant", bits, bn, L, K, N, masked, flush=True)
    rng = np.random.default_rng(21)
    n = 1 << bits
    M = bn * L
    A = rng.integers(0, n, (M, K)).astype(np.uint8)
    B = rng.integers(0, n, (K, N)).astype(np.uint8)
    if masked:
        A[M // 2, 3] = n
    T = oracle.synth_lut(bits, 64, rng)
    flat = oracle.pack_table(T, bits, np.uint16)
    a, b, lut = (torch.tensor(v, device="cuda") for v in (A, B, flat))
    g = torch.Generator(device="cuda").manual_seed(4)
    x_sum = torch.randint(0, 9 * 64 * 127, (M,), device="cuda", generator=g).float()
    w_resp = torch.randint(0, 9 * 64 * 127, (N, L), device="cuda", generator=g).float()
    taps = torch.randint(1, 577, (L,), device="cuda", generator=g).float()
    z_a, z_w = torch.tensor([-3.0], device="cuda"), torch.tensor([-61.0], device="cuda")
    s_a, s_w = torch.tensor([0.0213], device="cuda"), torch.tensor([0.0037], device="cuda")
    bvec = torch.randn(N, device="cuda", generator=g) if bias else None
    side = int(round(L ** 0.5))
    hw = (side, side) if side * side == L else (1, L)
    # mode 2: the expanded-table kernels wherever the shape allows (the test sizes are below the sizes the library picks them at)
    old = approx_ops._lib.amr_set_expanded_table_kernels(2)
    try:
        c = torch.empty((M, N), dtype=torch.float32, device="cuda")
        approx_ops.approx_gemm_forward(a, b, c, lut)
        want = torch.full((bn, N, *hw), float("nan"), device="cuda")
        approx_ops.conv_dequant(c, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, want)
        got = torch.full((bn, N, *hw), float("nan"), device="cuda")
        approx_ops.approx_conv_forward_dequant(a, b, lut, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, got)
    finally:
        approx_ops._lib.amr_set_expanded_table_kernels(old)
    rows = slice(0, min(M, 2048))
    assert (c[rows].cpu().numpy() == oracle.forward_c(A[rows], B, flat, bits).astype(np.float32)).all()
    assert torch.equal(got, want)


@pytest.mark.parametrize("bits,bn,c,h,w,n,masked,bias", [
    # (the kernel serves shapes that fill the device without a K split: column tiles x blocks of 1024 rows >= compute units)
    (7, 128, 64, 32, 32, 64, False, True),     # conv2_x
    (7, 2100, 16, 7, 9, 40, False, False),     # image sides that are no powers of two, ragged column tile
    (7, 16400, 32, 4, 4, 32, False, True),     # 4x4 images: most pixels touch the border
    (7, 146, 16, 31, 29, 64, False, True),     # rows not a multiple of a wave's 64
    (6, 128, 32, 32, 32, 64, False, True),     # narrower table
    (7, 128, 64, 32, 32, 64, True, True),      # a masked code: fall-back with the window matrix, NaN without
])
def test_convolution_shaped_forward_equals_the_forward_pass_on_the_window_matrix(ops, oracle, bits, bn, c, h, w, n, masked, bias):
    """approx_conv_forward_implicit (no window matrix: the kernel reads the neighbouring pixels' codes, code 0 for padding)
    against approx_conv_forward_dequant on the window matrix of the same codes: identical bits; the sums of the first rows
    against the oracle's LUT GEMM on that window matrix."""
    import approx_ops
    print("implicit forward", bits, bn, c, h, w, n, masked, flush=True)
    rng = np.random.default_rng(31)
    nc = 1 << bits
    M, L, K = bn * h * w, h * w, 9 * c
    X = rng.integers(0, nc, (bn, c, h, w)).astype(np.uint8)
    B = rng.integers(0, nc, (K, n)).astype(np.uint8)
    if masked:
        X[bn // 2, 3, h // 2, 1] = nc
    T = oracle.synth_lut(bits, 64, rng)
    flat = oracle.pack_table(T, bits, np.uint16)
    x, bt, lut = (torch.tensor(v, device="cuda") for v in (X, B, flat))
    codes = x.permute(0, 2, 3, 1).reshape(M, c).contiguous()
    a = torch.empty((M, K), dtype=torch.uint8, device="cuda")
    approx_ops.im2col_nhwc(codes, a, (bn, c, h, w), (3, 3), 1, 1, 1)
    g = torch.Generator(device="cuda").manual_seed(4)
    x_sum = torch.randint(0, 9 * 64 * 127, (M,), device="cuda", generator=g).float()
    w_resp = torch.randint(0, 9 * 64 * 127, (n, L), device="cuda", generator=g).float()
    taps = torch.randint(1, 577, (L,), device="cuda", generator=g).float()
    z_a, z_w = torch.tensor([-3.0], device="cuda"), torch.tensor([-61.0], device="cuda")
    s_a, s_w = torch.tensor([0.0213], device="cuda"), torch.tensor([0.0037], device="cuda")
    bvec = torch.randn(n, device="cuda", generator=g) if bias else None
    old = approx_ops._lib.amr_set_expanded_table_kernels(2)
    try:
        assert approx_ops.conv_forward_implicit_supported(lut, (bn, c, h, w), n)
        want = torch.full((bn, n, h, w), float("nan"), device="cuda")
        approx_ops.approx_conv_forward_dequant(a, bt, lut, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, want)
        got = torch.full((bn, n, h, w), float("nan"), device="cuda")
        approx_ops.approx_conv_forward_implicit(codes, bt, lut, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, got, (bn, c, h, w),
                                                a_fallback=a if masked else None)
        assert torch.equal(got, want)
        if masked:
            lost = torch.zeros((bn, n, h, w), device="cuda")
            approx_ops.approx_conv_forward_implicit(codes, bt, lut, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, lost, (bn, c, h, w))
            assert torch.isnan(lost).all()
        # with the expansion kept between calls: a miss, then a hit, same bits
        cache = approx_ops.ForwardCache()
        for _ in range(2):
            again = torch.full((bn, n, h, w), float("nan"), device="cuda")
            approx_ops.approx_conv_forward_implicit(codes, bt, lut, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, again, (bn, c, h, w),
                                                    a_fallback=a if masked else None, cache=cache, b_version=5)
            assert torch.equal(again, want)
        assert cache.stats()[:2] == (1, 1)
        # refused: channels no multiple of 16, 8-bit tables
        assert not approx_ops.conv_forward_implicit_supported(lut, (bn, c + 8, h, w), n)
        assert not approx_ops.conv_forward_implicit_supported(torch.zeros(66306, dtype=torch.uint16, device="cuda"), (bn, c, h, w), n)
    finally:
        approx_ops._lib.amr_set_expanded_table_kernels(old)
    # the sums behind the activation, against the oracle on the window matrix (first rows)
    rows = slice(0, min(M, 1024))
    csum = torch.empty((M, n), dtype=torch.float32, device="cuda")
    approx_ops.approx_gemm_forward(a, bt, csum, lut)
    assert (csum[rows].cpu().numpy() == oracle.forward_c(a[rows].cpu().numpy(), B, flat, bits).astype(np.float32)).all()
    plain = torch.empty_like(want)
    approx_ops.conv_dequant(csum, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bvec, plain)
    assert torch.equal(plain, want)


def test_layer_reads_the_codes_itself_where_no_window_matrix_is_needed(ops):
    """ApproxConv2d (3x3, stride 1, padding 1): under no_grad, and with frozen weights, the forward pass takes the
    convolution-shaped kernel (no im2col call); outputs and the input gradient equal those of the pass on the window matrix."""
    import approx_ops
    import app_layers as L
    torch.manual_seed(3)
    layer = L.ApproxConv2d(64, 64, 3, padding=1, bias=False, a_bits=7, w_bits=7).cuda().train()
    x = torch.randn(512, 64, 16, 16, device="cuda") * 2 + 0.3
    layer(x)
    layer.eval()
    calls = []
    native = approx_ops.im2col_nhwc
    approx_ops.im2col_nhwc = lambda *a, **k: (calls.append(1), native(*a, **k))[1]
    try:
        xi = x.clone().requires_grad_()
        y_train = layer(xi)                               # weights require a gradient: window matrix
        assert len(calls) == 1
        y_train.square().mean().backward()
        with torch.no_grad():
            y_eval = layer(x)
        assert len(calls) == 1 and torch.equal(y_eval, y_train.detach())
        layer.weight.requires_grad_(False)
        xj = x.clone().requires_grad_()
        y_frozen = layer(xj)                              # only the input gradient is asked for: convolution-shaped both ways
        assert len(calls) == 1 and torch.equal(y_frozen.detach(), y_train.detach())
        y_frozen.square().mean().backward()
        torch.testing.assert_close(xj.grad, xi.grad, rtol=1e-5, atol=1e-6 * float(xi.grad.abs().max()))
    finally:
        approx_ops.im2col_nhwc = native


def test_expansions_kept_in_training_mode_for_weights_that_outlive_a_step(ops):
    """keep_expansions_in_training: a frozen 3x3 layer in training mode expands its forward and input-gradient tables once;
    later passes hit both caches (and the prepared weight operand) with identical results; an in-place weight update
    invalidates them.  The convolution-shaped input gradient with a cache of its own: miss, hit, stale on purpose, new number."""
    import copy
    import approx_ops
    import app_layers as L
    from self_ops.ops_py import approx_ops as P
    torch.manual_seed(5)
    layer = L.ApproxConv2d(64, 64, 3, padding=1, bias=False, a_bits=7, w_bits=7).cuda().train()
    layer.weight.requires_grad_(False)
    plain = copy.deepcopy(layer)
    layer.keep_expansions_in_training = True
    x = torch.randn(16, 64, 32, 32, device="cuda") * 2 + 0.3
    gy = None
    for it in range(3):
        if it == 2:
            with torch.no_grad():
                layer.weight.add_(0.01); plain.weight.add_(0.01)
        xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
        ya, yb = layer(xa), plain(xb)
        if gy is None:
            gy = torch.randn_like(ya)
        ya.backward(gy); yb.backward(gy)
        assert torch.equal(ya, yb) and torch.equal(xa.grad, xb.grad), it
    assert layer._fwd_cache.stats()[:2] == (1, 2)         # hit on the second pass, miss again after the weight update
    assert layer._bwd_cache.stats()[:2] == (1, 2)
    assert plain.__dict__.get("_fwd_cache") is None
    # the entry point by itself
    bn, c, h, w, n = 8, 32, 16, 16, 64
    g = torch.Generator(device="cuda").manual_seed(8)
    M = bn * h * w
    codes = torch.randint(0, 128, (M, c), device="cuda", generator=g, dtype=torch.int32).to(torch.uint8)
    bt = torch.randint(0, 128, (9 * c, n), device="cuda", generator=g, dtype=torch.int32).to(torch.uint8)
    rows = torch.randn(M, n, device="cuda", generator=g)
    t = rows.sum(dim=1).contiguous()
    inside = (torch.rand(bn, c, h, w, device="cuda", generator=g) < 0.9).to(torch.uint8)
    zw, sc = torch.tensor([-61.0], device="cuda"), torch.tensor([0.037], device="cuda")
    old = approx_ops._lib.amr_set_expanded_table_kernels(2)
    try:
        def run(b, cache=None, version=0):
            gx = torch.full((bn, c, h, w), float("nan"), device="cuda")
            approx_ops.approx_conv_input_grad(rows, codes, b, P.lut_grad_a, t, zw, inside, sc, gx, cache=cache, b_version=version)
            return gx
        want = run(bt)
        cache = approx_ops.ForwardCache()
        assert torch.equal(run(bt, cache, 1), want) and torch.equal(run(bt, cache, 1), want)
        bt2 = bt.clone(); bt2[5, 7] ^= 1
        assert torch.equal(run(bt2, cache, 1), want)                 # same number: the old expansion, on purpose
        assert torch.equal(run(bt2, cache, 2), run(bt2))
        assert cache.stats()[:2] == (2, 2)
    finally:
        approx_ops._lib.amr_set_expanded_table_kernels(old)


def _conv_grad_case(oracle, seed, bn, c, h, w, n, lo=-1024, hi=3073, masked=False):
    """Operands of one input-gradient problem of a 3x3 / stride 1 / padding 1 convolution and its float64 answer."""
    rng = np.random.default_rng(seed)
    x_codes = rng.integers(0, 128, (bn, c, h, w)).astype(np.uint8)
    if masked:
        x_codes[bn // 2, 3, h // 2, w // 2] = 128
    bt = rng.integers(0, 128, (9 * c, n)).astype(np.uint8)                              # rows (tap, channel)
    la = oracle.pack_table(rng.integers(lo, hi, (128, 128)), 7, np.int16)
    g_rows = rng.standard_normal((bn * h * w, n)).astype(np.float32)
    t = g_rows.sum(axis=1)
    inside = (rng.random((bn, c, h, w)) < 0.85).astype(np.uint8)
    zw, scale = -61.0, 0.037
    a_ref, _, _ = oracle.im2col_np(x_codes, 3, 3, 1, 1, 1)                              # columns (channel, tap)
    a_tap = a_ref.reshape(-1, c, 9).transpose(0, 2, 1).reshape(-1, 9 * c)
    ga64, _ = oracle.backward_c_f64(g_rows, a_tap, bt, la, la, 7)
    cols = torch.tensor(ga64).view(bn, h * w, 9, c).permute(0, 3, 2, 1).reshape(bn, c * 9, h * w)      # fold's (channel, tap) order
    fold = lambda cc: F.fold(cc, (h, w), (3, 3), padding=1)
    t_cols = torch.tensor(t, dtype=torch.float64).view(bn, 1, h * w).expand(bn, 9, h * w)
    want = (fold(cols) + zw * fold(t_cols)) / scale * torch.tensor(inside, dtype=torch.float64)
    codes = np.ascontiguousarray(x_codes.transpose(0, 2, 3, 1).reshape(bn * h * w, c))
    return dict(codes=codes, a_tap=a_tap, bt=bt, la=la, g_rows=g_rows, t=t, inside=inside, zw=zw, scale=scale, want=want)


@pytest.mark.parametrize("bn,c,h,w,n", [
    (2, 16, 16, 16, 32),        # one block of 512 pixels, 16 channels per tile
    (8, 64, 32, 32, 64),        # conv2_x of the benchmark network: 32 channels per tile, half an image per tile
    (3, 48, 16, 16, 96),        # channels and columns that are multiples of 16 / 32 only
    (40, 16, 4, 4, 32),         # 4x4 images: most pixels sit on a border
    (3, 16, 15, 17, 32),        # sizes that are no powers of two, pixel count no multiple of 32, 255 positions per image
    (10, 32, 8, 8, 128),        # four column tiles
])
def test_convolution_shaped_input_gradient_against_oracle_and_gemm_shaped_path(ops, oracle, bn, c, h, w, n):
    """amr_lut_conv_input_grad_f32 (implicit GEMM over the input pixels) against the float64 oracle (LUT gradient GEMM, fold,
    zero-point term, straight-through mask) and against the library's GEMM-shaped composition of the same steps."""
    import approx_ops
    print("conv-shaped gradA", bn, c, h, w, n, flush=True)
    k = _conv_grad_case(oracle, 31, bn, c, h, w, n)
    dev = lambda v, dt=None: torch.tensor(v, device="cuda", dtype=dt)
    codes, a_tap, bt, la, g_rows, t, inside = (dev(k[x]) for x in ("codes", "a_tap", "bt", "la", "g_rows", "t", "inside"))
    zw, scale = dev([k["zw"]], torch.float32), dev([k["scale"]], torch.float32)
    old = approx_ops._lib.amr_set_expanded_table_kernels(2)
    try:
        assert approx_ops.conv_input_grad_supported(la, (bn, c, h, w), n)
        gx = torch.full((bn, c, h, w), float("nan"), device="cuda")
        approx_ops.approx_conv_input_grad(g_rows, codes, bt, la, t, zw, inside, scale, gx)
        cols = torch.empty((bn, 9 * c, h * w), device="cuda")
        approx_ops.approx_gemm_backward(g_rows, a_tap, bt, cols, None, la, la, ga_rows_per_image=h * w)
        gx2 = torch.full((bn, c, h, w), float("nan"), device="cuda")
        approx_ops.conv_input_grad(cols, t, zw, inside, scale, gx2, (3, 3), 1, 1, 1)
    finally:
        approx_ops._lib.amr_set_expanded_table_kernels(old)
    want = k["want"].cuda()
    tol = 1e-5 * float(want.abs().max())
    torch.testing.assert_close(gx.double(), want, rtol=0, atol=tol)
    torch.testing.assert_close(gx2.double(), want, rtol=0, atol=tol)
    assert (gx[inside == 0] == 0).all()


def test_convolution_shaped_input_gradient_fall_backs(ops, oracle):
    """A gradient table that cannot be held as halves, and a masked code among the operand codes: with the window matrix as
    fall-back operand the GEMM-shaped kernels queued behind give the oracle's answer; without it the result is NaN, not a
    silently wrong gradient.  Shapes the kernel does not serve are refused before anything is launched."""
    import approx_ops
    print("conv-shaped gradA fall-backs", flush=True)
    bn, c, h, w, n = 4, 32, 16, 16, 64
    dev = lambda v, dt=None: torch.tensor(v, device="cuda", dtype=dt)
    old = approx_ops._lib.amr_set_expanded_table_kernels(2)
    try:
        for name, kw in (("wide table", dict(lo=-20000, hi=20000)), ("masked code", dict(masked=True))):
            k = _conv_grad_case(oracle, 32, bn, c, h, w, n, **kw)
            assert approx_ops.grad_table_fits_halves(k["la"]) == (name == "masked code")
            codes, a_tap, bt, la, g_rows, t, inside = (dev(k[x]) for x in ("codes", "a_tap", "bt", "la", "g_rows", "t", "inside"))
            zw, scale = dev([k["zw"]], torch.float32), dev([k["scale"]], torch.float32)
            gx = torch.full((bn, c, h, w), 5.0, device="cuda")
            approx_ops.approx_conv_input_grad(g_rows, codes, bt, la, t, zw, inside, scale, gx, a_fallback=a_tap)
            want = k["want"].cuda()
            torch.testing.assert_close(gx.double(), want, rtol=0, atol=1e-5 * float(want.abs().max()), msg=name)
            gx.fill_(5.0)
            approx_ops.approx_conv_input_grad(g_rows, codes, bt, la, t, zw, inside, scale, gx)
            assert torch.isnan(gx).all(), name
        # refused: fewer than 512 pixels; channels no multiple of 16; 8-bit table
        la7 = dev(oracle.pack_table(np.zeros((128, 128), np.int64), 7, np.int16))
        la8 = dev(oracle.pack_table(np.zeros((256, 256), np.int64), 8, np.int16))
        assert not approx_ops.conv_input_grad_supported(la7, (1, 16, 16, 16), 32)
        assert not approx_ops.conv_input_grad_supported(la7, (4, 24, 16, 16), 32)
        assert not approx_ops.conv_input_grad_supported(la8, (4, 32, 16, 16), 32)
        assert approx_ops.conv_input_grad_supported(la7, (4, 32, 16, 16), 32)
        with pytest.raises(RuntimeError, match="not served"):
            approx_ops.approx_conv_input_grad(torch.zeros(256, 32, device="cuda"), torch.zeros((256, 16), dtype=torch.uint8, device="cuda"),
                                              torch.zeros((144, 32), dtype=torch.uint8, device="cuda"), la7, torch.zeros(256, device="cuda"),
                                              zw, torch.zeros((1, 16, 16, 16), dtype=torch.uint8, device="cuda"), scale,
                                              torch.zeros(1, 16, 16, 16, device="cuda"))
    finally:
        approx_ops._lib.amr_set_expanded_table_kernels(old)


def test_uint8_layer_takes_the_convolution_shaped_input_gradient(ops):
    """A layer of the benchmark network's size (32 -> 64 channels, 32 x 32, batch 8) takes the implicit-GEMM input gradient
    by itself; its gradients agree with the float-code path."""
    import app_layers as L
    import approx_ops
    print("layer, conv-shaped gradA", flush=True)
    torch.manual_seed(9)
    layer = L.ApproxConv2d(32, 64, 3, stride=1, padding=1, bias=False, a_bits=7, w_bits=7).cuda().train()
    x = torch.randn(8, 32, 32, 32, device="cuda")
    layer(x)
    layer.eval()
    calls = []
    native = approx_ops.approx_conv_input_grad
    approx_ops.approx_conv_input_grad = lambda *a, **k: (calls.append(1), native(*a, **k))[1]
    try:
        res = []
        gy = None
        for fused in (True, False):
            layer.fused_layer = fused
            xi = x.clone().requires_grad_()
            layer.zero_grad()
            y = layer(xi)
            gy = torch.randn_like(y) if gy is None else gy
            y.backward(gy)
            res.append((y.detach(), xi.grad, layer.weight.grad.clone()))
    finally:
        approx_ops.approx_conv_input_grad = native
    assert len(calls) == 1
    assert torch.equal(res[0][0], res[1][0])
    for a, b in zip(res[0][1:], res[1][1:]):
        torch.testing.assert_close(a, b, rtol=0, atol=1e-5 * float(b.abs().max()))


def test_forward_expansion_cache_hits_and_invalidates(ops, oracle):
    """amr_lut_gemm_forward_cached through the module function: the first call expands, calls with the same version reuse the
    expansion (also with other rows A, also after a call whose A held a masked code), a changed B under an unchanged version
    gives the OLD B's sums -- the expansion really was reused -- and a new version gives the new ones; every result checked
    against the oracle."""
    import approx_ops
    print("forward cache", flush=True)
    rng = np.random.default_rng(41)
    M, K, N, bits = 4096, 256, 64, 7
    T = oracle.synth_lut(bits, 64, rng)
    flat = oracle.pack_table(T, bits, np.uint16)
    lut = torch.tensor(flat, device="cuda")
    A1, A2 = (rng.integers(0, 128, (M, K)).astype(np.uint8) for _ in range(2))
    A2[7, 5] = 128                                             # a masked code: the gated direct kernel serves this call
    B1, B2 = (rng.integers(0, 128, (K, N)).astype(np.uint8) for _ in range(2))
    a1, a2, b = torch.tensor(A1, device="cuda"), torch.tensor(A2, device="cuda"), torch.tensor(B1, device="cuda")
    c = torch.empty((M, N), dtype=torch.uint32, device="cuda")
    want = lambda A, B: oracle.forward_c(A, B, flat, bits)
    got = lambda: c.cpu().numpy().view(np.uint32)
    cache = approx_ops.ForwardCache()
    old = approx_ops._lib.amr_set_expanded_table_kernels(2)
    try:
        approx_ops.approx_gemm_forward(a1, b, c, lut, cache=cache, b_version=1)
        assert (got() == want(A1, B1)).all() and cache.stats()[:2] == (0, 1) and cache.stats()[2] >= K * N * 256
        approx_ops.approx_gemm_forward(a2, b, c, lut, cache=cache, b_version=1)
        assert (got() == want(A2, B1)).all() and cache.stats()[:2] == (1, 1)
        approx_ops.approx_gemm_forward(a1, b, c, lut, cache=cache, b_version=1)       # (the fall-back request of the call before is gone)
        assert (got() == want(A1, B1)).all() and cache.stats()[:2] == (2, 1)
        b.copy_(torch.tensor(B2))
        approx_ops.approx_gemm_forward(a1, b, c, lut, cache=cache, b_version=1)       # stale on purpose: same version, other contents
        assert (got() == want(A1, B1)).all() and cache.stats()[:2] == (3, 1)
        approx_ops.approx_gemm_forward(a1, b, c, lut, cache=cache, b_version=2)
        assert (got() == want(A1, B2)).all() and cache.stats()[:2] == (3, 2)
        cf = torch.empty((M, N), dtype=torch.float32, device="cuda")
        approx_ops.approx_gemm_forward(a1, b, cf, lut, cache=cache, b_version=2)
        assert (cf.cpu().numpy() == want(A1, B2).astype(np.float32)).all() and cache.stats()[:2] == (4, 2)
        # a larger shape replaces the buffer; a shape the expanded-table kernels do not take leaves the cache alone
        b_big = torch.tensor(rng.integers(0, 128, (2 * K, N)).astype(np.uint8), device="cuda")
        a_big = torch.tensor(rng.integers(0, 128, (M, 2 * K)).astype(np.uint8), device="cuda")
        approx_ops.approx_gemm_forward(a_big, b_big, c, lut, cache=cache, b_version=2)
        assert (got() == want(a_big.cpu().numpy(), b_big.cpu().numpy())).all() and cache.stats()[:2] == (4, 3)
        small_a, small_c = a1[:100].contiguous(), torch.empty((100, N), dtype=torch.uint32, device="cuda")
        approx_ops.approx_gemm_forward(small_a, b, small_c, lut, cache=cache, b_version=9)
        assert (small_c.cpu().numpy().view(np.uint32) == want(A1[:100], B2)).all() and cache.stats()[:2] == (4, 3)
    finally:
        approx_ops._lib.amr_set_expanded_table_kernels(old)
        cache.close()


def test_layer_keeps_its_expansion_in_evaluation_mode(ops):
    """An ApproxConv2d in evaluation mode expands the forward table once for its frozen weights; an in-place weight update, a
    training-mode pass or new tables make it expand again; outputs equal those of a layer without the cache throughout."""
    import app_layers as L
    import copy
    self_ops, P = ops
    print("layer forward cache", flush=True)
    torch.manual_seed(11)
    layer = L.ApproxConv2d(64, 64, 3, padding=1, bias=False, a_bits=7, w_bits=7).cuda().train()
    x = torch.randn(16, 64, 32, 32, device="cuda")           # 16384 x 576 x 64: a shape the library expands the table for by itself
    layer(x)
    plain = copy.deepcopy(layer)
    plain.keep_expansion_in_eval = False
    layer.eval(); plain.eval()
    with torch.no_grad():
        for _ in range(3):
            assert torch.equal(layer(x), plain(x))
        assert layer._fwd_cache.stats()[:2] == (2, 1)
        layer.weight.mul_(1.01); plain.weight.mul_(1.01)                       # in place: the version counter moves
        assert torch.equal(layer(x), plain(x)) and layer._fwd_cache.stats()[:2] == (2, 2)
        assert torch.equal(layer(x * 0.5), plain(x * 0.5)) and layer._fwd_cache.stats()[:2] == (3, 2)
        layer.train(); plain.train()
        assert torch.equal(layer(x * 2), plain(x * 2)) and layer._fwd_cache.stats()[:2] == (3, 2)   # training mode: no cache
        layer.eval(); plain.eval()
        assert torch.equal(layer(x), plain(x)) and layer._fwd_cache.stats()[:2] == (3, 3)            # the ranges may have moved
        keep = (P.lut_appmult, P.lut_grad_a, P.lut_grad_b)
        try:
            P.set_lookup_tables("cuda", keep[0].cpu().numpy(), keep[1].cpu().numpy(), keep[2].cpu().numpy())
            assert torch.equal(layer(x), plain(x)) and layer._fwd_cache.stats()[:2] == (3, 4)        # new tables: expanded again
        finally:
            P.lut_appmult, P.lut_grad_a, P.lut_grad_b = keep
