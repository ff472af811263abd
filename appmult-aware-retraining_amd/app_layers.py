"""Quantised layers that call the LUT operators (counterpart of the reference's ``micronet+/app_layers.py``).

Same class names, constructor arguments, buffers and numerics as the reference, so a model prepared
with :func:`prepare` behaves like one prepared there:

* per-layer asymmetric quantisation to unsigned codes, ``scale = max((max-min)/(2^b-1), eps)``,
  ``zp_neg = round(min/scale)``, real value ``= (code + zp_neg) * scale`` (reference ``app_layers.py:154-160``);
* activations are tracked by an exponential moving average of min/max (momentum 0.1), weights by the
  running extremes (reference ``:21-53``); both only update in training mode;
* ``ApproxConv2d`` evaluates ``s_a*s_w*(AM(X,W) + conv(X,Zw) + conv(Za,W) + conv(Za,Zw)) + bias`` where
  ``AM`` is the LUT convolution and the three ordinary convolutions undo the zero points
  (reference ``:175-183``); rounding uses the straight-through estimator (``:147-150``);
* ``QuantLinear`` and the pooling layers fake-quantise and call the ordinary torch op (``:101-111``,
  ``:188-267``).
"""
import copy

import torch
import torch.nn as nn
import torch.nn.functional as F

import self_ops


# ------------------------------------------------------------------------------------------ range tracking
class ObserverBase(nn.Module):
    """Tracks a (min, max) pair of the tensors it sees; never takes part in autograd."""

    def __init__(self, q_level):
        super().__init__()
        self.q_level = q_level
        self.num_flag = 0           # 0 until the first batch has been seen (python attribute, as in the reference)
        self.register_buffer("min_val", torch.zeros(1, dtype=torch.float32))
        self.register_buffer("max_val", torch.zeros(1, dtype=torch.float32))

    def update_range(self, min_val_cur, max_val_cur):
        raise NotImplementedError

    @torch.no_grad()
    def forward(self, input):
        lo, hi = torch.aminmax(input)
        if self.num_flag == 0:
            self.num_flag = 1
            self.min_val, self.max_val = lo, hi
        else:
            self.update_range(lo, hi)


class MinMaxObserver(ObserverBase):
    """Running extremes."""
    fused_mode = 1

    def __init__(self, q_level, out_channels):
        super().__init__(q_level)

    def update_range(self, min_val_cur, max_val_cur):
        self.min_val = torch.min(min_val_cur, self.min_val)
        self.max_val = torch.max(max_val_cur, self.max_val)


class MovingAverageMinMaxObserver(ObserverBase):
    """Exponential moving average of the per-batch extremes."""
    fused_mode = 2

    def __init__(self, q_level, out_channels, momentum=0.1):
        super().__init__(q_level)
        self.momentum = momentum

    def update_range(self, min_val_cur, max_val_cur):
        self.min_val = (1 - self.momentum) * self.min_val + self.momentum * min_val_cur
        self.max_val = (1 - self.momentum) * self.max_val + self.momentum * max_val_cur


def _scale_and_zero_point(observer, quant_max, eps):
    scale = torch.max((observer.max_val - observer.min_val) / quant_max, eps)
    return scale, torch.round(observer.min_val / scale)


def _observe(observer, x, quant_max, eps, scale, zp_neg, relu=False):
    """One observer step on ``x`` followed by the scale / zero point it implies; returns (scale, zp_neg) as NEW tensors,
    like the reference's ``self.activation_scale = torch.max(...)`` (``app_layers.py:154-160``): an autograd graph built by
    an earlier forward pass keeps the values it saw.  ``scale`` / ``zp_neg`` (the layer's current buffers) only say where the
    results live.  On the GPU the scalar arithmetic (range update, scale, zero point: a dozen one-element tensor operations
    in the reference, ``app_layers.py:21-53,154-160``) is one launch that updates the observer's range buffers in place
    (no graph ever holds those) and writes the two results; the values are those of the tensor expressions."""
    fused_mode = getattr(observer, "fused_mode", None)
    ok = (fused_mode is not None and x.is_cuda and x.dtype == torch.float32 and
          all(t is not None and t.is_cuda and t.dtype == torch.float32 and t.numel() == 1 and t.is_contiguous()
              for t in (observer.min_val, observer.max_val, scale, zp_neg)))
    if not ok:
        observer(F.relu(x) if relu else x)
        return _scale_and_zero_point(observer, quant_max, eps)
    import approx_ops
    with torch.no_grad():
        mode = 0 if observer.num_flag == 0 else fused_mode
        observer.num_flag = 1
        fresh = torch.empty(2, dtype=torch.float32, device=x.device)
        new_scale, new_zp = fresh[0:1], fresh[1:2]
        # torch divides by a host-side scalar through its reciprocal rounded to float32
        inv_qmax = 0.0 if quant_max.is_cuda else float(torch.tensor(1.0, dtype=torch.float32) / quant_max.to(torch.float32))
        momentum = getattr(observer, "momentum", 0.0)
        if x.is_contiguous() and x.numel() > 0:
            # extremes of x and the scalar update in one launch (the workgroups meet in four words owned by this observer)
            state = observer.__dict__.get("_minmax_state")
            if state is None or state.device != x.device:
                state = torch.zeros(approx_ops.MINMAX_STATE_WORDS, dtype=torch.int32, device=x.device)
                observer.__dict__["_minmax_state"] = state
            approx_ops.observe_minmax(x.detach(), state, observer.min_val, observer.max_val, new_scale, new_zp, mode, momentum,
                                      float(quant_max), float(eps), inv_qmax, relu=relu)
        else:
            lo, hi = torch.aminmax(F.relu(x) if relu else x)
            approx_ops.observer_update(lo.reshape(1), hi.reshape(1), observer.min_val, observer.max_val, new_scale, new_zp, mode,
                                       momentum, float(quant_max), float(eps), inv_qmax)
    return new_scale, new_zp


class _ToCodesFn(torch.autograd.Function):
    """clamp(round(x / scale - zp_neg), 0, quant_max) with straight-through rounding, one device pass each way
    (same values and gradients as the torch expression in :func:`_to_codes`)."""

    @staticmethod
    def forward(ctx, x, scale, zp_neg, quant_max):
        import approx_ops
        xc = x.contiguous()
        s, z = scale.detach().reshape(1).contiguous(), zp_neg.detach().reshape(1).contiguous()
        codes = torch.empty_like(xc)
        approx_ops.quantize_codes(xc, s, z, quant_max, codes)
        ctx.save_for_backward(xc, s, z)
        ctx.quant_max = quant_max
        return codes

    @staticmethod
    def backward(ctx, g):
        import approx_ops
        xc, s, z = ctx.saved_tensors
        gx = torch.empty_like(xc)
        approx_ops.quantize_codes_backward(g.contiguous(), xc, s, z, ctx.quant_max, gx)
        return gx, None, None, None


def _to_codes(x, scale, zp_neg, quant_max):
    """Affine map to [0, quant_max] with straight-through rounding; returns integer-valued floats."""
    if x.is_cuda and x.dtype == torch.float32 and scale.is_cuda and zp_neg.is_cuda:
        return _ToCodesFn.apply(x, scale, zp_neg, float(quant_max))
    affine = x / scale - zp_neg
    return torch.clamp(affine - affine.detach() + torch.round(affine), 0, quant_max)


def _to_codes_torch(x, scale, zp_neg, quant_max):
    """The same map written with torch operators (what the reference's quantize_v2 composes)."""
    affine = x / scale - zp_neg
    return torch.clamp(affine - affine.detach() + torch.round(affine), 0, quant_max)


class _ConvDequantFn(torch.autograd.Function):
    """(s_a*s_w) * (c + z_w*x_sum + z_a*w_resp + z_a*z_w*taps) + bias from the GEMM's [B*L, N] rows to a contiguous
    [B,N,oh,ow] activation in one device pass (same operations in the same order as the torch expression of
    ApproxConv2d.forward, so the same bits); backward: one transposing pass for the rows plus three reductions."""

    @staticmethod
    def forward(ctx, c_rows, x_sum, w_resp, taps, z_a, z_w, s_a, s_w, bias, out_shape):
        import approx_ops
        one = lambda t: t.detach().reshape(1).contiguous()
        z_a, z_w, s_a, s_w = one(z_a), one(z_w), one(s_a), one(s_w)
        out = torch.empty(out_shape, dtype=torch.float32, device=c_rows.device)
        approx_ops.conv_dequant(c_rows.contiguous(), x_sum.contiguous(), w_resp.contiguous(), taps.contiguous(), z_a, z_w, s_a, s_w,
                                None if bias is None else bias.detach().contiguous(), out)
        ctx.save_for_backward(z_a, z_w, s_a, s_w)
        ctx.shapes = (c_rows.shape, x_sum.shape, w_resp.shape, bias is not None)
        return out

    @staticmethod
    def backward(ctx, g):
        import approx_ops
        z_a, z_w, s_a, s_w = ctx.saved_tensors
        c_shape, xs_shape, wr_shape, has_bias = ctx.shapes
        g = g.contiguous()
        s = s_a * s_w
        g_rows = g_xs = g_wr = g_bias = None
        if ctx.needs_input_grad[0]:
            g_rows = torch.empty(c_shape, dtype=torch.float32, device=g.device)
            approx_ops.conv_dequant_backward(g, s_a, s_w, g_rows)
        if ctx.needs_input_grad[1]:
            g_xs = ((z_w * s) * g.sum(dim=1, keepdim=True)).reshape(xs_shape)
        if ctx.needs_input_grad[2]:
            g_wr = ((z_a * s) * g.sum(dim=0, keepdim=True)).reshape(wr_shape)
        if has_bias and ctx.needs_input_grad[8]:
            g_bias = g.sum(dim=(0, 2, 3))
        return g_rows, g_xs, g_wr, None, None, None, None, None, g_bias, None


def _box_sum(xs, kernel, stride, padding, dilation):
    """Sum of a one-channel tensor over every convolution window (zero padding): conv2d with an all-ones kernel."""
    kh, kw = kernel
    if tuple(dilation) == (1, 1) and 2 * padding[0] <= kh and 2 * padding[1] <= kw:
        # (no single-channel convolution: the library runs those image by image)
        return F.avg_pool2d(xs, (kh, kw), stride=stride, padding=padding, divisor_override=1)
    return F.conv2d(xs, torch.ones(1, 1, kh, kw, dtype=xs.dtype, device=xs.device), bias=None, stride=stride, padding=padding,
                    dilation=dilation)


IMPLICIT_FORWARD = True      # False: every forward pass of the uint8 layer path builds its window matrix


class _ApproxConvLayerFn(torch.autograd.Function):
    """The activation side of ApproxConv2d.forward as one operator on uint8 codes (reference ``app_layers.py:172-183`` with
    ``approx_ops.py:556-571`` inlined): quantiser -> pixel-major uint8 codes, in-range mask and channel sums in one pass;
    uint8 im2col; LUT GEMM; zero-point terms, scaling and bias from the GEMM's rows to the NCHW activation.  Backward: the
    output gradient to GEMM rows (with its row sums) in one pass, the two LUT gradient GEMMs, then col2im + gradient of the
    zero-point term + straight-through backward of the quantiser in one pass.  No float32 code tensor exists on this path.
    A 3x3 / stride 1 / padding 1 layer takes its input gradient from an implicit GEMM over the input pixels and, where no
    weight gradient will need the window matrix (``grad_mode`` off, frozen weights), its forward pass reads the pixel-major
    codes itself.  ``pre_relu``: the layer computes the convolution of max(x, 0); the quantiser's mask byte then also holds
    the ReLU's backward mask, so the gradient returned for ``x`` is the one in front of the ReLU.

    The weight side comes in one of two forms.  ``prepared`` = (b_mat uint8 [kh*kw*C, N], inside_w uint8 [N,C,kh,kw],
    w_resp float32 [N, L], tapmask float32 [kh*kw, L]) from ``approx_ops.conv_weight_prepare``: then ``w`` is the layer's real
    weight, ``w_resp`` is None and backward finishes the weight gradient itself (LUT gradient + zero-point term + the
    quantiser's straight-through backward in one launch).  Without it ``w`` holds float32 integer codes [N,C,kh,kw] and
    ``w_resp`` their response to an all-ones image, both from torch operators, which receive their gradients."""

    @staticmethod
    def forward(ctx, x, w, w_resp, taps, a_scale, a_zp, w_scale, w_zp, bias, a_qmax, stride, padding, dilation, fwd_cache=None,
                prepared=None, grad_mode=True, pre_relu=False):
        import approx_ops
        from self_ops.ops_py import approx_ops as ops
        one = lambda t: t.detach().reshape(1).contiguous()
        s_a, z_a, s_w, z_w = one(a_scale), one(a_zp), one(w_scale), one(w_zp)
        xc = x.detach().contiguous()
        bn, cin, h, w_in = xc.shape
        cout, _, kh, kw = w.shape
        s, p, d = stride[0], padding[0], dilation[0]
        oh = (h + 2 * p - d * (kh - 1) - 1) // s + 1
        ow = (w_in + 2 * p - d * (kw - 1) - 1) // s + 1
        dev = xc.device
        codes = torch.empty((bn * h * w_in, cin), dtype=torch.uint8, device=dev)
        inside = torch.empty((bn, cin, h, w_in), dtype=torch.uint8, device=dev)
        xs = torch.empty((bn, 1, h, w_in), dtype=torch.float32, device=dev)
        # (pre_relu: the layer's input is max(x, 0); `inside` then carries the ReLU's backward mask as well)
        approx_ops.quantize_codes_nhwc(xc, s_a, z_a, a_qmax, codes, inside, xs, relu=pre_relu)
        # a 3x3 / stride 1 / padding 1 layer takes its input gradient from one implicit GEMM over the input pixels (no
        # [M][9C] gradient matrix, no col2im) where the library serves the shape and the gradient table fits halves
        same3x3 = (kh, kw, s, p, d) == (3, 3, 1, 1, 1)
        # (grad_mode: whether the caller records a graph at all -- inside forward the mode is always off)
        need_x, need_w = grad_mode and ctx.needs_input_grad[0], grad_mode and ctx.needs_input_grad[1]
        conv_shaped = (same3x3 and need_x and ops.lut_grad_a_fits_halves
                       and approx_ops.conv_input_grad_supported(ops.lut_grad_a, (bn, cin, h, w_in), cout))
        # The window matrix is the operand of the weight gradient (and of a GEMM-shaped input gradient).  Where nobody will ask
        # for those (evaluation, frozen weights) the forward pass of such a layer reads the pixel-major codes itself.
        implicit = (IMPLICIT_FORWARD and same3x3 and not need_w and (conv_shaped or not need_x) and ops.lut_appmult_fits_packed
                    and approx_ops.conv_forward_implicit_supported(ops.lut_appmult, (bn, cin, h, w_in), cout))
        if (kh, kw, s, p) == (1, 1, 1, 0):
            a_mat = codes                                           # a 1x1 window is the pixel itself
        elif implicit:
            a_mat = None
        else:
            a_mat = torch.empty((bn * oh * ow, kh * kw * cin), dtype=torch.uint8, device=dev)
            approx_ops.im2col_nhwc(codes, a_mat, (bn, cin, h, w_in), (kh, kw), s, p, d)
        # rows of B in the order of A's columns: (tap, channel)
        if prepared is not None:
            b_mat, inside_w, w_resp, tapmask = prepared
        else:
            b_mat = w.detach().permute(2, 3, 1, 0).reshape(kh * kw * cin, cout).to(torch.uint8).contiguous()
            inside_w = tapmask = None
        x_sum = _box_sum(xs, (kh, kw), stride, padding, dilation)
        out = torch.empty((bn, cout, oh, ow), dtype=torch.float32, device=dev)
        # (LUT GEMM whose store applies the zero-point terms, the scaling and the bias and writes NCHW)
        dq_args = (ops.lut_appmult, x_sum.contiguous(), w_resp.detach().contiguous(), taps.contiguous(), z_a, z_w, s_a, s_w,
                   None if bias is None else bias.detach().contiguous(), out)
        cache_args = dict(cache=fwd_cache[0] if fwd_cache else None, b_version=fwd_cache[1] if fwd_cache else 0)
        if implicit:
            approx_ops.approx_conv_forward_implicit(codes, b_mat, *dq_args, (bn, cin, h, w_in), **cache_args)
        else:
            approx_ops.approx_conv_forward_dequant(a_mat, b_mat, *dq_args, **cache_args)
        ctx.save_for_backward(a_mat, b_mat, inside, s_a, z_a, s_w, z_w, codes if conv_shaped else None, inside_w, tapmask)
        ctx.geo = (bn, cin, h, w_in, cout, kh, kw, s, p, d, oh, ow)
        ctx.aux = (w_resp.shape, bias is not None, x.dtype)
        ctx.bwd_cache = (fwd_cache[2], fwd_cache[1]) if fwd_cache and len(fwd_cache) > 2 else None
        return out

    @staticmethod
    def backward(ctx, g):
        import approx_ops
        from self_ops.ops_py import approx_ops as ops
        a_mat, b_mat, inside, s_a, z_a, s_w, z_w, codes, inside_w, tapmask = ctx.saved_tensors
        bn, cin, h, w, cout, kh, kw, s, p, d, oh, ow = ctx.geo
        wr_shape, has_bias, x_dtype = ctx.aux
        fused_w = inside_w is not None
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_wr = need_w if fused_w else ctx.needs_input_grad[2]
        g = g.contiguous()
        dev = g.device
        g_x = g_w = g_wr = g_bias = None
        g_z = None
        if need_x or need_w:
            g_rows = torch.empty((bn * oh * ow, cout), dtype=torch.float32, device=dev)
            t = torch.empty(bn * oh * ow, dtype=torch.float32, device=dev)
            if need_wr and fused_w:
                # (with the gradient of the zero-point term Za * w_resp folded onto the taps, from the same pass over g where it can be)
                g_z = torch.empty((approx_ops.conv_zero_point_grad_parts(oh * ow), cout, kh * kw), dtype=torch.float32, device=dev)
                approx_ops.conv_output_grad(g, z_a, s_a, s_w, tapmask, g_rows, t, g_z)
            else:
                approx_ops.conv_dequant_backward_rowsum(g, s_a, s_w, g_rows, t)
            # (a gradient nobody asked for -- the images in front of the first layer -- is not computed)
            conv_shaped = codes is not None and need_x
            g_a = torch.empty((bn, kh * kw * cin, oh * ow), dtype=torch.float32, device=dev) if need_x and not conv_shaped else None
            g_b = torch.empty(b_mat.shape, dtype=torch.float32, device=dev) if need_w else None
            if g_a is not None or g_b is not None:
                approx_ops.approx_gemm_backward(g_rows, a_mat, b_mat, g_a, g_b, ops.lut_grad_a, ops.lut_grad_b, ga_rows_per_image=oh * ow)
            if need_x:
                g_x = torch.empty((bn, cin, h, w), dtype=torch.float32, device=dev)
                if conv_shaped:
                    bc = ctx.bwd_cache
                    approx_ops.approx_conv_input_grad(g_rows, codes, b_mat, ops.lut_grad_a, t, z_w, inside, s_a, g_x,
                                                      cache=bc[0] if bc else None, b_version=bc[1] if bc else 0)
                else:
                    approx_ops.conv_input_grad(g_a, t, z_w, inside, s_a, g_x, (kh, kw), s, p, d)
                g_x = g_x.to(x_dtype)
            if need_w and not fused_w:
                g_w = g_b.view(kh, kw, cin, cout).permute(3, 2, 0, 1)
        if need_wr and fused_w:
            # everything that ends in the real weight in one launch: LUT gradient + zero-point term, mask, weight scale
            g_w = torch.empty((cout, cin, kh, kw), dtype=torch.float32, device=dev)
            approx_ops.conv_weight_grad(g_b, g_z, inside_w, s_w, g_w)
        elif need_wr:
            g_wr = ((z_a * (s_a * s_w)) * g.sum(dim=0, keepdim=True)).reshape(wr_shape)
        if has_bias and ctx.needs_input_grad[8]:
            g_bias = g.sum(dim=(0, 2, 3))
        return g_x, g_w, g_wr, None, None, None, None, None, g_bias, None, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------ quantiser module
class AsymmetricQuantizer(nn.Module):
    """Fake quantiser used in front of the pooling layers (reference ``app_layers.py:56-74``; note that its
    rounding happens before the clamp, unlike the layer quantisers)."""

    def __init__(self, bits, observer, activation_weight_flag=False, qaft=False, union=False):
        super().__init__()
        self.observer = observer
        self.register_buffer("scale", torch.ones(1, dtype=torch.float32))
        self.register_buffer("eps", torch.tensor(torch.finfo(torch.float32).eps, dtype=torch.float32))
        self.register_buffer("quant_max_val", torch.tensor((1 << bits) - 1, dtype=torch.float32))
        self.register_buffer("zero_point_neg", torch.zeros(1, dtype=torch.float32))

    def forward(self, input):
        if self.training:
            self.scale, self.zero_point_neg = _observe(self.observer, input, self.quant_max_val, self.eps, self.scale,
                                                       self.zero_point_neg)
        q = input / self.scale - self.zero_point_neg
        q = q - q.detach() + torch.round(q)
        return (torch.clamp(q, 0, self.quant_max_val) + self.zero_point_neg) * self.scale


class _QuantParamsMixin:
    """Observers, scale / zero-point buffers shared by QuantLinear and ApproxConv2d."""

    def _init_quant(self, a_bits, w_bits):
        self.activation_observer = MovingAverageMinMaxObserver(q_level="L", out_channels=None)
        self.weight_observer = MinMaxObserver(q_level="L", out_channels=None)
        self.eps = torch.tensor(torch.finfo(torch.float32).eps, dtype=torch.float32)
        self.activation_quant_max = torch.tensor((1 << a_bits) - 1, dtype=torch.float32)
        self.register_buffer("activation_scale", torch.ones(1, dtype=torch.float32))
        self.register_buffer("activation_zp_neg", torch.zeros(1, dtype=torch.float32))
        self.weight_quant_max = torch.tensor((1 << w_bits) - 1, dtype=torch.float32)
        self.register_buffer("weight_scale", torch.ones(1, dtype=torch.float32))
        self.register_buffer("weight_zp_neg", torch.zeros(1, dtype=torch.float32))

    def _update_ranges(self, input, relu=False):
        if self.training:
            self.__dict__["_range_epoch"] = self.__dict__.get("_range_epoch", 0) + 1     # (the quantisation parameters may move)
            self.activation_scale, self.activation_zp_neg = _observe(
                self.activation_observer, input, self.activation_quant_max, self.eps, self.activation_scale, self.activation_zp_neg,
                relu=relu)
            self.weight_scale, self.weight_zp_neg = _observe(
                self.weight_observer, self.weight, self.weight_quant_max, self.eps, self.weight_scale, self.weight_zp_neg)


# ------------------------------------------------------------------------------------------ layers
class QuantLinear(nn.Linear, _QuantParamsMixin):
    """Fake-quantised fully connected layer (exact products, reference ``app_layers.py:78-113``)."""

    def __init__(self, in_features, out_features, bias=True, a_bits=8, w_bits=8):
        super().__init__(in_features, out_features, bias)
        self._init_quant(a_bits, w_bits)

    def quantize(self, x, s, zpn, qmax):
        return (_to_codes(x, s, zpn, qmax) + zpn) * s

    def forward(self, input):
        self._update_ranges(input)
        input_fq = self.quantize(input, self.activation_scale, self.activation_zp_neg, self.activation_quant_max)
        weight_fq = self.quantize(self.weight, self.weight_scale, self.weight_zp_neg, self.weight_quant_max)
        return F.linear(input_fq, weight_fq, self.bias)


class ApproxLinear(QuantLinear):
    """Fully connected layer whose code products come from the approximate-multiplier table, the way ApproxConv2d
    treats a convolution.  The reference keeps its linear layers on exact products (``app_layers.py:109-111``);
    this variant is opt-in (``prepare(..., approx_linear=True)``) for models whose classifier is to run on the
    approximate multiplier as well:  y = s_a*s_w*(AM(X,W^T) + X.Zw + Za.W^T + K*Za*Zw) + bias."""

    def __init__(self, in_features, out_features, bias=True, a_bits=8, w_bits=8, use_ste_gradient=False):
        super().__init__(in_features, out_features, bias, a_bits=a_bits, w_bits=w_bits)
        self.gemm_op = self_ops.approx_gemm_baseline_op if use_ste_gradient else self_ops.approx_gemm_op

    def forward(self, input):
        self._update_ranges(input)
        lead = input.shape[:-1]
        x_codes = _to_codes(input.reshape(-1, self.in_features), self.activation_scale, self.activation_zp_neg, self.activation_quant_max)
        w_codes = _to_codes(self.weight, self.weight_scale, self.weight_zp_neg, self.weight_quant_max)
        z_a, z_w = self.activation_zp_neg, self.weight_zp_neg
        total = self.gemm_op(x_codes, w_codes.t())
        total = total + (z_w * x_codes.sum(dim=1, keepdim=True) + z_a * w_codes.sum(dim=1).unsqueeze(0)
                         + (z_a * z_w) * float(self.in_features))
        output = self.activation_scale * self.weight_scale * total
        if self.bias is not None:
            output = output + self.bias
        return output.reshape(*lead, self.out_features)


class ApproxConv2d(nn.Conv2d, _QuantParamsMixin):
    """Convolution whose code products come from the approximate-multiplier table
    (reference ``app_layers.py:116-185``)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1, bias=True,
                 padding_mode="zeros", a_bits=8, w_bits=8, use_ste_gradient=False):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias, padding_mode)
        self._init_quant(a_bits, w_bits)
        self.conv2d_op = self_ops.approx_conv2d_baseline_op if use_ste_gradient else self_ops.approx_conv2d_op
        self.reference_zero_point_terms = False     # True: evaluate the three correction terms as full convolutions
        self.fused_dequant = True                   # False: zero-point terms and scaling as torch operators
        self.fused_layer = True                     # False: float32 code tensors between quantiser, convolution and dequantisation
        self.keep_expansion_in_eval = True          # evaluation mode: the forward table expanded along the weight codes stays on the device
        self.keep_expansions_in_training = False    # True: the expanded forward and input-gradient tables stay on the device in training
                                                    # mode too (frozen layers, gradient accumulation: weights that outlive a step)
        self.fused_weight_side = True               # False: weight codes, their all-ones response and their gradients as torch operators
        self.pre_relu = False                       # True: the layer computes conv(max(input, 0)) -- a ReLU in front folded into its quantiser

    def quantize_v2(self, x, s, zpn, qmax):
        return _to_codes(x, s, zpn, qmax)

    def _zero_point_parts(self, x_codes, w_codes, conv_args):
        """The three factors of conv(X,Zw) + conv(Za,W) + conv(Za,Zw) = Zw*x_sum + Za*w_resp + Za*Zw*taps: a convolution with a
        constant operand factorises, conv(X, Zw*1) = Zw * box-sum of X over channels and window (one
        output channel), conv(Za*1, W) = Za * (response of W to an all-ones image, batch of one), and
        conv(Za*1, Zw*1) = Za*Zw*C * (number of taps inside the image).  All quantities are integer valued,
        so as long as they stay below 2^24 the result is bit-identical to the literal form; autograd sees
        ordinary torch ops and yields the same gradients for the codes."""
        kh, kw = w_codes.shape[2], w_codes.shape[3]
        x_sum = _box_sum(x_codes.sum(dim=1, keepdim=True), (kh, kw), conv_args["stride"], conv_args["padding"], conv_args["dilation"])
        w_resp, taps = self._weight_zero_point_parts(w_codes, x_codes.shape[1:], conv_args, x_codes.dtype, x_codes.device)
        return x_sum, w_resp, taps

    def _weight_zero_point_parts(self, w_codes, chw, conv_args, dtype, device):
        """w_resp [1,N,oh,ow] = conv(all-ones image, W) and taps [1,1,oh,ow] = C * (taps inside the image)."""
        cin, h, w = chw
        cout, kh, kw = w_codes.shape[0], w_codes.shape[2], w_codes.shape[3]
        s, p, d = conv_args["stride"], conv_args["padding"], conv_args["dilation"]
        mask = self._tap_mask(h, w, kh, kw, s, p, d, dtype, device)                                  # [kh*kw, oh*ow]
        oh = (h + 2 * p[0] - d[0] * (kh - 1) - 1) // s[0] + 1
        ow = mask.shape[1] // oh
        w_resp = (w_codes.sum(dim=1).reshape(cout, kh * kw) @ mask).view(1, cout, oh, ow)           # [1,N,oh,ow]
        taps = (mask.sum(dim=0) * float(cin)).view(1, 1, oh, ow)
        return w_resp, taps

    def _tap_mask(self, h, w, kh, kw, stride, padding, dilation, dtype, device):
        """mask[i*kw+j, l] = 1 where tap (i,j) of output position l lies inside the h x w image (constant per
        geometry, cached)."""
        key = (h, w, kh, kw, tuple(stride), tuple(padding), tuple(dilation), dtype, str(device))
        cache = self.__dict__.setdefault("_tap_masks", {})
        if key not in cache:
            ones = torch.ones(1, 1, h, w, dtype=dtype, device=device)
            cache[key] = F.unfold(ones, (kh, kw), dilation=dilation, padding=padding, stride=stride)[0]
        return cache[key]

    def _frozen_weight_cache(self):
        """In evaluation mode the weight codes only change when the weights, their quantisation parameters or the tables do:
        the expansion of the forward table along them is then kept on the device between calls (approx_ops.ForwardCache) under a
        number made of everything that could change them.  Training mode: None (the weights move every step)."""
        if not (self.keep_expansions_in_training if self.training else self.keep_expansion_in_eval):
            return None
        import approx_ops
        from self_ops.ops_py import approx_ops as ops
        cache = self.__dict__.get("_fwd_cache")
        if cache is None:
            cache = self.__dict__["_fwd_cache"] = approx_ops.ForwardCache()
            self.__dict__["_bwd_cache"] = approx_ops.ForwardCache()      # (the input-gradient table expanded along the same codes)
        if self.training:
            # Every training pass leaves NEW scale / zero-point tensors, so their identity says nothing.  The weight observer keeps
            # running extremes: weights it has already seen (same tensor, same version) give the same parameters again, and with
            # them the same codes -- the weight alone identifies them.  (Any other kind of weight observer: no caching.)
            if type(self.weight_observer) is not MinMaxObserver:
                return None
            token = hash(("training", self.weight._version, self.weight.data_ptr(), float(self.weight_quant_max), ops.table_generation))
        else:
            token = hash((self.weight._version, self.weight.data_ptr(), self.weight_scale._version, self.weight_scale.data_ptr(),
                          self.weight_zp_neg._version, self.weight_zp_neg.data_ptr(), self.__dict__.get("_range_epoch", 0),
                          ops.table_generation))
        return cache, token & 0xFFFFFFFFFFFFFFFF, self.__dict__["_bwd_cache"]

    def _takes_uint8_path(self, input):
        """The one-operator path on uint8 codes serves the LUT-gradient convolution of float32 CUDA tensors with square
        geometry (the reference's operator reads element 0 of stride / padding / dilation, ``approx_ops.py:545-547``)."""
        square = all(len(set(t)) == 1 for t in (self.stride, self.padding, self.dilation)) and not isinstance(self.padding, str)
        return (self.fused_layer and self.fused_dequant and not self.reference_zero_point_terms and square and self.groups == 1
                and self.conv2d_op is self_ops.approx_conv2d_op and input.is_cuda and input.dtype == torch.float32
                and self.weight.dtype == torch.float32 and float(self.activation_quant_max) <= 255
                and self.activation_scale.is_cuda and self.weight_scale.is_cuda)

    def _prepared_weight_side(self, input, frozen):
        """(b_mat, inside_w, w_resp, tapmask) and taps of ``_ApproxConvLayerFn`` from the real weight in one launch (reference
        ``app_layers.py:173,179``: quantize_v2 on the weights and conv(Za, W)).  In evaluation mode the result is kept under the
        number of ``_frozen_weight_cache`` and the geometry."""
        import approx_ops
        cin, h, w = input.shape[1:]
        kh, kw = self.kernel_size
        key = (frozen[1], h, w) if frozen else None
        kept = self.__dict__.get("_prepared")
        if key is not None and kept is not None and kept[0] == key:
            return kept[1], kept[2]
        dev = input.device
        tapmask = self._tap_mask(h, w, kh, kw, self.stride, self.padding, self.dilation, torch.float32, dev)
        positions = tapmask.shape[1]
        oh = (h + 2 * self.padding[0] - self.dilation[0] * (kh - 1) - 1) // self.stride[0] + 1
        tkey = ("taps", h, w, cin, str(dev))
        masks = self.__dict__["_tap_masks"]
        if tkey not in masks:
            masks[tkey] = (tapmask.sum(dim=0) * float(cin)).view(1, 1, oh, positions // oh)
        cout = self.out_channels
        b_mat = torch.empty((kh * kw * cin, cout), dtype=torch.uint8, device=dev)
        inside_w = torch.empty((cout, cin, kh, kw), dtype=torch.uint8, device=dev)
        w_resp = torch.empty((cout, positions), dtype=torch.float32, device=dev)
        one = lambda t: t.detach().reshape(1).contiguous()
        approx_ops.conv_weight_prepare(self.weight.detach().contiguous(), one(self.weight_scale), one(self.weight_zp_neg),
                                       float(self.weight_quant_max), tapmask, b_mat, inside_w, w_resp)
        prepared = (b_mat, inside_w, w_resp, tapmask)
        self.__dict__["_prepared"] = (key, prepared, masks[tkey]) if key is not None else None
        return prepared, masks[tkey]

    def forward(self, input):
        uint8_path = self._takes_uint8_path(input)
        if self.pre_relu and not uint8_path:
            input = F.relu(input)                    # (the paths on float32 codes take the ReLU as its own operator)
        relu = self.pre_relu and uint8_path
        self._update_ranges(input, relu=relu)
        conv_args = dict(bias=None, stride=self.stride, padding=self.padding, dilation=self.dilation, groups=self.groups)
        if (self.fused_weight_side and uint8_path and float(self.weight_quant_max) <= 255
                and self.kernel_size[0] * self.kernel_size[1] <= 64):
            frozen = self._frozen_weight_cache()
            prepared, taps = self._prepared_weight_side(input, frozen)
            return _ApproxConvLayerFn.apply(input, self.weight, None, taps, self.activation_scale, self.activation_zp_neg,
                                            self.weight_scale, self.weight_zp_neg, self.bias, float(self.activation_quant_max),
                                            tuple(self.stride), tuple(self.padding), tuple(self.dilation), frozen, prepared,
                                            torch.is_grad_enabled(), relu)
        w_codes = self.quantize_v2(self.weight, self.weight_scale, self.weight_zp_neg, self.weight_quant_max)
        if uint8_path:
            w_resp, taps = self._weight_zero_point_parts(w_codes, input.shape[1:], conv_args, torch.float32, input.device)
            return _ApproxConvLayerFn.apply(input, w_codes, w_resp, taps, self.activation_scale, self.activation_zp_neg,
                                            self.weight_scale, self.weight_zp_neg, self.bias, float(self.activation_quant_max),
                                            tuple(self.stride), tuple(self.padding), tuple(self.dilation), self._frozen_weight_cache(),
                                            None, torch.is_grad_enabled(), relu)
        x_codes = self.quantize_v2(input, self.activation_scale, self.activation_zp_neg, self.activation_quant_max)
        total = self.conv2d_op(x_codes, w_codes, **conv_args)       # approximate products of the codes
        if self.reference_zero_point_terms:
            # the reference's literal form: three full convolutions with constant operands
            x_zp = torch.ones_like(x_codes) * self.activation_zp_neg
            w_zp = torch.ones_like(w_codes) * self.weight_zp_neg
            total = total + F.conv2d(x_codes, w_zp, **conv_args) + F.conv2d(x_zp, w_codes, **conv_args) + F.conv2d(x_zp, w_zp, **conv_args)
        else:
            z_a, z_w = self.activation_zp_neg, self.weight_zp_neg
            x_sum, w_resp, taps = self._zero_point_parts(x_codes, w_codes, conv_args)
            if total.is_cuda and total.dtype == torch.float32 and self.fused_dequant:
                rows = total.permute(0, 2, 3, 1).reshape(-1, total.shape[1])     # the GEMM's own rows: a view of the op's result
                return _ConvDequantFn.apply(rows, x_sum, w_resp, taps, z_a, z_w, self.activation_scale, self.weight_scale,
                                            self.bias, tuple(total.shape))
            total = total + (z_w * x_sum + z_a * w_resp + (z_a * z_w) * taps)
        output = self.activation_scale * self.weight_scale * total
        if self.bias is not None:
            output += self.bias.view(1, -1, 1, 1)
        return output


def _pool_quantizer(a_bits, qaft):
    return AsymmetricQuantizer(bits=a_bits, observer=MovingAverageMinMaxObserver(q_level="L", out_channels=None),
                               activation_weight_flag=1, qaft=qaft)


class QuantMaxPool2d(nn.MaxPool2d):
    def __init__(self, kernel_size, stride=None, padding=0, dilation=1, return_indices=False, ceil_mode=False, a_bits=8,
                 q_type=0, qaft=False, ptq=False, percentile=0.9999):
        super().__init__(kernel_size, stride, padding, dilation, return_indices, ceil_mode)
        self.activation_quantizer = _pool_quantizer(a_bits, qaft)

    def forward(self, input):
        return F.max_pool2d(self.activation_quantizer(input), self.kernel_size, self.stride, self.padding, self.dilation,
                            self.return_indices, self.ceil_mode)


class QuantAvgPool2d(nn.AvgPool2d):
    def __init__(self, kernel_size, stride=None, padding=0, ceil_mode=False, count_include_pad=True, divisor_override=None,
                 a_bits=8, q_type=0, qaft=False, ptq=False, percentile=0.9999):
        super().__init__(kernel_size, stride, padding, ceil_mode, count_include_pad, divisor_override)
        self.activation_quantizer = _pool_quantizer(a_bits, qaft)

    def forward(self, input):
        return F.avg_pool2d(self.activation_quantizer(input), self.kernel_size, self.stride, self.padding, self.ceil_mode,
                            self.count_include_pad, self.divisor_override)


# ------------------------------------------------------------------------------------------ model rewriting
def add_quant_op(module, a_bits=8, w_bits=8, q_type=0, q_level=0, weight_observer=0, bn_fuse=False, bn_fuse_calib=False,
                 pretrained_model=False, qaft=False, ptq=False, percentile=0.9999, use_ste_gradient=False, approx_linear=False):
    """Replace, in place and recursively, Linear / Conv2d / MaxPool2d / AvgPool2d children by their quantised
    versions; parameters are shared with the replaced module (reference ``app_layers.py:285-339``)."""
    opts = dict(a_bits=a_bits, w_bits=w_bits, q_type=q_type, q_level=q_level, weight_observer=weight_observer, bn_fuse=bn_fuse,
                bn_fuse_calib=bn_fuse_calib, pretrained_model=pretrained_model, qaft=qaft, ptq=ptq, percentile=percentile,
                use_ste_gradient=use_ste_gradient, approx_linear=approx_linear)
    for name, child in module.named_children():
        if isinstance(child, nn.Linear) and approx_linear:
            new = ApproxLinear(child.in_features, child.out_features, bias=child.bias is not None, a_bits=a_bits, w_bits=w_bits,
                               use_ste_gradient=use_ste_gradient)
        elif isinstance(child, nn.Linear):
            new = QuantLinear(child.in_features, child.out_features, bias=child.bias is not None, a_bits=a_bits, w_bits=w_bits)
        elif isinstance(child, nn.Conv2d):
            new = ApproxConv2d(child.in_channels, child.out_channels, child.kernel_size, stride=child.stride, padding=child.padding,
                               dilation=child.dilation, groups=child.groups, bias=child.bias is not None,
                               padding_mode=child.padding_mode, a_bits=a_bits, w_bits=w_bits, use_ste_gradient=use_ste_gradient)
        elif isinstance(child, nn.MaxPool2d):
            new = QuantMaxPool2d(child.kernel_size, stride=child.stride, padding=child.padding, a_bits=a_bits, q_type=q_type,
                                 qaft=qaft, ptq=ptq, percentile=percentile)
        elif isinstance(child, nn.AvgPool2d):
            new = QuantAvgPool2d(child.kernel_size, stride=child.stride, padding=child.padding, a_bits=a_bits, q_type=q_type,
                                 qaft=qaft, ptq=ptq, percentile=percentile)
        else:
            add_quant_op(child, **opts)
            continue
        if isinstance(child, (nn.Linear, nn.Conv2d)):
            new.weight.data = child.weight
            if child.bias is not None:
                new.bias.data = child.bias
        module._modules[name] = new


def fold_relu(model):
    """Inside every ``nn.Sequential`` of ``model``: a ReLU directly in front of an ApproxConv2d is replaced by ``nn.Identity``
    and the layer takes the ReLU into its quantiser (``pre_relu``): the layer observes and quantises max(x, 0) and its in-range
    mask carries the ReLU's backward mask, so the ReLU costs no pass over the activation in either direction.  Same values
    and gradients as the two modules (in a Sequential the ReLU's output has no other reader).  Returns the number of ReLUs
    folded.  An addition to the reference's ``prepare``; call it on a prepared model."""
    folded = 0
    for m in model.modules():
        if isinstance(m, nn.Sequential):
            names = list(m._modules.keys())
            for a, b in zip(names, names[1:]):
                if isinstance(m._modules[a], nn.ReLU) and isinstance(m._modules[b], ApproxConv2d) and not m._modules[b].pre_relu:
                    m._modules[a] = nn.Identity()
                    m._modules[b].pre_relu = True
                    folded += 1
    return folded


def prepare(model, inplace=False, a_bits=8, w_bits=8, q_type=0, q_level=0, weight_observer=0, bn_fuse=False, bn_fuse_calib=False,
            pretrained_model=False, qaft=False, ptq=False, percentile=0.9999, use_ste_gradient=False, approx_linear=False):
    """Return ``model`` (a deep copy unless ``inplace``) with every supported layer quantised
    (reference ``app_layers.py:342-377``; ``approx_linear`` is an addition: linear layers on the table as well)."""
    print(f'Quantizing model with a_bits={a_bits}, w_bits={w_bits}, use_ste_gradient={use_ste_gradient}')
    if not inplace:
        model = copy.deepcopy(model)
    add_quant_op(model, a_bits=a_bits, w_bits=w_bits, q_type=q_type, q_level=q_level, weight_observer=weight_observer,
                 bn_fuse=bn_fuse, bn_fuse_calib=bn_fuse_calib, pretrained_model=pretrained_model, qaft=qaft, ptq=ptq,
                 percentile=percentile, use_ste_gradient=use_ste_gradient, approx_linear=approx_linear)
    return model
