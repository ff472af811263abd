"""Autograd operators over the native LUT-GEMM (host-side mirror of ``self_ops/ops_py/approx_ops.py``).

Public names, argument meaning and error behaviour follow the reference module; the work is done by
the ``approx_ops`` native module (HIP, gfx950).  The three look-up tables live in module globals with
the reference's names (``lut_appmult``, ``lut_grad_a``, ``lut_grad_b``; reference ``approx_ops.py:13-15``).
"""
import gzip

import numpy as np
import torch
import torch.nn.functional as F
from torch.autograd import Function

import approx_ops  # native module: approx_gemm_forward / acc_gemm_forward_fp32 / approx_gemm_backward

lut_appmult = None   # uint16 padded table of the approximate products
lut_grad_a = None    # int16 padded table, 16 x d(product)/d(first operand)
lut_grad_b = None    # int16 padded table, 16 x d(product)/d(second operand)
table_generation = 0             # counts set_lookup_tables calls: part of what identifies an expansion kept between calls
lut_grad_a_fits_halves = False   # whether the expanded-table backward kernels can hold lut_grad_a as halves (int16 tables)
lut_appmult_fits_packed = False  # whether four entries of lut_appmult add up in 16 bits (the expanded-table forward kernel's packed sums)

_SECTION_HEADERS = (
    ("LUT for approximate multiplier:", 0),
    ("LUT for the gradient of the approximate multiplier w.r.t. the first operand:", 1),
    ("LUT for the gradient of the approximate multiplier w.r.t. the second operand:", 2),
)
_TAIL = {7: 638, 8: 0, 4: 718, 6: 830}


def lut_geometry(quantization_bit):
    """(rows, cols, elem_num) of the padded table (reference ``approx_ops.py:21-41``)."""
    if quantization_bit not in _TAIL:
        raise NotImplementedError(f'quantization_bit = {quantization_bit} is not supported')
    maxval = 2 ** quantization_bit - 1
    rows, cols = maxval + 2, maxval + 3
    return rows, cols, rows * cols + _TAIL[quantization_bit]


def pad_table(table2d, quantization_bit, dtype):
    """A (2^b, 2^b) table as the padded 1-D array of the boundary: entry (a, b) at a * cols + b, zeros elsewhere
    (reference ``approx_ops.py:21-41,70-77``)."""
    rows, cols, elems = lut_geometry(quantization_bit)
    n = 1 << quantization_bit
    t = np.asarray(table2d)
    assert t.shape == (n, n), f"table must be {n} x {n}"
    flat = np.zeros(elems, dtype)
    flat[:rows * cols].reshape(rows, cols)[:n, :n] = t.astype(dtype)
    return flat


def read_lut_file(file_name, quantization_bit):
    """Parse a table file into three padded 1-D NumPy arrays (uint16, int16, int16).

    Same acceptance rules as the reference's line-by-line state machine (``approx_ops.py:54-79``):
    everything before the first section header is ignored, a header switches the section, every
    other line must be ``a b value``; entries the file does not mention stay 0.  The sections are
    parsed in bulk instead of one device write per entry.  ``.gz`` files are accepted as well.
    """
    rows, cols, elems = lut_geometry(quantization_bit)
    opener = gzip.open if str(file_name).endswith(".gz") else open
    with opener(file_name, "rt") as f:
        lines = f.readlines()
    marks = []  # (line index, section id)
    for i, line in enumerate(lines):
        if line[:3] == "LUT":
            for header, sec in _SECTION_HEADERS:
                if line.startswith(header):
                    marks.append((i, sec))
                    break
    tables = [np.zeros(elems, np.uint16), np.zeros(elems, np.int16), np.zeros(elems, np.int16)]
    for j, (start, sec) in enumerate(marks):
        stop = marks[j + 1][0] if j + 1 < len(marks) else len(lines)
        body = lines[start + 1:stop]
        if not body:
            continue
        vals = np.array(" ".join(body).split(), dtype=np.int64)
        if vals.size != 3 * len(body):
            raise ValueError(f"{file_name}: every table line must hold three integers 'a b value'")
        vals = vals.reshape(-1, 3)
        idx = vals[:, 0] * cols + vals[:, 1]
        if idx.size and (idx.min() < 0 or idx.max() >= elems):
            raise IndexError(f"{file_name}: operand outside the {quantization_bit}-bit table")
        tables[sec][idx] = vals[:, 2].astype(tables[sec].dtype)
    return tables


def set_lookup_tables(device, appmult, grad_a, grad_b):
    """Install padded tables given as arrays/tensors (uint16, int16, int16); one copy per table.

    Gradient tables of a floating dtype are installed as float32 and taken as the slopes themselves (no factor 1/16):
    the backward pass then runs on the native float-table entry point."""
    global lut_appmult, lut_grad_a, lut_grad_b, lut_grad_a_fits_halves, lut_appmult_fits_packed, table_generation
    table_generation += 1
    lut_appmult_fits_packed = int(np.max(np.asarray(appmult), initial=0)) < 16384
    lut_appmult = torch.as_tensor(np.ascontiguousarray(appmult, np.uint16)).to(device)
    as_float = np.issubdtype(np.asarray(grad_a).dtype, np.floating) and np.issubdtype(np.asarray(grad_b).dtype, np.floating)
    gdt = np.float32 if as_float else np.int16
    lut_grad_a_fits_halves = (not as_float) and approx_ops.grad_table_fits_halves(np.ascontiguousarray(grad_a, np.int16))
    lut_grad_a = torch.as_tensor(np.ascontiguousarray(grad_a, gdt)).to(device)
    lut_grad_b = torch.as_tensor(np.ascontiguousarray(grad_b, gdt)).to(device)


def init_lookup_tables(device, file_name, quantization_bit):
    """Load the forward and gradient tables of an approximate multiplier onto ``device``
    (reference ``approx_ops.py:18-79``)."""
    lut_geometry(quantization_bit)  # raises NotImplementedError first, like the reference
    print(f'Initializing lookup tables from {file_name}...')
    fwd, ga, gb = read_lut_file(file_name, quantization_bit)
    set_lookup_tables(device, fwd, ga, gb)


def _codes(x):
    return x.to(torch.uint8).contiguous()


def _lut_forward(a_codes, b_codes):
    M, N = a_codes.shape[0], b_codes.shape[1]
    # float32 output: the uint32 sums converted by the kernel's store (the reference converts them in a pass of its own)
    c = torch.empty((M, N), dtype=torch.float32, device=a_codes.device)
    approx_ops.approx_gemm_forward(a_codes, b_codes, c, lut_appmult)
    return c


class AccGemm(Function):
    """Accurate fp32 GEMM through the native kernel (reference ``approx_ops.py:89-145``)."""

    @staticmethod
    def forward(ctx, a, b):
        a_c, b_c = a.contiguous().to(torch.float32), b.contiguous().to(torch.float32)
        c = torch.empty((a_c.shape[0], b_c.shape[1]), dtype=torch.float32, device=a_c.device)
        approx_ops.acc_gemm_forward_fp32(a_c, b_c, c)
        ctx.save_for_backward(a_c, b_c)
        return c

    @staticmethod
    def backward(ctx, g_c):
        assert g_c.dtype == torch.float32
        a_c, b_c = ctx.saved_tensors
        return torch.matmul(g_c, b_c.t()), torch.matmul(a_c.t(), g_c)


acc_gemm_op = AccGemm.apply


class ApproxGemm(Function):
    """LUT GEMM with LUT gradients (reference ``approx_ops.py:148-205``).

    ``a`` [M,K] and ``b`` [K,N] hold integer codes (any dtype convertible to uint8, any strides);
    returns fp32 [M,N]."""

    @staticmethod
    def forward(ctx, a, b):
        a_c, b_c = _codes(a), _codes(b)
        ctx.save_for_backward(a_c, b_c)
        return _lut_forward(a_c, b_c)

    @staticmethod
    def backward(ctx, g_c):
        assert g_c.dtype == torch.float32
        a_c, b_c = ctx.saved_tensors
        g_a = torch.empty(a_c.shape, dtype=torch.float32, device=g_c.device)
        g_b = torch.empty(b_c.shape, dtype=torch.float32, device=g_c.device)
        approx_ops.approx_gemm_backward(g_c.contiguous(), a_c, b_c, g_a, g_b, lut_grad_a, lut_grad_b)
        return g_a, g_b


approx_gemm_op = ApproxGemm.apply


class ApproxGemmBaseline(Function):
    """LUT GEMM forward, straight-through (dense) gradients on the original operands
    (reference ``approx_ops.py:210-262``)."""

    @staticmethod
    def forward(ctx, a, b):
        ctx.save_for_backward(a, b)
        return _lut_forward(_codes(a), _codes(b))

    @staticmethod
    def backward(ctx, g_c):
        assert g_c.dtype == torch.float32
        a, b = ctx.saved_tensors
        g = g_c.contiguous()
        return torch.matmul(g, b.t().contiguous()), torch.matmul(a.t().contiguous(), g)


approx_gemm_baseline_op = ApproxGemmBaseline.apply


def _conv2d_by_gemm(gemm, input, weight, bias, stride, padding, dilation, groups):
    # reference: approx_ops.py:545-571.  Only element 0 of the tuples is used; padding pixels hold
    # code 0 (not the zero-point); K index order is c*kh*kw + i*kw + j.
    assert bias is None, 'bias is not supported in approximate convolution'
    assert groups == 1, 'groups is not supported in approximate convolution'
    s, p, d = stride[0], padding[0], dilation[0]
    batch, cin, h, w = input.shape
    cout, _, kh, kw = weight.shape
    oh = (h + 2 * p - d * (kh - 1) - 1) // s + 1
    ow = (w + 2 * p - d * (kw - 1) - 1) // s + 1
    cols = F.unfold(F.pad(input, (p, p, p, p), mode='constant', value=0), kernel_size=(kh, kw), dilation=(d, d), stride=(s, s))
    lhs = cols.transpose(1, 2).reshape(-1, cin * kh * kw)      # [batch*oh*ow, cin*kh*kw]
    rhs = weight.view(cout, -1).t()                            # [cin*kh*kw, cout]
    out = gemm(lhs, rhs)                                       # [batch*oh*ow, cout]
    return out.view(batch, oh * ow, cout).transpose(1, 2).view(batch, cout, oh, ow)


def _conv_geometry(input, weight, stride, padding, dilation):
    s, p, d = stride[0], padding[0], dilation[0]
    batch, cin, h, w = input.shape
    cout, _, kh, kw = weight.shape
    oh = (h + 2 * p - d * (kh - 1) - 1) // s + 1
    ow = (w + 2 * p - d * (kw - 1) - 1) // s + 1
    return s, p, d, batch, cin, h, w, cout, kh, kw, oh, ow


def _conv_forward_codes(input, weight, geo):
    """uint8 operand matrices of the convolution and its LUT-GEMM result as fp32 [B,O,oh,ow] (a view of the
    [B*oh*ow, O] product, as the reference returns it, approx_ops.py:569-571)."""
    s, p, d, batch, cin, h, w, cout, kh, kw, oh, ow = geo
    x = input.detach().contiguous().to(torch.float32)
    a_c = torch.empty((batch * oh * ow, cin * kh * kw), dtype=torch.uint8, device=x.device)
    approx_ops.im2col_codes(x, a_c, (kh, kw), s, p, d)
    b_c = weight.detach().reshape(cout, -1).t().to(torch.uint8).contiguous()
    out = _lut_forward(a_c, b_c)
    return a_c, b_c, out.view(batch, oh * ow, cout).transpose(1, 2).view(batch, cout, oh, ow)


def _conv_grad_rows(g_out, geo):
    """[B,O,oh,ow] output gradient as the contiguous [B*oh*ow, O] matrix of the GEMM (free when the gradient
    arrives in the strides the forward result had)."""
    batch, cout, oh, ow = geo[3], geo[7], geo[10], geo[11]
    return g_out.permute(0, 2, 3, 1).reshape(batch * oh * ow, cout).contiguous()


class ApproxConv2dFn(Function):
    """Convolution of code tensors by im2col + LUT GEMM with LUT gradients: the computation of the reference's
    approx_conv2d_op (approx_ops.py:530-573) with the unfold / transpose / cast glue done by one uint8 im2col pass,
    and the input gradient produced directly in the [B, C*kh*kw, oh*ow] layout that fold consumes."""

    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation):
        geo = _conv_geometry(input, weight, stride, padding, dilation)
        a_c, b_c, out = _conv_forward_codes(input, weight, geo)
        ctx.save_for_backward(a_c, b_c)
        ctx.geo = geo
        ctx.dtypes = (input.dtype, weight.dtype)
        return out

    @staticmethod
    def backward(ctx, g_out):
        assert g_out.dtype == torch.float32
        a_c, b_c = ctx.saved_tensors
        s, p, d, batch, cin, h, w, cout, kh, kw, oh, ow = ctx.geo
        g_c = _conv_grad_rows(g_out, ctx.geo)
        # a gradient nobody asked for (the images in front of the first layer) is not computed: the reference
        # always runs both kernels (approx_gemm_backward.cu:561,588)
        need_in, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        g_a = torch.empty((batch, cin * kh * kw, oh * ow), dtype=torch.float32, device=g_c.device) if need_in else None
        g_b = torch.empty(b_c.shape, dtype=torch.float32, device=g_c.device) if need_w else None
        if need_in or need_w:
            approx_ops.approx_gemm_backward(g_c, a_c, b_c, g_a, g_b, lut_grad_a, lut_grad_b, ga_rows_per_image=oh * ow)
        g_in = None
        if need_in:
            g_in = torch.empty((batch, cin, h, w), dtype=torch.float32, device=g_c.device)
            approx_ops.col2im(g_a, g_in, (kh, kw), s, p, d)          # = F.fold(g_a, (h, w), (kh, kw), d, p, s)
            g_in = g_in.to(ctx.dtypes[0])
        g_w = g_b.t().reshape(cout, cin, kh, kw).to(ctx.dtypes[1]) if need_w else None
        return g_in, g_w, None, None, None


class ApproxConv2dBaselineFn(Function):
    """Same forward; straight-through gradients, i.e. those of an exact convolution of the code tensors
    (reference approx_conv2d_baseline_op, approx_ops.py:576-619, whose dense g_c.b^T and a^T.g_c followed by
    fold are the input and weight gradients of conv2d)."""

    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation):
        geo = _conv_geometry(input, weight, stride, padding, dilation)
        _, _, out = _conv_forward_codes(input, weight, geo)
        ctx.save_for_backward(input, weight)
        ctx.geo = geo
        return out

    @staticmethod
    def backward(ctx, g_out):
        assert g_out.dtype == torch.float32
        input, weight = ctx.saved_tensors
        s, p, d = ctx.geo[:3]
        g = g_out.contiguous()
        x, wt = input.to(torch.float32), weight.to(torch.float32)
        g_in = torch.nn.grad.conv2d_input(x.shape, wt, g, stride=s, padding=p, dilation=d)
        g_w = torch.nn.grad.conv2d_weight(x, wt.shape, g, stride=s, padding=p, dilation=d)
        return g_in.to(input.dtype), g_w.to(weight.dtype), None, None, None


def _check_conv_args(bias, groups):
    assert bias is None, 'bias is not supported in approximate convolution'
    assert groups == 1, 'groups is not supported in approximate convolution'


def approx_conv2d_op(input, weight, bias, stride, padding, dilation, groups):
    """conv2d as im2col + LUT GEMM with LUT gradients (reference ``approx_ops.py:530-573``).
    ``input`` [B,C,H,W] and ``weight`` [O,C,kh,kw] hold integer codes; returns fp32 [B,O,oh,ow].
    Only element 0 of the stride / padding / dilation tuples is used, padding pixels hold code 0 (not the
    zero-point) and the K index order is c*kh*kw + i*kw + j, all as in the reference."""
    _check_conv_args(bias, groups)
    return ApproxConv2dFn.apply(input, weight, tuple(stride), tuple(padding), tuple(dilation))


def approx_conv2d_baseline_op(input, weight, bias, stride, padding, dilation, groups):
    """Same forward, straight-through gradients (reference ``approx_ops.py:576-619``)."""
    _check_conv_args(bias, groups)
    return ApproxConv2dBaselineFn.apply(input, weight, tuple(stride), tuple(padding), tuple(dilation))


def approx_conv2d_unfold_op(input, weight, bias, stride, padding, dilation, groups):
    """approx_conv2d_op composed exactly as the reference composes it (pad, unfold, transpose, GEMM op); kept as the
    cross-check of the fused path."""
    return _conv2d_by_gemm(approx_gemm_op, input, weight, bias, stride, padding, dilation, groups)


def approx_conv2d_baseline_unfold_op(input, weight, bias, stride, padding, dilation, groups):
    return _conv2d_by_gemm(approx_gemm_baseline_op, input, weight, bias, stride, padding, dilation, groups)
