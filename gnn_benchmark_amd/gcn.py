"""A GCN layer stack around the aggregation path, used for the full train-step workload.

The aggregation is the reference's ``Aggregator`` contract (aggregate-then-transform, the
order of self_benchmark/a64fx/model/layers/sageconv.py:65-93: ``out = Aggregator(...)``,
``out /= graph.in_degrees``, then the dense transform).  Everything after the
aggregation is this build's own definition of the workload: one weight matrix per layer
(``Z = ((A X) W) / deg + b`` -- the degree normalisation is applied behind the dense
product, where it fuses into the epilogue: D^-1 (A X) W == D^-1 ((A X) W)), ReLU, dropout
with a precomputed seeded mask, log-softmax + NLL on the labelled nodes, Adam.  Every dense
product runs on the matrix cores in libgnnagg's own kernels wherever they take the widths
(inner width a multiple of 16 -- or padded to one for the input gradient --, at most 256 output
columns per call): with dense activations a layer runs fused (``_FusedLayer``): the product
(fp32, or bf16 inputs), the degree division, bias, ReLU and dropout are one kernel, and in the
gradient direction the ReLU / dropout mask, the degree division, the bias gradient and the weight
gradient are another, plus the input-gradient product (the same product kernel).  The forms
that keep the product apart from the elementwise passes (``fused_layers=False``, a layer that
multiplies first, packed activations in front of the product) call the same product kernel
bare.  ``gemm="bf16x3"`` keeps fp32 accuracy but feeds the matrix units every fp32 operand as
three bf16 pieces (six bf16 MFMAs a product, a fraction of the fp32 MFMA's cycles); plain
``gemm="fp32"`` products (no epilogue) run that way too, where it is the fastest fp32-accurate
form.  What the kernels do not take falls through to the BLAS library behind ``torch.mm`` --
never silently: every such call goes through ``library_product``, which counts it
(``LIBRARY_PRODUCTS``) and raises under ``forbid_library_products()``.
"""
import contextlib
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F

from . import _lib, packed
from . import aggregator as aggregator_module
from .aggregator import Aggregator, AggregatorPacked
from .sparse_tensor import _row_stride, _rows_are_dense


# Dense products that libgnnagg's kernels do not take go to the BLAS library through this one door.  The counter says
# how many did (a benchmark reports it per train step); ``forbid_library_products()`` turns every such call into an
# error, for runs that must stay on the hand-written kernels.
LIBRARY_PRODUCTS = {"count": 0, "forbidden": False}


def library_product(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None, bf16_inputs: bool = False,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``a @ b (+ bias)`` by the BLAS library (``bf16_inputs``: operands rounded to bf16, fp32 accumulation and
    result), counted in ``LIBRARY_PRODUCTS``."""
    if LIBRARY_PRODUCTS["forbidden"]:
        raise RuntimeError("a dense product [%d, %d] @ [%d, %d] that libgnnagg's kernels do not take fell through to "
                           "the BLAS library under forbid_library_products()" % (tuple(a.shape) + tuple(b.shape)))
    LIBRARY_PRODUCTS["count"] += 1
    if bf16_inputs:
        y = torch.mm(a.to(torch.bfloat16), b.to(torch.bfloat16), out_dtype=torch.float32)
        y = y if bias is None else y + bias
        return y if out is None else out.copy_(y)
    if bias is not None:
        return torch.addmm(bias, a, b) if out is None else torch.addmm(bias, a, b, out=out)
    return torch.mm(a, b) if out is None else torch.mm(a, b, out=out)


@contextlib.contextmanager
def forbid_library_products():
    """Inside the block a dense product that would go to the BLAS library raises instead."""
    previous = LIBRARY_PRODUCTS["forbidden"]
    LIBRARY_PRODUCTS["forbidden"] = True
    try:
        yield
    finally:
        LIBRARY_PRODUCTS["forbidden"] = previous


def plain_product(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor], form: int) -> torch.Tensor:
    """``a @ b (+ bias)`` without an epilogue, in libgnnagg's product kernel where it takes the widths: operands
    rounded to bf16 for ``BF16``, every operand as three bf16 pieces for ``FP32`` and ``BF16X3`` alike (fp32 accuracy;
    for a plain product faster than the fp32 matrix instruction and than the BLAS library's fp32 product -- 7 M x 512
    x 256: 10.8 ms against 14.8 and 12.9).  The BLAS library, counted, otherwise."""
    if (a.is_cuda and a.dtype == torch.float32 and a.size(0) > 0
            and _lib.lib().gnnagg_linear_shape_supported(a.size(1), b.size(1))):
        return _fused_product(_kernel_ready(a), b.contiguous(), None if bias is None else bias.contiguous(), None, None,
                              1.0, False, BF16 if form == BF16 else BF16X3)
    return library_product(a, b, bias, bf16_inputs=form == BF16)


class _Bf16InputLinear(torch.autograd.Function):
    """y = x @ w with x, w rounded to bf16, products accumulated in fp32, fp32 result; the
    input gradient is computed the same way.  The weight gradient stays in fp32: the
    hand-written kernel reads the fp32 operands as they are, which is faster than rounding
    7 M-row operands to bf16 first, and more exact."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return plain_product(x, w, None, BF16)

    @staticmethod
    def backward(ctx, g):
        x, w = ctx.saved_tensors
        gx = input_gradient(g, w, BF16) if ctx.needs_input_grad[0] else None
        gw = weight_gradient(x, g) if ctx.needs_input_grad[1] else None
        return gx, gw


def weight_gradient(x: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """x^T @ g for tall-skinny fp32 operands through libgnnagg's MFMA kernel; the BLAS library (counted) for shapes
    that kernel does not take (more than 256 columns).  Column blocks of wider row-major tensors are read where they
    lie."""
    if not _rows_are_dense(x):
        x = x.contiguous()
    if not _rows_are_dense(g):
        g = g.contiguous()
    rows, fi, fo = x.size(0), x.size(1), g.size(1)
    L = _lib.lib()
    nbytes = int(L.gnnagg_wgrad_workspace_bytes(rows, fi, fo)) if x.is_cuda and x.dtype == torch.float32 else 0
    if nbytes == 0:
        return library_product(x.t(), g)
    out = torch.empty(fi, fo, dtype=torch.float32, device=x.device)
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(L.gnnagg_wgrad_strided_f32(_lib.ptr(x), _row_stride(x), _lib.ptr(g), _row_stride(g), _lib.ptr(out),
                                              _lib.ptr(workspace), nbytes, rows, fi, fo,
                                              _lib.current_stream(x.device)))
    return out


def weight_and_bias_gradient(x: torch.Tensor, g: torch.Tensor, form: int = 0):
    """(x^T @ g, g.sum(0)): the column sums come out of the weight-gradient kernel's pass over g.
    Falls back to separate torch ops for shapes the kernel does not take.  ``form`` ``BF16X3``: the product
    with every operand as three bf16 pieces (fp32 accuracy, fewer matrix-unit cycles)."""
    x, g = _kernel_ready(x), _kernel_ready(g)
    rows, fi, fo = x.size(0), x.size(1), g.size(1)
    L = _lib.lib()
    ok = x.is_cuda and x.dtype == torch.float32 and g.dtype == torch.float32
    nbytes = int(L.gnnagg_wgrad_relu_dropout_backward_workspace_bytes(rows, fi, fo)) if ok else 0
    if nbytes == 0:
        return weight_gradient(x, g), g.sum(dim=0)
    grad_w = torch.empty(fi, fo, dtype=torch.float32, device=x.device)
    grad_b = torch.empty(fo, dtype=torch.float32, device=x.device)
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        entry = L.gnnagg_wgrad_relu_dropout_backward_bf16x3_f32 if form == 2 else L.gnnagg_wgrad_relu_dropout_backward_f32
        _lib.check(entry(
            _lib.ptr(x), _row_stride(x), _lib.ptr(g), _row_stride(g), None, 0, None, 1.0, None, _lib.ptr(grad_w),
            _lib.ptr(grad_b), _lib.ptr(workspace), nbytes, rows, fi, fo, _lib.current_stream(x.device)))
    return grad_w, grad_b


class _Fp32Linear(torch.autograd.Function):
    """y = x @ w to fp32 accuracy: the product and the input-gradient product in libgnnagg's product kernel (three
    bf16 pieces an operand), the weight gradient (a reduction over millions of rows) in its fp32 MFMA kernel."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return plain_product(x, w, None, FP32)

    @staticmethod
    def backward(ctx, g):
        x, w = ctx.saved_tensors
        gx = input_gradient(g, w, FP32) if ctx.needs_input_grad[0] else None
        gw = weight_gradient(x, g) if ctx.needs_input_grad[1] else None
        return gx, gw


_Bf16x3Linear = _Fp32Linear   # a bare product has one fp32-accurate form: the two names run the same kernels


def pack_keep_mask(keep: torch.Tensor) -> torch.Tensor:
    """Bool / uint8 keep-mask [rows, feat] -> int32 [rows, ceil(feat / 32)]: bit q of word (r, v)
    is keep[r, 32 v + q].  The form the fused layer kernel reads (1 bit instead of 1 byte per unit)."""
    if not keep.is_cuda or keep.dtype not in (torch.bool, torch.uint8) or keep.dim() != 2 or not keep.is_contiguous():
        raise RuntimeError("Input mismatch: keep must be a contiguous bool/uint8 [rows, feat] GPU (HIP) tensor")
    rows, feat = keep.shape
    bits = torch.empty(rows, (feat + 31) // 32, dtype=torch.int32, device=keep.device)
    with torch.cuda.device(keep.device):
        _lib.check(_lib.lib().gnnagg_pack_keep_bits(_lib.ptr(keep), _lib.ptr(bits), rows, feat,
                                                    _lib.current_stream(keep.device)))
    return bits


def _row_divisors(graph):
    """The in-degrees a layer divides its aggregation by, or None when the graph's matrices already carry that
    division in their values (``sage.fold_in_degrees``)."""
    return None if getattr(graph, "in_degrees_folded", False) else graph.in_degrees


def fused_layer_supported(x: torch.Tensor, in_channels: int, out_channels: int) -> bool:
    """Whether ``_FusedLayer`` takes a [rows, in_channels] operand on x's device and these widths."""
    if not (x.is_cuda and x.dtype == torch.float32):
        return False
    L = _lib.lib()
    return bool(L.gnnagg_linear_shape_supported(in_channels, out_channels)
                and L.gnnagg_wgrad_relu_dropout_backward_workspace_bytes(max(x.size(0), 1), in_channels, out_channels) > 0)


def _kernel_ready(x: torch.Tensor) -> torch.Tensor:
    """x as the fused kernels read it: dense rows, 16-byte aligned rows."""
    if x.dim() == 2 and _rows_are_dense(x) and _row_stride(x) % 4 == 0 and x.data_ptr() % 16 == 0:
        return x
    return x.contiguous()


# how the matrix units see the fp32 operands of a product (the result is accumulated and returned in fp32):
FP32, BF16, BF16X3 = 0, 1, 2  # as they are / rounded to bf16 / as three bf16 pieces each (six bf16 MFMAs a product:
#                               fp32 accuracy at a fraction of the fp32 MFMA's cycles)
_FORMS = {"fp32": FP32, "bf16": BF16, "bf16x3": BF16X3}


def _fused_product(x, w, bias, keep_bits, row_div, scale, relu, form, out=None):
    """The one-kernel layer product of libgnnagg on kernel-ready operands (``out``: a kernel-ready [rows, n] array,
    e.g. a column block of a wider one, to write into)."""
    rows, k, n = x.size(0), x.size(1), w.size(1)
    y = torch.empty(rows, n, dtype=torch.float32, device=x.device) if out is None else out
    L = _lib.lib()
    entry = (L.gnnagg_linear_bias_relu_dropout_f32, L.gnnagg_linear_bias_relu_dropout_bf16_f32,
             L.gnnagg_linear_bias_relu_dropout_bf16x3_f32)[int(form)]
    with torch.cuda.device(x.device):
        _lib.check(entry(_lib.ptr(x), _row_stride(x), _lib.ptr(w), n, _lib.ptr(bias), _lib.ptr(keep_bits),
                         _lib.ptr(row_div), float(scale), 1 if relu else 0, _lib.ptr(y), _row_stride(y), rows, k, n,
                         _lib.current_stream(x.device)))
    return y


def stacked_product(cat: torch.Tensor, weight: torch.Tensor, bias, form: int) -> torch.Tensor:
    """cat @ weight (+ bias): ``plain_product`` (the SAGE layer's [A x | x] @ [W_neigh ; W_self])."""
    return plain_product(cat, weight, bias, form)


def input_gradient(g: torch.Tensor, weight: torch.Tensor, form: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """g @ weight^T, [rows, weight rows], through libgnnagg's product kernel: one call per block of at most 256 output
    columns, each writing its columns of the result.  ``form`` ``BF16`` rounds the operands to bf16; ``FP32`` and
    ``BF16X3`` both feed every operand as three bf16 pieces -- fp32 accuracy (errors at the level of the BLAS library's
    fp32 product), and for this plain product faster than the fp32 matrix instruction and than the library
    (7 M x 256 x 256: 5.8 ms against 8.0 and 7.0).  An inner width that is no multiple of 16 goes through a zero-padded
    copy of ``g``.  ``out``: a [rows, weight rows] array with kernel-ready rows (a column block of a wider one is fine)
    to write into.  The BLAS library's product, counted, only for what the kernel does not take."""
    wide, inner = weight.size(0), weight.size(1)
    blocks = [(c, min(c + 256, wide)) for c in range(0, wide, 256)]
    L = _lib.lib()
    padded = inner + (-inner) % 16
    if (g.is_cuda and g.dtype == torch.float32 and g.size(0) > 0 and wide % 4 == 0
            and all(L.gnnagg_linear_shape_supported(padded, hi - lo) for lo, hi in blocks)):
        if padded != inner:
            g = torch.nn.functional.pad(g, (0, padded - inner))
            weight = torch.nn.functional.pad(weight, (0, padded - inner))
        g = _kernel_ready(g)
        kernel_form = BF16 if form == BF16 else BF16X3
        if out is None:
            out = torch.empty(g.size(0), wide, dtype=torch.float32, device=g.device)
        elif (out.shape != (g.size(0), wide) or out.dtype != torch.float32 or not _rows_are_dense(out)
              or _row_stride(out) % 4 != 0 or out.data_ptr() % 16 != 0):
            raise RuntimeError("Input mismatch: out must be float32 [rows, weight rows] with 16-byte aligned rows")
        for lo, hi in blocks:
            _fused_product(g, weight[lo:hi].t().contiguous(), None, None, None, 1.0, False, kernel_form, out=out[:, lo:hi])
        return out
    return library_product(g, weight.t(), bf16_inputs=form == BF16, out=out)


class _FusedLayer(torch.autograd.Function):
    """y = relu((x @ w) / row_div + bias) * (keep ? scale : 0) in one kernel (``relu`` False and
    ``keep_bits`` None: y = (x @ w) / row_div + bias, the last layer).  The gradient direction
    is one more kernel -- mask, degree division, bias gradient and weight gradient in a single
    pass over x, the incoming gradient and y -- plus the product for the input gradient.  With
    ``form`` ``BF16`` all three products round their operands to bf16 on the way into the matrix units
    (fp32 accumulation); with ``BF16X3`` they feed every operand as three bf16 pieces (fp32 accuracy); mask,
    division and bias gradient stay in fp32.  The input-gradient product is ``input_gradient``: libgnnagg's kernel in
    every form (three bf16 pieces an operand for ``FP32`` too), no BLAS-library call."""

    @staticmethod
    def forward(ctx, x, w, bias, keep_bits, scale, row_div, relu, form=FP32):
        rows, k, n = x.size(0), x.size(1), w.size(1)
        if keep_bits is not None and (keep_bits.dtype != torch.int32 or keep_bits.shape != (rows, (n + 31) // 32)
                                      or not keep_bits.is_contiguous()):
            raise RuntimeError("Input mismatch: keep_bits must be contiguous int32 [rows, ceil(feat / 32)] "
                               "(gcn.pack_keep_mask)")
        if row_div is not None and (row_div.dtype != torch.float32 or row_div.numel() != rows
                                    or not row_div.is_contiguous()):
            raise RuntimeError("Input mismatch: row_div must be contiguous float32 with one entry per row")
        if keep_bits is not None and not relu:
            # the gradient reads which units count off the output (y > 0), which needs the ReLU in front
            raise RuntimeError("Input mismatch: the fused layer applies dropout behind a ReLU only")
        w = w.contiguous()
        y = _fused_product(x, w, bias.contiguous(), keep_bits, row_div, scale, relu, form)
        ctx.save_for_backward(x, w, y if relu else None)
        ctx.scale = float(scale)
        ctx.row_div = row_div
        ctx.form = int(form)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, w, y = ctx.saved_tensors
        grads = _fused_backward(x, w, grad_y, y, None, ctx.row_div, ctx.scale, ctx.form, ctx.needs_input_grad[0])
        return grads + (None, None, None, None, None)


def _fused_backward(x, w, grad_y, y, header, row_div, scale, form, want_x):
    """(grad_x, grad_w, grad_bias) of the fused layer: one pass of the weight-gradient kernel (mask from ``y`` or from
    the packed output's ``header``, degree division, bias gradient, weight gradient) plus the input-gradient product."""
    grad_y = _kernel_ready(grad_y)
    rows, k, n = x.size(0), x.size(1), w.size(1)
    L = _lib.lib()
    nbytes = int(L.gnnagg_wgrad_relu_dropout_backward_workspace_bytes(max(rows, 1), k, n))
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    grad_z = torch.empty(rows, n, dtype=torch.float32, device=x.device) if want_x else None
    grad_w = torch.empty(k, n, dtype=torch.float32, device=x.device)
    grad_bias = torch.empty(n, dtype=torch.float32, device=x.device)
    stream = _lib.current_stream(x.device)
    with torch.cuda.device(x.device):
        if header is not None:
            _lib.check(L.gnnagg_wgrad_relu_dropout_backward_from_header_f32(
                _lib.ptr(x), _row_stride(x), _lib.ptr(grad_y), _row_stride(grad_y), _lib.ptr(header), _lib.ptr(row_div),
                scale, _lib.ptr(grad_z), _lib.ptr(grad_w), _lib.ptr(grad_bias), _lib.ptr(workspace), nbytes, rows, k, n,
                int(form), stream))
        else:
            entry = (L.gnnagg_wgrad_relu_dropout_backward_f32, L.gnnagg_wgrad_relu_dropout_backward_bf16_f32,
                     L.gnnagg_wgrad_relu_dropout_backward_bf16x3_f32)[int(form)]
            _lib.check(entry(_lib.ptr(x), _row_stride(x), _lib.ptr(grad_y), _row_stride(grad_y), _lib.ptr(y),
                             n if y is not None else 0, _lib.ptr(row_div), scale, _lib.ptr(grad_z), _lib.ptr(grad_w),
                             _lib.ptr(grad_bias), _lib.ptr(workspace), nbytes, rows, k, n, stream))
    grad_x = input_gradient(grad_z, w, form) if want_x else None
    return grad_x, grad_w, grad_bias


class _FusedLayerPacked(torch.autograd.Function):
    """``_FusedLayer`` writing its result packed (``packed.py``): returns ``(values, header)``.  The gradient that comes
    back for ``values`` is the one with respect to the dense activations the pair stands for (``AggregatorPacked``
    returns exactly that); which units were active is read from the header's bitmaps."""

    @staticmethod
    def forward(ctx, x, w, bias, keep_bits, scale, row_div, form):
        rows, k, n = x.size(0), x.size(1), w.size(1)
        if keep_bits is not None and (keep_bits.dtype != torch.int32 or keep_bits.shape != (rows, (n + 31) // 32)
                                      or not keep_bits.is_contiguous()):
            raise RuntimeError("Input mismatch: keep_bits must be contiguous int32 [rows, ceil(feat / 32)] "
                               "(gcn.pack_keep_mask)")
        if row_div is not None and (row_div.dtype != torch.float32 or row_div.numel() != rows
                                    or not row_div.is_contiguous()):
            raise RuntimeError("Input mismatch: row_div must be contiguous float32 with one entry per row")
        w = w.contiguous()
        values, header = packed.empty(rows, n, x.device)
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().gnnagg_linear_bias_relu_dropout_pack_f32(
                _lib.ptr(x), _row_stride(x), _lib.ptr(w), n, _lib.ptr(bias.contiguous()), _lib.ptr(keep_bits),
                _lib.ptr(row_div), float(scale), _lib.ptr(values), _lib.ptr(header), rows, k, n, int(form),
                _lib.current_stream(x.device)))
        ctx.mark_non_differentiable(header)
        ctx.save_for_backward(x, w, header)
        ctx.scale = float(scale)
        ctx.row_div = row_div
        ctx.form = int(form)
        return values, header

    @staticmethod
    def backward(ctx, grad_y, _grad_header):
        x, w, header = ctx.saved_tensors
        grads = _fused_backward(x, w, grad_y, None, header, ctx.row_div, ctx.scale, ctx.form, ctx.needs_input_grad[0])
        return grads + (None, None, None, None)


class _BiasReluDropout(torch.autograd.Function):
    """y = relu(z / row_div + bias) * (keep ? scale : 0), one fused pass, written over ``z``
    (the GEMM output, which nothing else reads); the gradient needs only ``y``."""

    @staticmethod
    def forward(ctx, z, bias, keep, scale, row_div):
        if not z.is_cuda:
            raise RuntimeError("the fused epilogue runs on a GPU (HIP) device only")
        if z.dtype != torch.float32 or bias.dtype != torch.float32 or not z.is_contiguous() or z.dim() != 2:
            raise RuntimeError("Input mismatch: z must be contiguous float32 [rows, feat]")
        if keep is not None and (keep.dtype not in (torch.bool, torch.uint8) or keep.shape != z.shape
                                 or not keep.is_contiguous()):
            raise RuntimeError("Input mismatch: keep must be a contiguous bool/uint8 mask shaped like z")
        if row_div is not None and (row_div.dtype != torch.float32 or row_div.numel() != z.size(0)
                                    or not row_div.is_contiguous()):
            raise RuntimeError("Input mismatch: row_div must be contiguous float32 with one entry per row")
        with torch.cuda.device(z.device):
            _lib.check(_lib.lib().gnnagg_bias_relu_dropout_f32(
                _lib.ptr(z), _lib.ptr(bias.contiguous()), _lib.ptr(keep), _lib.ptr(row_div), float(scale), _lib.ptr(z),
                z.size(0), z.size(1), _lib.current_stream(z.device)))
        ctx.mark_dirty(z)
        ctx.save_for_backward(z)
        ctx.scale = float(scale)
        ctx.row_div = row_div
        return z

    @staticmethod
    def backward(ctx, grad_y):
        (y,) = ctx.saved_tensors
        grad_y = grad_y.contiguous()
        grad_z = torch.empty_like(grad_y)
        row_div = ctx.row_div
        L = _lib.lib()
        # d/d bias sums the gradient BEFORE the per-row division; where the width allows, the
        # kernel emits per-block partial sums of exactly that in the same pass
        blocks = int(L.gnnagg_relu_dropout_backward_blocks(y.size(0), y.size(1))) if ctx.needs_input_grad[1] else 0
        partial = torch.empty(blocks, y.size(1), dtype=torch.float32, device=y.device) if blocks else None
        with torch.cuda.device(y.device):
            _lib.check(L.gnnagg_relu_dropout_backward_f32(
                _lib.ptr(grad_y), _lib.ptr(y), _lib.ptr(row_div), ctx.scale, _lib.ptr(grad_z), _lib.ptr(partial),
                y.size(0), y.size(1), _lib.current_stream(y.device)))
        grad_bias = None
        if ctx.needs_input_grad[1]:
            if partial is not None:
                grad_bias = partial.sum(dim=0)
            elif row_div is None:
                grad_bias = grad_z.sum(dim=0)
            else:
                grad_bias = (grad_z * row_div.view(-1, 1)).sum(dim=0)
        return grad_z, grad_bias, None, None, None


class _BiasReluDropoutPacked(torch.autograd.Function):
    """The same epilogue writing its result packed (``packed.py``): returns ``(values,
    header)``.  The gradient that comes back for ``values`` is the one with respect to the
    dense activations the pair stands for (``AggregatorPacked`` returns exactly that); which
    units were active is read from the header's bitmap."""

    @staticmethod
    def forward(ctx, z, bias, keep, scale, row_div):
        if not z.is_cuda or z.dtype != torch.float32 or not z.is_contiguous() or z.dim() != 2:
            raise RuntimeError("Input mismatch: z must be a contiguous float32 [rows, feat] GPU (HIP) tensor")
        values, header = packed.empty(z.size(0), z.size(1), z.device)
        with torch.cuda.device(z.device):
            _lib.check(_lib.lib().gnnagg_bias_relu_dropout_pack_f32(
                _lib.ptr(z), _lib.ptr(bias.contiguous()), _lib.ptr(keep), _lib.ptr(row_div), float(scale),
                _lib.ptr(values), _lib.ptr(header), z.size(0), z.size(1), _lib.current_stream(z.device)))
        ctx.mark_non_differentiable(header)
        ctx.save_for_backward(header)
        ctx.scale = float(scale)
        ctx.row_div = row_div
        return values, header

    @staticmethod
    def backward(ctx, grad_y, _grad_header):
        (header,) = ctx.saved_tensors
        grad_y = grad_y.contiguous()
        rows, feat = grad_y.shape
        grad_z = torch.empty_like(grad_y)
        L = _lib.lib()
        blocks = int(L.gnnagg_relu_dropout_backward_blocks(rows, feat))
        partial = torch.empty(blocks, feat, dtype=torch.float32, device=grad_y.device)
        with torch.cuda.device(grad_y.device):
            _lib.check(L.gnnagg_relu_dropout_backward_packed_f32(
                _lib.ptr(grad_y), _lib.ptr(header), _lib.ptr(ctx.row_div), ctx.scale, _lib.ptr(grad_z),
                _lib.ptr(partial), rows, feat, _lib.current_stream(grad_y.device)))
        grad_bias = partial.sum(dim=0) if ctx.needs_input_grad[1] else None
        return grad_z, grad_bias, None, None, None


class GCNLayer(torch.nn.Module):
    def __init__(self, in_channels: int, out_channels: int, gemm: str = "fp32", num_bits: int = 32):
        super().__init__()
        if gemm not in _FORMS:
            raise ValueError("gemm must be 'fp32', 'bf16' or 'bf16x3'")
        self.gemm = gemm
        self.num_bits = num_bits  # width of the boundary rows on the wire (``Aggregator``'s fourth argument)
        self.linear_first = False
        self.fuse = True  # use the fused layer kernels where they apply
        self.weight = torch.nn.Parameter(torch.empty(in_channels, out_channels))
        self.bias = torch.nn.Parameter(torch.zeros(out_channels))
        torch.nn.init.xavier_uniform_(self.weight, gain=torch.nn.init.calculate_gain("relu"))

    def _product(self, t: torch.Tensor) -> torch.Tensor:
        if self.gemm == "bf16":
            return _Bf16InputLinear.apply(t, self.weight)
        if self.gemm == "bf16x3":
            return _Bf16x3Linear.apply(t, self.weight)
        return _Fp32Linear.apply(t, self.weight)

    def transform(self, graph, x, layer: int, is_pre_delay: bool) -> torch.Tensor:
        """(A x) W: neither the degree normalisation nor the bias yet.  ``x`` is a dense tensor
        or a packed ``(values, header)`` pair.  With ``linear_first`` (and dense ``x``) the
        product comes first, A (x W): the same up to rounding, and the aggregation, its backward
        and the boundary rows then have the output width."""
        if isinstance(x, tuple):
            agg = AggregatorPacked.apply(graph, x[0], x[1], layer, self.num_bits, is_pre_delay, self.training)
            return self._product(agg)
        if self.linear_first:
            return Aggregator.apply(graph, self._product(x), layer, self.num_bits, is_pre_delay, self.training)
        return self._product(Aggregator.apply(graph, x, layer, self.num_bits, is_pre_delay, self.training))

    def fused(self, graph, x, layer: int, is_pre_delay: bool, keep_bits, scale: float, relu: bool,
              pack_out: bool = False):
        """relu(((A x) W) / deg + bias) * keep * scale through the fused kernels -- dense, or as a packed
        ``(values, header)`` pair with ``pack_out`` -- or None where they do not apply (product-first order, widths
        the kernels do not take).  ``x`` is a dense tensor or a packed pair."""
        if self.linear_first or not self.fuse:
            return None
        probe = x[0] if isinstance(x, tuple) else x
        if not fused_layer_supported(probe, self.weight.size(0), self.weight.size(1)):
            return None
        if isinstance(x, tuple):
            agg = AggregatorPacked.apply(graph, x[0], x[1], layer, self.num_bits, is_pre_delay, self.training)
        else:
            agg = Aggregator.apply(graph, x, layer, self.num_bits, is_pre_delay, self.training)
        agg = _kernel_ready(agg)
        row_div = _row_divisors(graph)
        row_div = None if row_div is None else row_div.reshape(-1)
        form = _FORMS[self.gemm]
        if pack_out:
            return _FusedLayerPacked.apply(agg, self.weight, self.bias, keep_bits, scale, row_div, form)
        return _FusedLayer.apply(agg, self.weight, self.bias, keep_bits, scale, row_div, relu, form)

    def forward(self, graph, x: torch.Tensor, layer: int, is_pre_delay: bool) -> torch.Tensor:
        """((A x) W) / deg + bias."""
        out = self.fused(graph, x, layer, is_pre_delay, None, 1.0, False)
        if out is not None:
            return out
        z, row_div = self.transform(graph, x, layer, is_pre_delay), _row_divisors(graph)
        return z + self.bias if row_div is None else torch.addcdiv(self.bias, z, row_div)


class GCN(torch.nn.Module):
    def __init__(self, dims: Sequence[int], gemm: str = "fp32", dropout: float = 0.5, packed_activations: bool = False,
                 linear_first_when_narrowing: bool = False, fused_layers: bool = True, num_bits: int = 32):
        super().__init__()
        self.layers = torch.nn.ModuleList([GCNLayer(dims[i], dims[i + 1], gemm, num_bits) for i in range(len(dims) - 1)])
        for layer in self.layers:  # one-kernel layers where they apply (fp32 products, dense activations)
            layer.fuse = fused_layers
        if linear_first_when_narrowing:  # a layer with fewer outputs than inputs aggregates its outputs
            for i, layer in enumerate(self.layers):
                layer.linear_first = dims[i + 1] < dims[i]
        self.dropout = dropout
        # keep hidden activations packed (non-zero values + bitmap) where their width allows and
        # pre-aggregation is used: the next layer's aggregation then skips the zeros
        self.packed_activations = packed_activations
        self._mask_cache = {}

    def _packed_mask(self, mask: torch.Tensor) -> torch.Tensor:
        """Bit-packed form of a bool mask, remembered while the same tensor (unchanged) comes back --
        the seeded masks of a benchmark or test are reused step after step."""
        key = (mask.data_ptr(), tuple(mask.shape), mask._version)
        hit = self._mask_cache.get(key)
        if hit is None:
            if len(self._mask_cache) >= 2 * len(self.layers):
                self._mask_cache.clear()
            hit = self._mask_cache[key] = (mask, pack_keep_mask(mask))  # holding the mask keeps its address its own
        return hit[1]

    def forward(self, graph, x: torch.Tensor, is_pre_delay: bool, masks: Optional[List[torch.Tensor]] = None,
                log_probs: bool = True, last_rows: Optional[torch.Tensor] = None,
                hidden: Optional[list] = None) -> torch.Tensor:
        """``masks[l]``: keep-mask of the dropout after layer l (training only): bool [N, dims[l+1]], or
        its bit-packed form (``pack_keep_mask``) for a layer that runs fused.  ``log_probs=False``
        returns the last layer's output before the log-softmax.  ``last_rows`` (local node ids): evaluate the last
        layer for those nodes only and return ``[len(last_rows), classes]`` -- the rows a loss over them needs, at a
        fraction of the last aggregation and product, forward and backward (``aggregator.restrict_output_rows``).
        ``hidden``: a list that receives every hidden layer's output (the tensors themselves -- a ``(values, header)``
        pair where activations are kept packed), for callers that want to look at them."""
        h = x
        last = len(self.layers) - 1
        for l, layer in enumerate(self.layers):
            if hidden is not None and l > 0:
                hidden.append(h)
            if l == last:
                g_last = graph
                if last_rows is not None:
                    g_last = aggregator_module.restrict_output_rows(graph, last_rows, is_pre_delay)
                h = layer(g_last, h, l, is_pre_delay)
                break
            width = layer.weight.size(1)
            single_rank = getattr(graph, "exchange", None) is None
            # a next layer that multiplies first reads its input densely: nothing to gain from packing
            pack = (self.packed_activations and (is_pre_delay or single_rank)
                    and packed.header_words(width) > 0 and not self.layers[l + 1].linear_first)
            dropping = self.training and self.dropout > 0.0
            if dropping and masks is None:
                raise ValueError("training needs the seeded dropout masks")
            mask = masks[l] if dropping else None
            scale = 1.0 / (1.0 - self.dropout) if dropping else 1.0
            bits = mask
            if mask is not None and mask.dtype != torch.int32 and layer.fuse and not layer.linear_first:
                bits = self._packed_mask(mask)
            fused = layer.fused(graph, h, l, is_pre_delay, bits, scale, True, pack_out=pack)
            if fused is not None:
                h = fused
                continue
            if mask is not None and mask.dtype == torch.int32:
                raise RuntimeError("a bit-packed dropout mask only serves the fused layer kernels; this layer needs "
                                   "the bool mask")
            z = layer.transform(graph, h, l, is_pre_delay)
            epilogue = _BiasReluDropoutPacked if pack else _BiasReluDropout
            h = epilogue.apply(z, layer.bias, mask, scale, _row_divisors(graph))
        return F.log_softmax(h, dim=1) if log_probs else h


def make_dropout_masks(num_nodes: int, dims: Sequence[int], p: float, seed: int, device) -> List[torch.Tensor]:
    gen = torch.Generator(device=device).manual_seed(seed)
    return [torch.rand(num_nodes, dims[l + 1], device=device, generator=gen) >= p for l in range(len(dims) - 2)]


@contextlib.contextmanager
def scored_rows(graph, last_layer: int, rows: torch.Tensor, is_pre_delay: bool):
    """While a loss that scores only ``rows`` is back-propagated: the gradient that reaches the last layer's
    aggregation is zero in every other row, so its transposed products skip those rows (same result, a tenth of
    the gathers when a tenth of the nodes is labelled).  Declared for the duration of the backward pass only."""
    if not rows.is_cuda:
        yield
        return
    previous = getattr(graph, "backward_row_support", None)
    graph.backward_row_support = {last_layer: aggregator_module.backward_support(graph, rows, is_pre_delay)}
    try:
        yield
    finally:
        graph.backward_row_support = previous


def _mean_nll(log_probs: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    """F.nll_loss(log_probs, target) (mean over the rows, every target a class index) as a gather and a mean: the
    library's reduction kernel for it runs in a single block and takes 1.6 ms on 700 000 rows."""
    return -log_probs.gather(1, target.unsqueeze(1)).mean()


def train_step(model: GCN, optimizer, graph, x, labels, train_idx, is_pre_delay: bool, masks,
               restrict_last_layer: bool = True) -> torch.Tensor:
    """forward, NLL loss on the labelled nodes, backward, optimizer update.  Only the labelled rows of the last layer
    are evaluated (the loss reads no others): the same loss, gradients and update as evaluating every node, which
    ``restrict_last_layer=False`` does."""
    model.train()
    optimizer.zero_grad(set_to_none=True)
    if restrict_last_layer:
        out = model(graph, x, is_pre_delay, masks, log_probs=False, last_rows=train_idx)
    else:  # every node through the last layer, as the reference's epoch does; the loss reads the labelled rows
        out = model(graph, x, is_pre_delay, masks, log_probs=False)[train_idx]
    loss = _mean_nll(F.log_softmax(out, dim=1), labels[train_idx])
    loss.backward()
    optimizer.step()
    return loss.detach()
