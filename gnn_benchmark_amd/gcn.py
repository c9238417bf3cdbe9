"""A GCN layer stack around the aggregation path, used for the full train-step workload.

The aggregation is the reference's ``Aggregator`` contract (aggregate-then-transform, the
order of self_benchmark/a64fx/model/layers/sageconv.py:65-93: ``out = Aggregator(...)``,
``out /= graph.in_degrees``, then the dense transform).  Everything after the
aggregation is this build's own definition of the workload: one weight matrix per layer
(``Z = ((A X) W) / deg + b`` -- the degree normalisation is applied behind the dense
product, where it fuses into the epilogue: D^-1 (A X) W == D^-1 ((A X) W)), ReLU, dropout
with a precomputed seeded mask, log-softmax + NLL on the labelled nodes, Adam.  The
forward and input-gradient products run on the matrix cores through the BLAS library
behind ``torch.mm`` (fp32, or bf16 inputs with fp32 accumulation and fp32 output); the
weight gradient -- a reduction over millions of rows into at most 256 x 256 outputs, the
library's weakest shape -- runs in libgnnagg's own fp32 MFMA kernel.
"""
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F

from . import _lib, packed
from .aggregator import Aggregator, AggregatorPacked
from .sparse_tensor import _row_stride, _rows_are_dense


class _Bf16InputLinear(torch.autograd.Function):
    """y = x @ w with x, w rounded to bf16, products accumulated in fp32, fp32 result; the
    input gradient is computed the same way.  The weight gradient stays in fp32: the
    hand-written kernel reads the fp32 operands as they are, which is faster than rounding
    7 M-row operands to bf16 for the library's product, and more exact."""

    @staticmethod
    def _mm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        return torch.mm(a.to(torch.bfloat16), b.to(torch.bfloat16), out_dtype=torch.float32)

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return _Bf16InputLinear._mm(x, w)

    @staticmethod
    def backward(ctx, g):
        x, w = ctx.saved_tensors
        gx = _Bf16InputLinear._mm(g, w.t()) if ctx.needs_input_grad[0] else None
        gw = weight_gradient(x, g) if ctx.needs_input_grad[1] else None
        return gx, gw


def weight_gradient(x: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """x^T @ g for tall-skinny fp32 operands through the library's MFMA kernel; falls back to
    the BLAS library for shapes that kernel does not take (more than 256 columns).  Column
    blocks of wider row-major tensors are read where they lie."""
    if not _rows_are_dense(x):
        x = x.contiguous()
    if not _rows_are_dense(g):
        g = g.contiguous()
    rows, fi, fo = x.size(0), x.size(1), g.size(1)
    L = _lib.lib()
    nbytes = int(L.gnnagg_wgrad_workspace_bytes(rows, fi, fo)) if x.is_cuda and x.dtype == torch.float32 else 0
    if nbytes == 0:
        return torch.mm(x.t(), g)
    out = torch.empty(fi, fo, dtype=torch.float32, device=x.device)
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(L.gnnagg_wgrad_strided_f32(_lib.ptr(x), _row_stride(x), _lib.ptr(g), _row_stride(g), _lib.ptr(out),
                                              _lib.ptr(workspace), rows, fi, fo, _lib.current_stream(x.device)))
    return out


class _Fp32Linear(torch.autograd.Function):
    """y = x @ w in fp32; the weight gradient (a reduction over millions of rows) runs in
    the hand-written MFMA kernel, the two other products in the BLAS library."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return torch.mm(x, w)

    @staticmethod
    def backward(ctx, g):
        x, w = ctx.saved_tensors
        gx = torch.mm(g, w.t()) if ctx.needs_input_grad[0] else None
        gw = weight_gradient(x, g) if ctx.needs_input_grad[1] else None
        return gx, gw


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
    def __init__(self, in_channels: int, out_channels: int, gemm: str = "fp32"):
        super().__init__()
        if gemm not in ("fp32", "bf16"):
            raise ValueError("gemm must be 'fp32' or 'bf16'")
        self.gemm = gemm
        self.linear_first = False
        self.weight = torch.nn.Parameter(torch.empty(in_channels, out_channels))
        self.bias = torch.nn.Parameter(torch.zeros(out_channels))
        torch.nn.init.xavier_uniform_(self.weight, gain=torch.nn.init.calculate_gain("relu"))

    def _product(self, t: torch.Tensor) -> torch.Tensor:
        if self.gemm == "bf16":
            return _Bf16InputLinear.apply(t, self.weight)
        return _Fp32Linear.apply(t, self.weight)

    def transform(self, graph, x, layer: int, is_pre_delay: bool) -> torch.Tensor:
        """(A x) W: neither the degree normalisation nor the bias yet.  ``x`` is a dense tensor
        or a packed ``(values, header)`` pair.  With ``linear_first`` (and dense ``x``) the
        product comes first, A (x W): the same up to rounding, and the aggregation, its backward
        and the boundary rows then have the output width."""
        if isinstance(x, tuple):
            agg = AggregatorPacked.apply(graph, x[0], x[1], layer, 32, is_pre_delay, self.training)
            return self._product(agg)
        if self.linear_first:
            return Aggregator.apply(graph, self._product(x), layer, 32, is_pre_delay, self.training)
        return self._product(Aggregator.apply(graph, x, layer, 32, is_pre_delay, self.training))

    def forward(self, graph, x: torch.Tensor, layer: int, is_pre_delay: bool) -> torch.Tensor:
        """((A x) W) / deg + bias."""
        return torch.addcdiv(self.bias, self.transform(graph, x, layer, is_pre_delay), graph.in_degrees)


class GCN(torch.nn.Module):
    def __init__(self, dims: Sequence[int], gemm: str = "fp32", dropout: float = 0.5, packed_activations: bool = False,
                 linear_first_when_narrowing: bool = False):
        super().__init__()
        self.layers = torch.nn.ModuleList([GCNLayer(dims[i], dims[i + 1], gemm) for i in range(len(dims) - 1)])
        if linear_first_when_narrowing:  # a layer with fewer outputs than inputs aggregates its outputs
            for i, layer in enumerate(self.layers):
                layer.linear_first = dims[i + 1] < dims[i]
        self.dropout = dropout
        # keep hidden activations packed (non-zero values + bitmap) where their width allows and
        # pre-aggregation is used: the next layer's aggregation then skips the zeros
        self.packed_activations = packed_activations

    def forward(self, graph, x: torch.Tensor, is_pre_delay: bool,
                masks: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
        """``masks[l]``: bool keep-mask [N, dims[l+1]] of the dropout after layer l (training only)."""
        h = x
        last = len(self.layers) - 1
        for l, layer in enumerate(self.layers):
            if l == last:
                h = layer(graph, h, l, is_pre_delay)
                break
            z = layer.transform(graph, h, l, is_pre_delay)
            single_rank = getattr(graph, "exchange", None) is None
            # a next layer that multiplies first reads its input densely: nothing to gain from packing
            pack = (self.packed_activations and (is_pre_delay or single_rank)
                    and packed.header_words(z.size(1)) > 0 and not self.layers[l + 1].linear_first)
            epilogue = _BiasReluDropoutPacked if pack else _BiasReluDropout
            if self.training and self.dropout > 0.0:
                if masks is None:
                    raise ValueError("training needs the seeded dropout masks")
                h = epilogue.apply(z, layer.bias, masks[l], 1.0 / (1.0 - self.dropout), graph.in_degrees)
            else:
                h = epilogue.apply(z, layer.bias, None, 1.0, graph.in_degrees)
        return F.log_softmax(h, dim=1)


def make_dropout_masks(num_nodes: int, dims: Sequence[int], p: float, seed: int, device) -> List[torch.Tensor]:
    gen = torch.Generator(device=device).manual_seed(seed)
    return [torch.rand(num_nodes, dims[l + 1], device=device, generator=gen) >= p for l in range(len(dims) - 2)]


def train_step(model: GCN, optimizer, graph, x, labels, train_idx, is_pre_delay: bool, masks) -> torch.Tensor:
    """forward, NLL loss on the labelled nodes, backward, optimizer update."""
    model.train()
    optimizer.zero_grad(set_to_none=True)
    out = model(graph, x, is_pre_delay, masks)
    loss = F.nll_loss(out[train_idx], labels[train_idx])
    loss.backward()
    optimizer.step()
    return loss.detach()
