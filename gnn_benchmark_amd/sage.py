"""The reference's layer and model around the aggregation path: ``DistSAGEConvGrad``
(self_benchmark/a64fx/model/layers/sageconv.py:18-93) and ``DistSAGE``
(self_benchmark/a64fx/model/DistSAGE.py:13-69), same constructor arguments, same forward
call shapes, same mathematics:

    out = lin_neigh(Aggregator(graph, x) / in_degrees) + lin_self(x) + bias        (layer)
    x   = relu(LayerNorm(dropout(out)))  between layers, log_softmax at the end     (model)

How it runs here differs.  A layer keeps ``[aggregated | x]`` side by side in one
``[N, 2 * in_channels]`` array: the previous layer's fused dropout + LayerNorm + ReLU pass
writes ``x`` into the right half, the aggregation reads it there and writes the left half
(strided SpMM operands), and ``lin_neigh`` + ``lin_self`` are ONE dense product with the
stacked weight ``[2 * in_channels, out_channels]`` -- no concatenation copy, one pass over the
output instead of a product plus an accumulating product.  The backward mirrors it: one
product gives the gradient of both halves, the transposed aggregation of the left half is
accumulated straight onto the right half, and the weight gradient of each half runs in the
library's own fp32 MFMA kernel.  The degree normalisation is either an in-place division of
the left half (the reference's ``out /= graph.in_degrees``) or, for a graph prepared with
``fold_in_degrees``, already part of the matrix values and free.

Dropout takes explicit keep masks (seeded, reproducible); without them a mask is drawn with
``torch.rand`` per call, which is what ``F.dropout`` amounts to.
"""
import copy
from typing import List, Optional

import torch
import torch.nn.functional as F

from . import _lib, aggregator
from .gcn import (_FORMS, _mean_nll, input_gradient, plain_product, scored_rows, stacked_product,
                  weight_and_bias_gradient, weight_gradient)
from .sparse_tensor import SparseTensor, _row_stride


# --------------------------------------------------------------------- staged layer input
def stage_input(x: torch.Tensor) -> torch.Tensor:
    """``[N, 2F]`` array whose right half holds ``x`` (the left half is the layer's scratch for
    the aggregated rows).  For features that stay the same over the epochs do this once and hand
    the result to ``DistSAGE.forward`` / ``DistSAGEConvGrad.forward`` instead of ``x``."""
    if x.dim() != 2 or x.dtype != torch.float32:
        raise RuntimeError("Input mismatch: node features must be float32 [N, F]")
    cat = torch.empty(x.size(0), 2 * x.size(1), dtype=torch.float32, device=x.device)
    cat[:, x.size(1):] = x
    return cat


def fold_in_degrees(graph):
    """A copy of ``graph`` whose aggregation already divides by the in-degree: the rows of the
    matrices that produce local output rows (``local_adj_t`` and the post-aggregation / halo
    matrix) are scaled by ``1 / in_degrees``, so ``out /= graph.in_degrees`` (sageconv.py:80-82)
    costs nothing.  The result differs from divide-afterwards by rounding only
    (sum(a/d * x) against sum(a * x) / d)."""
    deg = graph.in_degrees.reshape(-1)

    def scaled(m: SparseTensor) -> SparseTensor:
        rowptr, col, value = m.csr()
        counts = rowptr[1:] - rowptr[:-1]
        per_element = torch.repeat_interleave(deg, counts)
        value = torch.ones_like(per_element) if value is None else value
        return SparseTensor(rowptr=rowptr, col=col, value=value / per_element, sparse_sizes=m.sparse_sizes())

    g = copy.copy(graph)
    g.local_adj_t = scaled(graph.local_adj_t)
    if hasattr(graph, "adj_t_pre_post_aggr_from"):
        g.adj_t_pre_post_aggr_from = scaled(graph.adj_t_pre_post_aggr_from)
    else:
        g.remote_adj_t = scaled(graph.remote_adj_t)
    g.in_degrees_folded = True
    return g


# ------------------------------------------------------------ dropout -> LayerNorm -> ReLU
class _DropoutLayerNormRelu(torch.autograd.Function):
    """``relu(layer_norm(z * keep * scale))`` in one pass, written into the right half of a fresh
    ``[N, 2F]`` array (returned whole: the next layer's staged input).  Keeps ``z`` and the mask
    for the backward, which takes the row moments again instead of storing them."""

    @staticmethod
    def forward(ctx, z, keep, scale, gamma, beta, eps):
        if not z.is_cuda or z.dtype != torch.float32 or z.dim() != 2 or not z.is_contiguous():
            raise RuntimeError("Input mismatch: z must be a contiguous float32 [rows, feat] GPU (HIP) tensor")
        rows, feat = z.shape
        if keep is not None and (keep.dtype not in (torch.bool, torch.uint8) or keep.shape != z.shape
                                 or not keep.is_contiguous()):
            raise RuntimeError("Input mismatch: keep must be a contiguous bool/uint8 mask shaped like z")
        if gamma.numel() != feat or beta.numel() != feat:
            raise RuntimeError("Input mismatch: LayerNorm weight / bias must hold one value per feature")
        gamma, beta = gamma.detach().contiguous(), beta.detach().contiguous()
        cat = torch.empty(rows, 2 * feat, dtype=torch.float32, device=z.device)
        with torch.cuda.device(z.device):
            _lib.check(_lib.lib().gnnagg_dropout_layernorm_relu_f32(
                _lib.ptr(z), _lib.ptr(keep), float(scale), _lib.ptr(gamma), _lib.ptr(beta), float(eps),
                _lib.ptr(cat[:, feat:]), 2 * feat, rows, feat, _lib.current_stream(z.device)))
        ctx.save_for_backward(z, keep, gamma, beta)
        ctx.scale, ctx.eps = float(scale), float(eps)
        return cat

    @staticmethod
    def backward(ctx, grad_cat):
        z, keep, gamma, beta = ctx.saved_tensors
        rows, feat = z.shape
        grad_y = grad_cat[:, feat:]  # the left half belongs to nobody
        if grad_y.stride(1) != 1 or grad_y.stride(0) % 4 != 0 or grad_y.data_ptr() % 16 != 0:
            grad_y = grad_y.contiguous()
        grad_z = torch.empty_like(z)
        L = _lib.lib()
        blocks = int(L.gnnagg_dropout_layernorm_relu_blocks(rows, feat))
        partial = torch.empty(blocks, 2, feat, dtype=torch.float32, device=z.device)
        with torch.cuda.device(z.device):
            _lib.check(L.gnnagg_dropout_layernorm_relu_backward_f32(
                _lib.ptr(grad_y), _row_stride(grad_y), _lib.ptr(z), _lib.ptr(keep), ctx.scale, _lib.ptr(gamma),
                _lib.ptr(beta), ctx.eps, _lib.ptr(grad_z), _lib.ptr(partial), rows, feat,
                _lib.current_stream(z.device)))
        sums = partial.sum(dim=0)
        return grad_z, None, None, sums[0], sums[1], None


def dropout_layernorm_relu(z, keep, scale, gamma, beta, eps) -> torch.Tensor:
    """Staged input ``[N, 2F]`` of the next layer (right half = the activations).  Widths the fused
    pass does not take (not a multiple of 4, or above 1024) go through the same torch ops on the GPU."""
    rows, feat = z.shape
    if z.is_cuda and rows > 0 and int(_lib.lib().gnnagg_dropout_layernorm_relu_blocks(rows, feat)) == 0:
        d = z if keep is None else z * keep * scale
        y = torch.relu(F.layer_norm(d, (feat,), gamma, beta, eps))
        return torch.cat([torch.zeros_like(y), y], dim=1)
    return _DropoutLayerNormRelu.apply(z, keep, scale, gamma, beta, eps)


# ---------------------------------------------------------------------------- the layer
class _SageConv(torch.autograd.Function):
    """``[A x / deg | x] @ W + bias`` on a staged input ``cat`` (right half = x; the left half is
    overwritten with the aggregated rows and kept for the weight gradient)."""

    @staticmethod
    def forward(ctx, graph, cat, weight, bias, layer, num_bits, is_pre_delay, is_training, normalize, form=0):
        fi = cat.size(1) // 2
        x, agg = cat[:, fi:], cat[:, :fi]
        aggregator._forward(ctx, graph, aggregator._DenseFeatures(x), layer, num_bits, is_pre_delay, is_training,
                            out=agg)
        ctx.divide = bool(normalize) and not getattr(graph, "in_degrees_folded", False)
        if ctx.divide:
            agg.div_(graph.in_degrees)  # sageconv.py:80-82
        else:
            # the library wrote the left half behind autograd's back: an (empty) in-place op bumps the
            # array's version, so that an earlier call that kept this same array for its backward
            # fails loudly there instead of reading rows that are no longer its own
            cat[:0].zero_()
        out = stacked_product(cat, weight, bias, form)
        ctx.save_for_backward(cat, weight)
        ctx.has_bias = bias is not None
        ctx.form = form
        return out

    @staticmethod
    def backward(ctx, g):
        cat, weight = ctx.saved_tensors
        fi = cat.size(1) // 2
        g = g.contiguous()
        grad_cat = grad_w = grad_b = None
        want_b = ctx.has_bias and ctx.needs_input_grad[3]
        if ctx.needs_input_grad[2]:
            # each half's rows of the stacked weight: x_half^T @ g, reading the half where it lies; the
            # bias gradient (column sums of g) comes out of the first of the two passes over g
            if want_b or ctx.form:
                top, grad_b = weight_and_bias_gradient(cat[:, :fi], g, ctx.form)
            else:
                top = weight_gradient(cat[:, :fi], g)
            bottom = weight_and_bias_gradient(cat[:, fi:], g, ctx.form)[0] if ctx.form else weight_gradient(cat[:, fi:], g)
            grad_w = torch.cat([top, bottom], dim=0)
            grad_b = grad_b if want_b else None
        elif want_b:
            grad_b = g.sum(dim=0)
        if ctx.needs_input_grad[1]:
            grad_cat = input_gradient(g, weight, ctx.form)  # [N, 2 fi]: d/d aggregated | d/d x (direct part)
            grad_agg = grad_cat[:, :fi]
            if ctx.divide:
                grad_agg.div_(ctx.graph.in_degrees)
            # d/d x += A^T (d/d aggregated), accumulated where the direct part already lies
            aggregator._backward(ctx, grad_agg, out=grad_cat[:, fi:], accumulate=True)
        return None, grad_cat, grad_w, grad_b, None, None, None, None, None, None


class _SageConvRows(torch.autograd.Function):
    """The same layer for the local nodes ``rows`` only: ``[A[rows] x / deg[rows] | x[rows]] @ W + bias`` through a
    row-restricted view of the graph (``aggregator.restrict_output_rows``).  What a loss over those nodes needs of the
    last layer, at a fraction of its aggregation and products, forward and backward; each row is the same FMA chain."""

    @staticmethod
    def forward(ctx, graph_rows, cat, weight, bias, layer, num_bits, is_pre_delay, is_training, normalize, rows, form=0):
        fi = cat.size(1) // 2
        x = cat[:, fi:]
        agg = aggregator._forward(ctx, graph_rows, aggregator._DenseFeatures(x), layer, num_bits, is_pre_delay,
                                  is_training)
        ctx.divide = bool(normalize) and not getattr(graph_rows, "in_degrees_folded", False)
        if ctx.divide:
            agg.div_(graph_rows.in_degrees)
        small = torch.cat([agg, x.index_select(0, rows)], dim=1)  # [len(rows), 2 fi]
        out = stacked_product(small, weight, bias, form)
        ctx.save_for_backward(small, weight, rows)
        ctx.has_bias = bias is not None
        ctx.form = form
        ctx.nodes = cat.size(0)
        return out

    @staticmethod
    def backward(ctx, g):
        small, weight, rows = ctx.saved_tensors
        fi = small.size(1) // 2
        g = g.contiguous()
        grad_cat = grad_w = grad_b = None
        want_b = ctx.has_bias and ctx.needs_input_grad[3]
        if ctx.needs_input_grad[2]:
            if want_b or ctx.form:
                top, grad_b = weight_and_bias_gradient(small[:, :fi], g, ctx.form)
            else:
                top = weight_gradient(small[:, :fi], g)
            bottom = weight_and_bias_gradient(small[:, fi:], g, ctx.form)[0] if ctx.form else weight_gradient(small[:, fi:], g)
            grad_w = torch.cat([top, bottom], dim=0)
            grad_b = grad_b if want_b else None
        elif want_b:
            grad_b = g.sum(dim=0)
        if ctx.needs_input_grad[1]:
            grad_small = input_gradient(g, weight, ctx.form)  # [len(rows), 2 fi]: d/d aggregated | d/d x[rows] (direct part)
            grad_agg = grad_small[:, :fi]
            if ctx.divide:
                grad_agg.div_(ctx.graph.in_degrees)
            # the gradient goes where the features were: the right half of an [N, 2 fi] array: A[rows]^T (d/d
            # aggregated), then the direct part added onto the rows it belongs to (every row once: deterministic).
            # The left half was scratch on the way forward: nothing depends on it, so its gradient is zero -- written
            # as such, because autograd hands this array on (to a leaf that requires grad, or into a sum with another
            # consumer's gradient) and uninitialised memory there could be anything, NaN included.
            grad_cat = torch.empty(ctx.nodes, 2 * fi, dtype=torch.float32, device=g.device)
            grad_cat[:, :fi].zero_()
            target = grad_cat[:, fi:]
            aggregator._backward(ctx, grad_agg, out=target, accumulate=False)
            target.index_add_(0, rows, grad_small[:, fi:])
        return None, grad_cat, grad_w, grad_b, None, None, None, None, None, None, None


class _SageConvLinearFirst(torch.autograd.Function):
    """The same layer with the products taken first: ``A (x W_n) / deg + x W_s + bias``.  Equal to
    aggregate-first up to rounding ((A x) W = A (x W)); the aggregation, its backward and the
    boundary exchange then run at the OUTPUT width, which pays when the layer narrows (the switch
    the reference sketches and leaves commented out, sageconv.py:67-71, :84)."""

    @staticmethod
    def forward(ctx, graph, feats_in, weight, bias, layer, num_bits, is_pre_delay, is_training, normalize, form=0):
        fi = weight.size(0) // 2
        ctx.staged = feats_in.size(1) == 2 * fi      # [N, 2 fi] with the features in the right half
        x = feats_in[:, fi:] if ctx.staged else feats_in
        folded = getattr(graph, "in_degrees_folded", False)
        ctx.divide = bool(normalize) and not folded
        ctx.form = form
        left = plain_product(x, weight[:fi], None, form)                  # x W_n
        out = plain_product(x, weight[fi:], bias, form)                   # x W_s + b
        feats = aggregator._DenseFeatures(left)
        if ctx.divide:
            agg = aggregator._forward(ctx, graph, feats, layer, num_bits, is_pre_delay, is_training)
            out.addcdiv_(agg, graph.in_degrees)
        else:  # degrees folded into the matrices (or no normalisation): add straight onto x W_s + b
            aggregator._forward(ctx, graph, feats, layer, num_bits, is_pre_delay, is_training, out=out,
                                accumulate=True)
        ctx.save_for_backward(feats_in, weight)
        ctx.has_bias = bias is not None
        return out

    @staticmethod
    def backward(ctx, g):
        feats_in, weight = ctx.saved_tensors
        fi = weight.size(0) // 2
        x = feats_in[:, fi:] if ctx.staged else feats_in
        g = g.contiguous()
        grad_left = aggregator._backward(ctx, g / ctx.graph.in_degrees if ctx.divide else g)   # d/d (x W_n)
        grad_x = grad_w = grad_b = None
        want_b = ctx.has_bias and ctx.needs_input_grad[3]
        if ctx.needs_input_grad[2]:
            if want_b:
                bottom, grad_b = weight_and_bias_gradient(x, g)
            else:
                bottom = weight_gradient(x, g)
            grad_w = torch.cat([weight_gradient(x, grad_left), bottom], dim=0)
        elif want_b:
            grad_b = g.sum(dim=0)
        if ctx.needs_input_grad[1]:
            # d/d x = (d/d (x W_n)) W_n^T + g W_s^T = [d/d (x W_n) | g] @ [W_n | W_s]^T: one product
            both = torch.cat([grad_left, g], dim=1)
            stacked = torch.cat([weight[:fi], weight[fi:]], dim=1)          # [fi, 2 fo]
            if ctx.staged:
                # the gradient goes where the features were: the right half of an [N, 2 fi] array
                # (its left half was scratch on the way forward: zero gradient, written as such)
                grad_x = torch.empty(x.size(0), 2 * fi, dtype=torch.float32, device=x.device)
                grad_x[:, :fi].zero_()
                input_gradient(both, stacked, ctx.form, out=grad_x[:, fi:])
            else:
                grad_x = input_gradient(both, stacked, ctx.form)
        return None, grad_x, grad_w, grad_b, None, None, None, None, None, None


class _LinearView:
    """What the reference's ``lin_neigh`` / ``lin_self`` expose: ``weight`` as ``[out, in]`` -- here
    a view of the layer's stacked weight."""

    def __init__(self, owner, first_row: int, rows: int):
        self._owner, self._first, self._rows = owner, first_row, rows

    @property
    def weight(self) -> torch.Tensor:
        return self._owner.weight[self._first:self._first + self._rows].t()


class DistSAGEConvGrad(torch.nn.Module):
    """sageconv.py:18-93.  Parameters: ``weight`` ``[2 * in_channels, out_channels]`` (rows
    ``[:in]`` are ``lin_neigh.weight.T``, rows ``[in:]`` are ``lin_self.weight.T``) and ``bias``."""

    def __init__(self, in_channels: int, out_channels: int, num_bits: int, is_pre_delay: bool,
                 add_self_loops: bool = False, normalize: bool = True, bias: bool = True, linear_first: bool = False,
                 gemm: str = "fp32"):
        super().__init__()
        # linear_first: apply lin_neigh before aggregating (same result up to rounding; the
        # aggregation and the exchange then run at out_channels)
        self.linear_first = linear_first
        # gemm "bf16x3": all of the layer's dense products in libgnnagg's kernels with every fp32 operand as three bf16
        # pieces (fp32 accuracy on the bf16 matrix units); "fp32": the stacked product and the input-gradient product
        # likewise (plain products, for which that form is the fastest fp32-accurate one), the weight gradients with the
        # fp32 matrix instruction
        if gemm not in ("fp32", "bf16x3"):
            raise ValueError("gemm must be 'fp32' or 'bf16x3'")
        self.gemm = gemm
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.add_self_loops = add_self_loops
        self.normalize = normalize
        self.num_bits = num_bits
        self.is_pre_delay = is_pre_delay
        self.weight = torch.nn.Parameter(torch.empty(2 * in_channels, out_channels))
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(out_channels))
        else:
            self.register_parameter("bias", None)
        # the reference leaves torch's default Linear initialisation in place (its
        # reset_parameters call is commented out, sageconv.py:48); per half, as two Linears would
        bound = 1.0 / in_channels ** 0.5
        with torch.no_grad():
            self.weight.uniform_(-bound, bound)

    @property
    def lin_neigh(self) -> _LinearView:
        return _LinearView(self, 0, self.in_channels)

    @property
    def lin_self(self) -> _LinearView:
        return _LinearView(self, self.in_channels, self.in_channels)

    def reset_parameters(self):
        gain = torch.nn.init.calculate_gain("relu")  # sageconv.py:50-53, per Linear
        with torch.no_grad():
            for half in (self.weight[:self.in_channels], self.weight[self.in_channels:]):
                torch.nn.init.xavier_uniform_(half.t(), gain=gain)

    def load_linear_weights(self, lin_neigh_weight: torch.Tensor, lin_self_weight: torch.Tensor) -> None:
        """Take over the reference's two ``[out, in]`` matrices."""
        with torch.no_grad():
            self.weight[:self.in_channels] = lin_neigh_weight.t()
            self.weight[self.in_channels:] = lin_self_weight.t()

    def forward(self, graph, local_nodes_feat: torch.Tensor, layer: int,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``local_nodes_feat``: ``[N, in_channels]`` features (staged here, one copy) or an
        already staged ``[N, 2 * in_channels]`` array (``stage_input`` / the fused LayerNorm
        pass) whose left half this call overwrites.  ``rows`` (local node ids): the output for
        those nodes only, ``[len(rows), out_channels]`` (aggregate-first order only)."""
        width = local_nodes_feat.size(-1)
        if self.linear_first and rows is not None:
            raise RuntimeError("a layer that multiplies first has no row-restricted form")
        if self.linear_first:
            if width not in (self.in_channels, 2 * self.in_channels):
                raise RuntimeError("Input mismatch: expected %d features (or %d staged), got %d"
                                   % (self.in_channels, 2 * self.in_channels, width))
            if not local_nodes_feat.is_cuda or local_nodes_feat.dtype != torch.float32:
                raise RuntimeError("Input mismatch: the features must be a float32 GPU (HIP) tensor")
            return _SageConvLinearFirst.apply(graph, local_nodes_feat, self.weight, self.bias, layer, self.num_bits,
                                              self.is_pre_delay, self.training, self.normalize, _FORMS[self.gemm])
        if width == self.in_channels:
            if local_nodes_feat.requires_grad:
                raise RuntimeError("features that need a gradient must be handed over staged (stage_input)")
            cat = stage_input(local_nodes_feat)
        elif width == 2 * self.in_channels:
            cat = local_nodes_feat
        else:
            raise RuntimeError("Input mismatch: expected %d features (or %d staged), got %d"
                               % (self.in_channels, 2 * self.in_channels, width))
        if not cat.is_cuda or cat.dtype != torch.float32 or not cat.is_contiguous():
            raise RuntimeError("Input mismatch: the staged input must be a contiguous float32 GPU (HIP) tensor")
        if rows is not None:
            graph_rows = aggregator.restrict_output_rows(graph, rows, self.is_pre_delay)
            return _SageConvRows.apply(graph_rows, cat, self.weight, self.bias, layer, self.num_bits, self.is_pre_delay,
                                       self.training, self.normalize, rows, _FORMS[self.gemm])
        return _SageConv.apply(graph, cat, self.weight, self.bias, layer, self.num_bits, self.is_pre_delay,
                               self.training, self.normalize, _FORMS[self.gemm])


# ---------------------------------------------------------------------------- the model
class DistSAGE(torch.nn.Module):
    """DistSAGE.py:13-69: ``num_layers`` SAGE layers, LayerNorm after all but the last."""

    def __init__(self, in_channels, hidden_channels, out_channels, num_layers=3, dropout=0.5, num_bits=32,
                 is_pre_delay=False, linear_first_when_narrowing=False, gemm="fp32"):
        super().__init__()
        self.convs = torch.nn.ModuleList()
        self.norms = torch.nn.ModuleList()
        self.convs.append(DistSAGEConvGrad(in_channels, hidden_channels, num_bits, is_pre_delay, gemm=gemm))
        self.norms.append(torch.nn.LayerNorm(hidden_channels))
        for _ in range(num_layers - 2):
            self.convs.append(DistSAGEConvGrad(hidden_channels, hidden_channels, num_bits, is_pre_delay, gemm=gemm))
            self.norms.append(torch.nn.LayerNorm(hidden_channels))
        self.convs.append(DistSAGEConvGrad(hidden_channels, out_channels, num_bits, is_pre_delay, gemm=gemm))
        if linear_first_when_narrowing:  # a layer with fewer outputs than inputs aggregates its outputs
            for conv in self.convs:
                conv.linear_first = conv.out_channels < conv.in_channels
        self.dropout = dropout

    def reset_parameters(self):
        for conv in self.convs:
            conv.reset_parameters()
        for norm in self.norms:
            norm.reset_parameters()

    def forward(self, graph, nodes_feats: torch.Tensor, masks: Optional[List[torch.Tensor]] = None,
                log_probs: bool = True, last_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``nodes_feats``: ``[N, in_channels]`` or staged (``stage_input``).  ``masks[i]``: keep
        mask ``[N, hidden]`` of the dropout after layer i (training; drawn here when None).
        ``log_probs=False`` returns the last layer's output before the log-softmax of
        model/DistSAGE.py:69 (a caller that scores a subset of the nodes applies it to those rows).
        ``last_rows`` (local node ids): evaluate the last layer for those nodes only and return
        ``[len(last_rows), out_channels]``."""
        for i, conv in enumerate(self.convs[:-1]):
            z = conv(graph, nodes_feats, i)
            keep, scale = None, 1.0
            if self.training and self.dropout > 0.0:
                keep = masks[i] if masks is not None else torch.rand_like(z) >= self.dropout
                scale = 1.0 / (1.0 - self.dropout)
            norm = self.norms[i]
            nodes_feats = dropout_layernorm_relu(z, keep, scale, norm.weight, norm.bias, norm.eps)
        out = self.convs[-1](graph, nodes_feats, len(self.convs) - 1, last_rows)
        return F.log_softmax(out, dim=1) if log_probs else out


def make_dropout_masks(num_nodes: int, hidden_channels: int, num_layers: int, p: float, seed: int,
                       device) -> List[torch.Tensor]:
    gen = torch.Generator(device=device).manual_seed(seed)
    return [torch.rand(num_nodes, hidden_channels, device=device, generator=gen) >= p for _ in range(num_layers - 1)]


def train_step(model: DistSAGE, optimizer, graph, nodes_feats, labels, train_idx, masks=None,
               restrict_last_layer: bool = True) -> torch.Tensor:
    """One epoch of train.py:82-98: forward, NLL loss on the training nodes, backward, update.
    The loss reads only the training rows of the last layer, so only those are evaluated (or, for a
    last layer that multiplies first, the zero rows of its gradient are skipped): the same loss and
    gradients as train.py:87-89, to the rounding of the last layer's dense products."""
    model.train()
    optimizer.zero_grad(set_to_none=True)
    last = model.convs[-1]
    if not restrict_last_layer:  # every node through the last layer, exactly as train.py:87-90
        out = model(graph, nodes_feats, masks, log_probs=False)
        loss = _mean_nll(F.log_softmax(out[train_idx], dim=1), labels[train_idx])
        loss.backward()
    elif last.linear_first:  # no row-restricted form: every node through the last layer, zero gradient rows skipped
        out = model(graph, nodes_feats, masks, log_probs=False)
        loss = _mean_nll(F.log_softmax(out[train_idx], dim=1), labels[train_idx])
        with scored_rows(graph, len(model.convs) - 1, train_idx, last.is_pre_delay):
            loss.backward()
    else:
        out = model(graph, nodes_feats, masks, log_probs=False, last_rows=train_idx)
        loss = _mean_nll(F.log_softmax(out, dim=1), labels[train_idx])
        loss.backward()
    optimizer.step()
    return loss.detach()
