"""The aggregation autograd.Function of one graph partition.

Reference: self_benchmark/a64fx/model/layers/aggregator.py:15-119 (forward), :121-208
(backward).  Same ``apply`` signature ``(graph, local_nodes_feat, layer, num_bits,
is_pre_delay, is_training)`` and the same backward arity ``(None, grad, None, None,
None, None)``.

Per direction: (1) fill the outgoing boundary buffer -- pre-aggregation SpMM or row
gather; (2) hand the buffers to the exchange; (3) local SpMM; (4) wait for the
exchange; (5) accumulate the received halo rows into the same output
(post-aggregation).  Backward runs the same pipeline on the transposed matrices with
the two buffers swapping roles (aggregator.py:141, :186).

What differs from the reference, on purpose:
* The boundary all-to-all (communicator.py:55-109) is ``graph.exchange``, a callable
  ``exchange(comm_splits, comm_buf, tag, direction) -> handle | None``: on "forward" it
  must leave the received halo rows in ``comm_buf.recv_buf``, on "backward" the received
  gradient rows in ``comm_buf.send_buf``.  A returned handle's ``wait()`` is called after
  the local SpMM, where the reference waits (aggregator.py:78, :175).  ``exchange is
  None`` is the single-rank world: pre/post steps are skipped (aggregator.py:47, :100).
* With ``num_bits`` 2 (the reference's int2 exchange, communicator.py:231-325; 4 and 8 are
  accepted with the same layout) the outgoing buffer is quantised here, per peer rank,
  into ``graph.comm_buf_for_quantization`` -- the reference does that inside its
  communicator (:281-284) -- and the byte exchange is ``graph.exchange_quantized``, a
  callable ``(comm_splits, comm_buf_for_quantization, tag, direction) -> handle | None``:
  on "forward" it must leave the peers' packed rows in ``quantized_recv_data_buf`` and
  their (zero_point, scale) rows, rounded through bf16 as on the reference's wire
  (:297-303), in ``quantized_recv_params_buf_fp32``; on "backward" the same with the
  roles of the send and receive buffers swapped (:266-276).  The received rows are
  dequantised after the wait, where the reference does it (aggregator.py:83-88,
  :180-187).  Outside training the forward exchange stays fp32 (communicator.py:64-65).
* With ``num_bits`` 16 (communicator.py:65-66, :111-137) the outgoing rows are rounded to bf16 into
  ``comm_buf.send_buf_fp16`` (backward: ``recv_buf_fp16``) and ``graph.exchange_bf16``, same call
  shape as ``graph.exchange``, must leave the peers' bf16 rows in ``comm_buf.recv_buf_fp16``
  (backward: ``send_buf_fp16``); they are widened to fp32 after the wait.  Outside training the
  forward exchange stays fp32.
* No process group or timers are touched; the quantiser is built from the buffers' width,
  not looked up as a singleton.
* ``torch.zeros`` + accumulate (aggregator.py:67-70, :167-170) and ``zero_()`` +
  accumulate (:44-49, :144-149) run as one overwriting SpMM; the values are identical
  because an FMA chain started from a stored 0 equals one started from a register 0.
* The backward ``index_add_`` (:197-199) runs as a deterministic SpMM with the
  selection matrix of ``idx_nodes_send_to_others``.
* ``graph.one_launch = True`` (off by default) runs the local product and the product with
  the received rows as ONE launch over ``[A_local | A_from]`` and the two dense operands
  (``sparse_tensor.side_by_side``): every output row is one FMA chain -- local elements, then
  received ones, the order of aggregator.py:70 then :102 -- written once, instead of written by
  the local product and read and written again behind the exchange.  Same bits, fewer bytes;
  the price is that the local product no longer runs while the exchange is in flight, so it
  pays where the exchange is short next to the local product.  Received rows are read in the
  format they arrived in (fp32, bf16, packed); dense features only (packed features and the
  row-restricted backward run the separate launches).

``AggregatorPacked`` is the same pipeline for local features handed over packed
(``packed.py``: non-zero values at the front of each row plus a bitmap header); only the
two forward products that read the features differ.
"""

import torch

from . import _lib, computation_ops, packed
from .sparse_tensor import SparseTensor, _rows_are_dense, side_by_side
from .spmm_kernel import SPMM_backward, SPMM_backward_quantized, SPMM_forward, SPMM_forward_quantized


def _gather_rows(src: torch.Tensor, index: torch.Tensor, out: torch.Tensor) -> None:
    # torch.index_select(local_nodes_feat, 0, idx, out=send_buf)   (aggregator.py:51)
    if not (src.is_cuda and index.is_cuda and out.is_cuda):
        raise RuntimeError("gather operands must be GPU (HIP) tensors; there is no CPU path")
    if src.dtype != torch.float32 or out.dtype not in (torch.float32, torch.bfloat16) or index.dtype != torch.int64:
        raise RuntimeError("Input mismatch: gather needs float32 rows and int64 indices")
    if out.size(0) != index.numel() or out.size(1) != src.size(1) or not out.is_contiguous():
        raise RuntimeError("Input mismatch: gather output shape")
    src = src.contiguous()
    # torch.index_select raises on an index outside the source; here the list is looked at once (cached per tensor)
    _lib.check_index(index, src.size(0), what="boundary row list (idx_nodes_send_to_others)")
    # bf16 result rows: the gather and the copy into the staging buffer of a 16-bit exchange in one pass
    L = _lib.lib()
    entry = L.gnnagg_gather_rows_f32_bf16 if out.dtype == torch.bfloat16 else L.gnnagg_gather_rows_f32
    with torch.cuda.device(src.device):
        _lib.check(entry(_lib.ptr(src), src.size(0), _lib.ptr(index), _lib.ptr(out), index.numel(), src.size(1),
                         _lib.current_stream(src.device)))


def _check_bits(num_bits: int) -> None:
    if num_bits not in (32, 16, 8, 4, 2):
        raise NotImplementedError("boundary exchange with num_bits=%r is not defined" % (num_bits,))


def _quantized(graph, num_bits: int) -> bool:
    # aggregator.py:35, :83, :136, :180: quantised buffers are used for widths other than 32 / 16
    if num_bits in (32, 16):
        return False
    qbuf = getattr(graph, "comm_buf_for_quantization", None)
    if qbuf is None or qbuf.bits != num_bits:
        raise RuntimeError("Input mismatch: the graph holds no %d-bit quantisation buffers "
                           "(build it with bits=%d)" % (num_bits, num_bits))
    if getattr(graph, "exchange_quantized", None) is None:
        raise RuntimeError("graph.exchange_quantized is required for a %d-bit boundary exchange" % num_bits)
    return True


def _bf16_wire(graph) -> bool:
    """communicator.py:65-66, :111-137: with ``num_bits == 16`` the rows travel as bf16 through the
    staging copies of ``CommBuffer``; the exchange of those copies is ``graph.exchange_bf16``."""
    cb = graph.comm_buf
    if getattr(cb, "send_buf_fp16", None) is None or getattr(cb, "recv_buf_fp16", None) is None:
        raise RuntimeError("Input mismatch: the graph holds no bf16 staging buffers (build it with bits=16)")
    if getattr(graph, "exchange_bf16", None) is None:
        raise RuntimeError("graph.exchange_bf16 is required for a 16-bit boundary exchange")
    return True


def _bf16_in_the_products(graph, feats_or_grad, feat_len: int) -> bool:
    """Whether the products next to a 16-bit exchange read and write the bf16 staging buffers themselves (the
    default; ``graph.fuse_bf16_staging = False`` keeps the two tensor copies of communicator.py:128,137 as separate
    passes).  The bits are the same either way: the copy rounds the fp32 sum to nearest even, widening is exact."""
    if getattr(graph, "fuse_bf16_staging", True) is False or feat_len % 4 != 0:
        return False
    t = getattr(feats_or_grad, "feat", feats_or_grad)
    return isinstance(t, torch.Tensor) and t.dtype == torch.float32


def _convert(src: torch.Tensor, dst: torch.Tensor) -> None:
    """fp32 -> bf16 (round to nearest even) or bf16 -> fp32: the two ``copy_`` calls around the
    16-bit exchange (communicator.py:128, :137)."""
    if src.numel() != dst.numel() or not src.is_contiguous() or not dst.is_contiguous() or not src.is_cuda:
        raise RuntimeError("Input mismatch: bf16 staging needs contiguous GPU (HIP) buffers of equal size")
    L = _lib.lib()
    with torch.cuda.device(src.device):
        if src.dtype == torch.float32 and dst.dtype == torch.bfloat16:
            _lib.check(L.gnnagg_f32_to_bf16(_lib.ptr(src), _lib.ptr(dst), src.numel(), _lib.current_stream(src.device)))
        elif src.dtype == torch.bfloat16 and dst.dtype == torch.float32:
            _lib.check(L.gnnagg_bf16_to_f32(_lib.ptr(src), _lib.ptr(dst), src.numel(), _lib.current_stream(src.device)))
        else:
            raise RuntimeError("Input mismatch: bf16 staging converts float32 <-> bfloat16 only")


def _poison_unfilled_rows(graph) -> None:
    """Once per pair of boundary buffers, when a run first lets the products write / read the exchange format
    themselves: the fp32 ``send_buf`` / ``recv_buf`` -- which the reference always fills (aggregator.py:85-88,
    communicator.py:128, :137) and these runs no longer touch -- are set to NaN over their whole storage, so that a
    hook or debugging code that still reads them sees at once that the rows are not there, instead of stale ones."""
    buf = graph.comm_buf
    if getattr(buf, "_fp32_rows_poisoned", False):
        return
    for t in (buf.send_buf, buf.recv_buf):
        whole = torch.empty(0, dtype=t.dtype, device=t.device).set_(t.untyped_storage())
        whole.fill_(float("nan"))
    buf._fp32_rows_poisoned = True


def _outgoing_quantized(graph, direction: str):
    """(fp32 rows, packed bytes, parameters, per-rank row prefix) of the outgoing side of a quantised exchange."""
    qbuf = graph.comm_buf_for_quantization
    if direction == "forward":
        return (graph.comm_buf.send_buf, qbuf.quantized_send_data_buf, qbuf.quantized_send_params_buf_fp32,
                qbuf.quantized_work_range_per_proc)
    return (graph.comm_buf.recv_buf, qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32,
            qbuf.dequantized_work_range_per_proc)


# the one-pass kernel gives a row to one lane group from its first element to its last; a matrix with a longer row than
# this goes through the product kernels (which spread such rows) and the quantise pass instead
_ONE_PASS_MAX_ROW_LEN = 4096


def _product_into_packed_rows(graph, plan, csr, dense: torch.Tensor, num_bits: int, direction: str) -> bool:
    """The product in front of a quantised exchange writing the packed bytes and parameters itself
    (``computation_ops.spmm_quantize_for_all_procs``: same bytes as the product followed by the quantise pass, without the
    fp32 rows; the fp32 buffer is then NOT filled).  The default; ``graph.fuse_quantize = False`` keeps the two passes.
    ``csr``: (rowptr, col, value) of the matrix whose rows are the outgoing rows, ``plan`` its plan.  False when
    nothing was done."""
    if (getattr(graph, "fuse_quantize", True) is False or dense.dtype != torch.float32 or csr[2] is None
            or plan.max_row_len > _ONE_PASS_MAX_ROW_LEN):
        return False
    _, data, params, work_range = _outgoing_quantized(graph, direction)
    if csr[0].numel() - 1 == 0:
        return False
    world = len(graph.comm_splits.send_splits)
    return computation_ops.spmm_quantize_for_all_procs(csr[0], csr[1], csr[2], dense, data, params, work_range, world,
                                                        num_bits)


def _transposed_csr(m: SparseTensor):
    s = m.storage
    return s.colptr(), s.row_T(), s.value_T()


def _transposed_matrix(m: SparseTensor) -> SparseTensor:
    """``m^T`` as a matrix of its own over the transposed arrays of ``m`` (kept on ``m``)."""
    hit = m.__dict__.get("_transposed_matrix")
    if hit is None:
        colptr, row_t, value_t = _transposed_csr(m)
        hit = m.__dict__["_transposed_matrix"] = SparseTensor(
            rowptr=colptr, col=row_t, value=value_t, sparse_sizes=(m.sparse_size(1), m.sparse_size(0)), is_sorted=True)
    return hit


def _quantize_and_exchange(graph, num_bits: int, tag: str, direction: str, already_packed: bool = False):
    """Pack the outgoing rows per peer rank (unless the product wrote them packed) and hand the bytes to the exchange
    (communicator.py:241-311)."""
    qbuf = graph.comm_buf_for_quantization
    world = len(graph.comm_splits.send_splits)
    if already_packed:
        return graph.exchange_quantized(graph.comm_splits, qbuf, tag, direction)
    outgoing, data, params, work_range = _outgoing_quantized(graph, direction)
    if outgoing.size(0) != 0:
        computation_ops.quantize_tensor_for_all_procs(outgoing, data, params, work_range, world, num_bits)
    return graph.exchange_quantized(graph.comm_splits, qbuf, tag, direction)


def _fused_dequantize(graph, feat_len: int) -> bool:
    """Whether the received rows of a quantised exchange are aggregated straight from the packed bytes (the default:
    same values, no fp32 pass over the buffer; the fp32 buffer is then NOT filled, unlike aggregator.py:85-88).
    ``graph.fuse_dequantize = False`` keeps the dequantise pass of its own.  Needs a width that is a multiple of 4."""
    return getattr(graph, "fuse_dequantize", True) is not False and feat_len % 4 == 0


def _dequantize_received(graph, num_bits: int, direction: str) -> None:
    qbuf = graph.comm_buf_for_quantization
    world = len(graph.comm_splits.send_splits)
    if direction == "forward":  # aggregator.py:85-88
        incoming, data, params, work_range = (graph.comm_buf.recv_buf, qbuf.quantized_recv_data_buf,
                                              qbuf.quantized_recv_params_buf_fp32,
                                              qbuf.dequantized_work_range_per_proc)
    else:  # aggregator.py:182-187
        incoming, data, params, work_range = (graph.comm_buf.send_buf, qbuf.quantized_send_data_buf,
                                              qbuf.quantized_send_params_buf_fp32, qbuf.quantized_work_range_per_proc)
    if incoming.size(0) != 0:
        computation_ops.dequantize_tensor_for_all_procs(data, incoming, params, work_range, world, num_bits)


def _kernel_rows(t: torch.Tensor) -> bool:
    """fp32 rows as the two-format launches take them: 16-byte aligned, row stride a multiple of 4 floats."""
    return t.data_ptr() % 16 == 0 and (t.size(0) <= 1 or t.stride(0) % 4 == 0)


def _one_launch_product(graph, both: SparseTensor, dense: torch.Tensor, result: torch.Tensor, accumulate: bool,
                        num_bits: int, direction: str, quantized: bool, half: bool, half_fused: bool, feat_len: int):
    """``result (+)= both @ (dense ; received rows)`` in one launch (``graph.one_launch``), the received rows read in
    the format they arrived in -- fp32, bf16 or packed -- where the products read exchange formats themselves
    (``fuse_dequantize`` / ``fuse_bf16_staging``), after the reference's dequantise / copy pass otherwise."""
    buf, qbuf = graph.comm_buf, graph.comm_buf_for_quantization if quantized else None
    plan, value = both.get_plan(), both.csr()[2]
    formats_ok = feat_len % 4 == 0 and _kernel_rows(dense) and _kernel_rows(result)
    if quantized:
        if _fused_dequantize(graph, feat_len) and formats_ok:
            _poison_unfilled_rows(graph)
            if direction == "forward":
                second = (qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32, qbuf.recv_row_code, num_bits)
            else:
                second = (qbuf.quantized_send_data_buf, qbuf.quantized_send_params_buf_fp32, qbuf.send_row_code, num_bits)
            plan.spmm_dense_then(value, both.first_counts, dense, second, result, accumulate)
            return
        _dequantize_received(graph, num_bits, direction)
    elif half:
        rows16 = buf.recv_buf_fp16 if direction == "forward" else buf.send_buf_fp16
        if half_fused and formats_ok:
            plan.spmm_dense_then(value, both.first_counts, dense, rows16, result, accumulate)
            return
        _convert(rows16, buf.recv_buf if direction == "forward" else buf.send_buf)
    plan.spmm_two_sources(value, dense, buf.recv_buf if direction == "forward" else buf.send_buf, result, accumulate)


class _DenseFeatures:
    """The local features as the forward pipeline reads them: two products and a row gather."""

    def __init__(self, feat: torch.Tensor):
        # a column block of a wider row-major tensor is read where it lies
        self.feat = feat if _rows_are_dense(feat) else feat.contiguous()
        self.width, self.device = feat.size(-1), feat.device

    def product(self, adj, out, accumulate):
        SPMM_forward(adj, self.feat, out, accumulate=accumulate)

    def gather(self, index, out):
        _gather_rows(self.feat, index, out)


class _PackedFeatures:
    """The same for features kept packed (non-zero values at the front of each row + header)."""

    def __init__(self, values: torch.Tensor, header: torch.Tensor):
        self.values, self.header = values, header
        self.width, self.device = values.size(-1), values.device

    def product(self, adj, out, accumulate):
        packed.spmm(adj, self.values, self.header, out, accumulate=accumulate)

    def gather(self, index, out):
        raise NotImplementedError("raw boundary rows of packed features: use pre-aggregation (is_pre_delay=True)")


class Aggregator(torch.autograd.Function):
    @staticmethod
    def forward(ctx, graph, local_nodes_feat, layer, num_bits: int, is_pre_delay: bool, is_training: bool):
        return _forward(ctx, graph, _DenseFeatures(local_nodes_feat), layer, num_bits, is_pre_delay, is_training)

    @staticmethod
    def backward(ctx, local_out_grad):
        return (None, _backward(ctx, local_out_grad), None, None, None, None)


class AggregatorPacked(torch.autograd.Function):
    """``Aggregator`` for features given packed (``packed.empty`` / the packing epilogue): the
    forward products read only the non-zero values; the backward is the dense one, and its
    result is the gradient with respect to the dense features the packed pair stands for."""

    @staticmethod
    def forward(ctx, graph, values, header, layer, num_bits: int, is_pre_delay: bool, is_training: bool):
        return _forward(ctx, graph, _PackedFeatures(values, header), layer, num_bits, is_pre_delay, is_training)

    @staticmethod
    def backward(ctx, local_out_grad):
        return (None, _backward(ctx, local_out_grad), None, None, None, None, None)


def _check_result(out: torch.Tensor, rows: int, feat_len: int, device) -> None:
    if (out.dtype != torch.float32 or out.device != device or tuple(out.shape) != (rows, feat_len)
            or not _rows_are_dense(out)):
        raise RuntimeError("Input mismatch: the result must be a float32 [%d, %d] tensor on %s with contiguous rows"
                           % (rows, feat_len, device))


def _forward(ctx, graph, feats, layer, num_bits: int, is_pre_delay: bool, is_training: bool, out=None,
             accumulate: bool = False):
    """``out``: where to write the result -- e.g. a column block of a wider tensor; a fresh tensor
    when None.  Every row is overwritten unless ``accumulate``, which adds onto what ``out`` holds."""
    _check_bits(num_bits)
    ctx.graph = graph
    ctx.num_bits = num_bits
    ctx.is_pre_delay = is_pre_delay
    ctx.layer = layer

    feat_len = feats.width
    graph.comm_buf.resize_buffer(graph.comm_splits, feat_len, num_bits)
    exchange = getattr(graph, "exchange", None)
    quantized = exchange is not None and _quantized(graph, num_bits)
    if quantized:
        graph.comm_buf_for_quantization.resize_buffer(graph.comm_splits, feat_len, num_bits)
    quantized = quantized and is_training  # communicator.py:64-65: fp32 rows outside training
    half = exchange is not None and num_bits == 16 and is_training and _bf16_wire(graph)
    comm_handle = None
    send_buf = graph.comm_buf.send_buf

    half_fused = half and isinstance(feats, _DenseFeatures) and _bf16_in_the_products(graph, feats, feat_len)
    if exchange is not None:
        packed_by_product = False
        if is_pre_delay:  # pre-aggregation: send_buf = A_to @ X (straight into the rows that travel, bf16 or packed)
            if quantized and isinstance(feats, _DenseFeatures) and send_buf.size(0) != 0:
                to = graph.adj_t_pre_post_aggr_to
                packed_by_product = _product_into_packed_rows(graph, to.get_plan(), to.csr(), feats.feat, num_bits,
                                                              "forward")
            if not packed_by_product:
                feats.product(graph.adj_t_pre_post_aggr_to, graph.comm_buf.send_buf_fp16 if half_fused else send_buf, False)
        elif (quantized and isinstance(feats, _DenseFeatures) and send_buf.size(0) != 0
              and getattr(graph, "fuse_quantize", True) is not False and feats.feat.is_contiguous()):
            # raw boundary rows quantised as they are gathered (the fp32 send rows are not written)
            _, data, params, work_range = _outgoing_quantized(graph, "forward")
            computation_ops.gather_quantize_for_all_procs(feats.feat, graph.idx_nodes_send_to_others, data, params,
                                                          work_range, len(graph.comm_splits.send_splits), num_bits)
            packed_by_product = True
        else:  # raw boundary rows (as bf16 at once when they travel so)
            feats.gather(graph.idx_nodes_send_to_others, graph.comm_buf.send_buf_fp16 if half_fused else send_buf)
        if packed_by_product or half_fused:
            _poison_unfilled_rows(graph)
        if quantized:
            comm_handle = _quantize_and_exchange(graph, num_bits, f"forward{layer}", "forward", packed_by_product)
        elif half:
            if not half_fused:
                _convert(send_buf, graph.comm_buf.send_buf_fp16)
            comm_handle = graph.exchange_bf16(graph.comm_splits, graph.comm_buf, f"forward{layer}", "forward")
        else:
            comm_handle = exchange(graph.comm_splits, graph.comm_buf, f"forward{layer}", "forward")

    if out is None:
        out = torch.empty([graph.local_adj_t.sparse_size(0), feat_len], dtype=torch.float32, device=feats.device)
        accumulate = False
    else:
        _check_result(out, graph.local_adj_t.sparse_size(0), feat_len, feats.device)
    remote_adj = None
    if exchange is not None:
        remote_adj = graph.adj_t_pre_post_aggr_from if is_pre_delay else graph.remote_adj_t
    one_launch = (getattr(graph, "one_launch", False) is True and remote_adj is not None
                  and isinstance(feats, _DenseFeatures) and feats.feat.dtype == torch.float32
                  and graph.comm_buf.recv_buf.size(0) != 0)
    if one_launch:  # local elements, then received ones: one chain per output row, one launch
        if comm_handle is not None:
            comm_handle.wait()
        both = side_by_side(graph.local_adj_t, remote_adj)
        _one_launch_product(graph, both, feats.feat, out, accumulate, num_bits, "forward", quantized,
                            half, half_fused, feat_len)
        return out
    feats.product(graph.local_adj_t, out, accumulate)

    if comm_handle is not None:
        comm_handle.wait()
    fused = quantized and _fused_dequantize(graph, feat_len) and out.stride(0) % 4 == 0
    if fused:
        _poison_unfilled_rows(graph)
    if quantized and not fused:
        _dequantize_received(graph, num_bits, "forward")
    half_fused = half_fused and out.stride(0) % 4 == 0
    if half and not half_fused:
        _convert(graph.comm_buf.recv_buf_fp16, graph.comm_buf.recv_buf)

    # (fused: the received bf16 rows are gathered as they are; recv_buf is not written)
    remote_nodes_feat = graph.comm_buf.recv_buf_fp16 if half_fused else graph.comm_buf.recv_buf
    if exchange is not None and remote_nodes_feat.size(0) != 0:
        adj = remote_adj  # post-aggregation / raw halo
        if fused:
            qbuf = graph.comm_buf_for_quantization
            SPMM_forward_quantized(adj, qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32,
                                   qbuf.recv_row_code, out, num_bits)
        else:
            SPMM_forward(adj, remote_nodes_feat, out)
    return out


class _BackwardSupport:
    """The transposed matrices of one layer's gradient direction with only the entries that meet a given set of
    gradient rows (``restricted_transpose``)."""

    def __init__(self, local_T, remote_T):
        self.local_T, self.remote_T = local_T, remote_T


def restricted_transpose(m: SparseTensor, row_mask: torch.Tensor) -> SparseTensor:
    """``m^T`` as a CSR of its own, keeping only the entries of ``m`` whose row is set in ``row_mask``: for a dense
    operand ``g`` whose other rows are zero, ``restricted @ g == m^T @ g`` -- every term left out is a product with
    zero, and the terms kept stay in their order, so each output row is the same FMA chain (up to the sign of a zero)."""
    s = m.storage
    colptr, row_t, value_t = s.colptr(), s.row_T(), s.value_T()
    keep = row_mask[row_t]
    kept_before = torch.zeros(row_t.numel() + 1, dtype=torch.int64, device=row_t.device)
    torch.cumsum(keep, dim=0, out=kept_before[1:])
    value = None if value_t is None else value_t[keep]
    return SparseTensor(rowptr=kept_before[colptr], col=row_t[keep], value=value,
                        sparse_sizes=(m.sparse_size(1), m.sparse_size(0)), is_sorted=True)


def backward_support(graph, rows: torch.Tensor, is_pre_delay: bool) -> _BackwardSupport:
    """What ``_backward`` needs to skip the zero rows of a gradient that is non-zero only in ``rows`` (local node
    ids): the restricted transposes of the local matrix and of the matrix that produces the outgoing halo gradients.
    Built once per (graph, row set) and kept on the graph."""
    cache = graph.__dict__.setdefault("_backward_support_cache", {})
    # (a shallow copy of a graph with other matrices -- degrees folded into the values -- shares this dictionary)
    key = (rows.data_ptr(), rows.numel(), rows._version, bool(is_pre_delay), id(graph.local_adj_t))
    hit = cache.get(key)
    if hit is None:
        n = graph.local_adj_t.sparse_size(0)
        mask = torch.zeros(n, dtype=torch.bool, device=rows.device)
        mask[rows] = True
        remote = graph.adj_t_pre_post_aggr_from if is_pre_delay else graph.remote_adj_t
        built = _BackwardSupport(restricted_transpose(graph.local_adj_t, mask),
                                 restricted_transpose(remote, mask) if remote is not None else None)
        for t in (built.local_T, built.remote_T):
            if t is not None:
                t.get_plan()
        if len(cache) >= 4:
            cache.clear()
        hit = cache[key] = (rows, built, graph.local_adj_t)  # holding the tensors keeps their addresses their own
    return hit[1]


def select_rows(m: SparseTensor, rows: torch.Tensor) -> SparseTensor:
    """``m[rows, :]`` as a CSR of its own (row i of the result is row ``rows[i]`` of ``m``, entries in their order)."""
    rowptr, col, value = m.csr()
    start = rowptr[rows]
    counts = rowptr[rows + 1] - start
    new_rowptr = torch.zeros(rows.numel() + 1, dtype=torch.int64, device=rowptr.device)
    torch.cumsum(counts, dim=0, out=new_rowptr[1:])
    total = int(new_rowptr[-1])
    index = (torch.arange(total, dtype=torch.int64, device=rowptr.device)
             + torch.repeat_interleave(start - new_rowptr[:-1], counts, output_size=total))
    return SparseTensor(rowptr=new_rowptr, col=col[index], value=None if value is None else value[index],
                        sparse_sizes=(rows.numel(), m.sparse_size(1)), is_sorted=True)


class _RowRestrictedGraph:
    """``graph`` with a few attributes replaced; everything else (buffers, splits, exchange hooks, the matrices that
    feed the send buffer) is read from ``graph`` at the time of use, so what is attached to it later is seen here."""

    def __init__(self, graph, replaced: dict):
        self.__dict__["_graph"] = graph
        self.__dict__.update(replaced)

    def __getattr__(self, name):  # only reached for names this object does not hold itself
        graph = self.__dict__.get("_graph")
        if graph is None or name.startswith("__"):
            raise AttributeError(name)
        return getattr(graph, name)


def restrict_output_rows(graph, rows: torch.Tensor, is_pre_delay: bool):
    """A view of ``graph`` whose aggregation produces only the output rows ``rows`` (local node ids, in that order):
    the local matrix and the matrix that adds the received rows keep just those rows, the in-degrees likewise; what
    is sent to other ranks is untouched.  ``Aggregator`` on it returns ``Aggregator(graph, ...)[rows]`` -- each kept
    row is the same FMA chain -- at the cost of those rows only, forward and backward.  For the last layer of a model
    whose loss scores a subset of the nodes.  Built once per (graph, row set) and kept on the graph."""
    cache = graph.__dict__.setdefault("_restricted_rows_cache", {})
    # (a shallow copy of a graph with other matrices -- degrees folded into the values -- shares this dictionary)
    key = (rows.data_ptr(), rows.numel(), rows._version, bool(is_pre_delay), id(graph.local_adj_t))
    hit = cache.get(key)
    if hit is None:
        name = "adj_t_pre_post_aggr_from" if is_pre_delay else "remote_adj_t"
        remote = getattr(graph, name, None)
        g = _RowRestrictedGraph(graph, {
            "local_adj_t": select_rows(graph.local_adj_t, rows),
            name: None if remote is None else select_rows(remote, rows),
            "in_degrees": graph.in_degrees[rows].contiguous(),
            "backward_row_support": None})
        for m in (g.local_adj_t, getattr(g, name)):
            if m is not None:
                m.get_plan()
                m.get_plan_for_transpose()
        if len(cache) >= 4:
            cache.clear()
        hit = cache[key] = (rows, g, graph.local_adj_t)  # holding the tensors keeps their addresses their own
    return hit[1]


def _backward(ctx, local_out_grad, out=None, accumulate: bool = False):
    """``out`` / ``accumulate``: write the gradient into ``out`` (a column block of a wider tensor
    is fine), on top of what it holds when ``accumulate``; a fresh tensor when ``out`` is None."""
    graph = ctx.graph
    num_bits = ctx.num_bits
    is_pre_delay = ctx.is_pre_delay
    layer = f"backward{ctx.layer}"

    if not _rows_are_dense(local_out_grad):
        local_out_grad = local_out_grad.contiguous()
    feat_len = local_out_grad.size(-1)
    graph.comm_buf.resize_buffer(graph.comm_splits, feat_len, num_bits)
    exchange = getattr(graph, "exchange", None)
    quantized = exchange is not None and _quantized(graph, num_bits)
    if quantized:
        graph.comm_buf_for_quantization.resize_buffer(graph.comm_splits, feat_len, num_bits)

    # the receive buffer carries the outgoing halo gradients on the way back
    # a caller that knows the gradient to be zero outside a set of rows (a loss that scores only the training nodes,
    # for the last layer) declares it in graph.backward_row_support[layer]: the products below then skip those rows
    support = (getattr(graph, "backward_row_support", None) or {}).get(ctx.layer)
    half = exchange is not None and num_bits == 16 and _bf16_wire(graph)
    half_fused = half and not quantized and _bf16_in_the_products(graph, local_out_grad, feat_len)
    # the outgoing halo gradients: straight into the bf16 staging rows when they travel as bf16
    remote_nodes_grad_buf = graph.comm_buf.recv_buf_fp16 if half_fused else graph.comm_buf.recv_buf
    packed_by_product = False
    if remote_nodes_grad_buf.size(0) != 0:
        remote = graph.adj_t_pre_post_aggr_from if is_pre_delay else graph.remote_adj_t
        if quantized:  # straight into the packed rows that travel
            if support is not None:
                plan, csr = support.remote_T.get_plan(), support.remote_T.csr()
            else:
                plan, csr = remote.get_plan_for_transpose(), _transposed_csr(remote)
            packed_by_product = _product_into_packed_rows(graph, plan, csr, local_out_grad, num_bits, "backward")
        if packed_by_product:
            pass
        elif support is not None:
            SPMM_forward(support.remote_T, local_out_grad, remote_nodes_grad_buf, accumulate=False)
        else:
            SPMM_backward(remote, local_out_grad, remote_nodes_grad_buf, accumulate=False)

    if packed_by_product or half_fused:
        _poison_unfilled_rows(graph)
    comm_handle = None
    if quantized:
        comm_handle = _quantize_and_exchange(graph, num_bits, layer, "backward", packed_by_product)
    elif half:  # the buffers swap roles on the way back (communicator.py:121-126)
        if not half_fused:
            _convert(remote_nodes_grad_buf, graph.comm_buf.recv_buf_fp16)
        comm_handle = graph.exchange_bf16(graph.comm_splits, graph.comm_buf, layer, "backward")
    elif exchange is not None:
        comm_handle = exchange(graph.comm_splits, graph.comm_buf, layer, "backward")

    if out is None:
        local_nodes_grad = torch.empty([graph.local_adj_t.sparse_size(-1), feat_len], dtype=torch.float32,
                                       device=local_out_grad.device)
        accumulate = False
    else:
        _check_result(out, graph.local_adj_t.sparse_size(-1), feat_len, local_out_grad.device)
        local_nodes_grad = out
    one_launch = (getattr(graph, "one_launch", False) is True and exchange is not None and support is None
                  and local_out_grad.dtype == torch.float32 and graph.comm_buf.send_buf.size(0) != 0)
    if one_launch:  # [A_local^T | A_to^T] over the gradient and the received gradient rows, one chain per row
        if comm_handle is not None:
            comm_handle.wait()
        if is_pre_delay:
            both = side_by_side(graph.local_adj_t, graph.adj_t_pre_post_aggr_to, transposed=True)
        else:  # local^T next to the selection matrix of the boundary row list (itself untransposed)
            both = side_by_side(_transposed_matrix(graph.local_adj_t), graph.send_scatter_adj_t())
        _one_launch_product(graph, both, local_out_grad, local_nodes_grad, accumulate, num_bits, "backward", quantized,
                            half, half_fused, feat_len)
        return local_nodes_grad
    if support is not None:
        SPMM_forward(support.local_T, local_out_grad, local_nodes_grad, accumulate=accumulate)
    else:
        SPMM_backward(graph.local_adj_t, local_out_grad, local_nodes_grad, accumulate=accumulate)

    if comm_handle is not None:
        comm_handle.wait()
    fused = quantized and _fused_dequantize(graph, feat_len) and local_nodes_grad.stride(0) % 4 == 0
    if fused:
        _poison_unfilled_rows(graph)
    if quantized and not fused:
        _dequantize_received(graph, num_bits, "backward")
    half_fused = half_fused and local_nodes_grad.stride(0) % 4 == 0
    if half and not half_fused:
        _convert(graph.comm_buf.send_buf_fp16, graph.comm_buf.send_buf)

    local_nodes_grad_buf = graph.comm_buf.send_buf_fp16 if half_fused else graph.comm_buf.send_buf
    if exchange is not None and local_nodes_grad_buf.size(0) != 0:
        qbuf = graph.comm_buf_for_quantization
        if is_pre_delay:
            if fused:
                SPMM_backward_quantized(graph.adj_t_pre_post_aggr_to, qbuf.quantized_send_data_buf,
                                        qbuf.quantized_send_params_buf_fp32, qbuf.send_row_code, local_nodes_grad,
                                        num_bits)
            else:
                SPMM_backward(graph.adj_t_pre_post_aggr_to, local_nodes_grad_buf, local_nodes_grad)
        elif fused:
            SPMM_forward_quantized(graph.send_scatter_adj_t(), qbuf.quantized_send_data_buf,
                                   qbuf.quantized_send_params_buf_fp32, qbuf.send_row_code, local_nodes_grad, num_bits)
        else:
            SPMM_forward(graph.send_scatter_adj_t(), local_nodes_grad_buf, local_nodes_grad)
    return local_nodes_grad
