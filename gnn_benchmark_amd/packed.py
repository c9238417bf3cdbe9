"""Packed activations: the output of a ReLU + dropout layer kept with every row's non-zero
values at the front of the row plus a per-row bitmap header, so that the next layer's
aggregation gathers only what is not zero (about a quarter of each row in training).

This is a layout between this build's own fused epilogue and its own SpMM kernel; the
reference keeps activations dense (self_benchmark/a64fx/model/DistSAGE.py:55-66).  Skipping a
zero leaves a row's FMA chain as it is, so the aggregation equals the dense one up to the
sign of a zero.
"""
import torch

from . import _lib
from .sparse_tensor import SparseTensor

SLACK = 4  # floats past the last row that the consumer's 16-byte loads may touch


def header_words(feat: int) -> int:
    """32-bit words of one row's header, 0 when the width cannot be packed (32, 64, 128, 256 can)."""
    return int(_lib.lib().gnnagg_packed_header_words(int(feat)))


def empty(rows: int, feat: int, device):
    """(values [rows, feat] fp32 with the required slack behind them, header [rows, words] int32)."""
    words = header_words(feat)
    if words == 0:
        raise RuntimeError("Input mismatch: packed activations exist for widths 32, 64, 128 and 256")
    store = torch.empty(rows * feat + SLACK, dtype=torch.float32, device=device)
    store[rows * feat:].zero_()
    return store[:rows * feat].view(rows, feat), torch.empty(rows, words, dtype=torch.int32, device=device)


def _check(values: torch.Tensor, header: torch.Tensor) -> int:
    if not (values.is_cuda and header.is_cuda):
        raise RuntimeError("packed activations live on a GPU (HIP) device only")
    words = header_words(values.size(1)) if values.dim() == 2 else 0
    if (words == 0 or values.dtype != torch.float32 or not values.is_contiguous() or header.dtype != torch.int32
            or not header.is_contiguous() or tuple(header.shape) != (values.size(0), words)):
        raise RuntimeError("Input mismatch: packed values must be contiguous float32 [rows, 32|64|128|256] with an "
                           "int32 [rows, words] header")
    if values.untyped_storage().nbytes() < (values.storage_offset() + values.numel() + SLACK - 1) * 4:
        raise RuntimeError("Input mismatch: packed values need %d floats of slack behind the last row "
                           "(allocate them with packed.empty)" % SLACK)
    return words


def spmm(src: SparseTensor, values: torch.Tensor, header: torch.Tensor, out: torch.Tensor,
         accumulate: bool = True) -> None:
    """``out (+)= src @ y`` where ``y`` is given packed: ``SPMM_forward`` for a packed operand."""
    _check(values, header)
    _, _, value = src.csr()
    if value is None or value.dtype != torch.float32:
        raise RuntimeError("Input mismatch: the sparse matrix needs float32 values")
    rows, cols = src.sparse_sizes()
    if (not out.is_cuda or out.dtype != torch.float32 or not out.is_contiguous() or out.dim() != 2
            or out.size(0) < rows or out.size(1) != values.size(1) or values.size(0) < cols):
        raise RuntimeError("Input mismatch: operand shapes do not match the sparse matrix")
    plan = src.get_plan()
    with torch.cuda.device(out.device):
        _lib.check(_lib.lib().gnnagg_plan_spmm_packed_f32(
            plan._handle, _lib.ptr(value.contiguous()), _lib.ptr(values), _lib.ptr(header), _lib.ptr(out),
            values.size(1), 1 if accumulate else 0, _lib.current_stream(out.device)))


def unpack(values: torch.Tensor, header: torch.Tensor) -> torch.Tensor:
    """The dense tensor a packed pair stands for (torch ops; for tests and debugging)."""
    rows, feat = values.shape
    bitmap = header[:, 0::2].to(torch.int64) & 0xFFFFFFFF   # (bitmap, non-zeros in front) pairs
    bits = ((bitmap.unsqueeze(-1) >> torch.arange(32, device=values.device)) & 1).reshape(rows, feat).bool()
    rank = torch.cumsum(bits.to(torch.int64), dim=1) - 1
    dense = torch.gather(values, 1, rank.clamp(min=0))
    return torch.where(bits, dense, torch.zeros_like(dense))
