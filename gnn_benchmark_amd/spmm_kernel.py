"""Operator wrappers with the reference's names and call shapes.

Reference: self_benchmark/a64fx/model/ops/spmm_kernel.py:45-67 (``SPMM_forward``) and
:71-90 (``SPMM_backward``).  Both accumulate into the caller's ``out``.  The forward
feeds the CSR arrays, the backward feeds the transposed arrays to the SAME kernel, so
``out += A.T @ other``; no gradient with respect to the sparse values exists.

What the reference caches per matrix -- the CPU thread split from
``distribute_work_for_row`` (:7-28) -- has no meaning on a GPU; the per-matrix object
cached here is the degree-binned plan (``SparseTensor.get_plan``).
"""
import torch

from . import _lib
from .sparse_tensor import SparseTensor, _row_stride, _rows_are_dense


def _as_f32(value: torch.Tensor, other: torch.Tensor) -> torch.Tensor:
    # reference: value = value.to(other.dtype) (spmm_kernel.py:59-60); the values stay fp32 beside bf16 rows (the staging
    # buffers of a 16-bit exchange, which the plan widens / rounds itself)
    if other.dtype == torch.bfloat16:
        return value if value.dtype == torch.float32 else value.float()
    return value if value.dtype == other.dtype else value.to(other.dtype)


def SPMM_forward(src: SparseTensor, other: torch.Tensor, out: torch.Tensor, accumulate: bool = True) -> None:
    """``out += src @ other`` (``accumulate=False``: ``out = src @ other``).  Returns None
    like the reference (spmm_kernel.py:65)."""
    _, _, value = src.csr()
    if value is None:
        raise RuntimeError("Input mismatch: the sparse matrix has no values")
    src.get_plan().spmm(_as_f32(value, other), other, out, accumulate)
    return None


def SPMM_backward(src: SparseTensor, other: torch.Tensor, out: torch.Tensor, accumulate: bool = True):
    """``out += src.T @ other`` through the transposed CSR arrays; returns ``(out, None)``
    like the native op it forwards (spmm_kernel.py:90)."""
    value_T = src.storage.value_T()
    if value_T is None:
        raise RuntimeError("Input mismatch: the sparse matrix has no values")
    src.get_plan_for_transpose().spmm(_as_f32(value_T, other), other, out, accumulate)
    return out, None


def _element_codes(plan, col: torch.Tensor, row_code: torch.Tensor) -> torch.Tensor:
    """``(row_code[col[e]] << 32) | col[e]`` per stored element, built once per (matrix, code table) and kept on the
    plan: with it the kernel can ask for a row's bytes as soon as the index chunk has arrived.  The entry keeps the
    code table alive, so its address cannot pass to another tensor while the entry exists; an in-place change bumps
    ``_version``."""
    cache = plan.__dict__.setdefault("_element_codes", {})
    key = (row_code.data_ptr(), row_code._version, int(row_code.numel()))
    hit = cache.get(key)
    if hit is None:
        if len(cache) >= 4:
            cache.clear()
        codes = (row_code[col].to(torch.int64) << 32) | col
        hit = cache[key] = (row_code, codes.contiguous())
    return hit[1]


def _spmm_quantized(plan, value, packed, params, row_code, out, bits, accumulate, operand_rows, col=None):
    if not all(t.is_cuda for t in (value, packed, params, row_code, out)):
        raise RuntimeError("quantised SpMM operands must be GPU (HIP) tensors; there is no CPU path")
    feat = out.size(1) if out.dim() == 2 else -1
    if (packed.dtype != torch.uint8 or not packed.is_contiguous() or packed.dim() != 2 or packed.size(1) != feat
            or params.dtype != torch.float32 or not params.is_contiguous() or tuple(params.shape) != (operand_rows, 2)
            or row_code.dtype != torch.int32 or not row_code.is_contiguous() or row_code.numel() != operand_rows
            or out.dtype != torch.float32 or not _rows_are_dense(out) or value.dtype != torch.float32):
        raise RuntimeError("Input mismatch: quantised SpMM needs uint8 [packed rows, F] bytes, float32 [rows, 2] "
                           "parameters, int32 [rows] row codes and a float32 [*, F] output with contiguous rows")
    # the kernel addresses byte row (row_code >> 3) of the packed buffer: checked once per code tensor and buffer height
    _lib.check_index(row_code, packed.size(0), shift=3, what="row codes of the packed buffer")
    L = _lib.lib()
    with torch.cuda.device(out.device):
        if col is not None and col.numel() > 0:
            codes = _element_codes(plan, col, row_code)
            _lib.check(L.gnnagg_plan_spmm_quantized_elements_f32(
                plan._handle, _lib.ptr(value.contiguous()), _lib.ptr(packed), _lib.ptr(params), _lib.ptr(codes),
                _lib.ptr(out), _row_stride(out), feat, int(bits), 1 if accumulate else 0,
                _lib.current_stream(out.device)))
        else:
            _lib.check(L.gnnagg_plan_spmm_quantized_f32(
                plan._handle, _lib.ptr(value.contiguous()), _lib.ptr(packed), _lib.ptr(params), _lib.ptr(row_code),
                _lib.ptr(out), _row_stride(out), feat, int(bits), 1 if accumulate else 0,
                _lib.current_stream(out.device)))


def SPMM_forward_quantized(src: SparseTensor, packed: torch.Tensor, params: torch.Tensor, row_code: torch.Tensor,
                           out: torch.Tensor, bits: int, accumulate: bool = True) -> None:
    """``out += src @ dequantize(packed, params)`` without materialising the dequantised rows:
    ``SPMM_forward`` whose dense operand is a boundary buffer still in its exchange format
    (``CommBufferForQuantization``: packed bytes, per-row parameters, ``*_row_code``).  Equal,
    bit for bit, to dequantising first."""
    _, col, value = src.csr()
    if value is None:
        raise RuntimeError("Input mismatch: the sparse matrix has no values")
    if out.size(0) < src.sparse_size(0):
        raise RuntimeError("Input mismatch: out has fewer rows than the sparse matrix")
    _spmm_quantized(src.get_plan(), value, packed, params, row_code, out, bits, accumulate, src.sparse_size(1), col)
    return None


def SPMM_backward_quantized(src: SparseTensor, packed: torch.Tensor, params: torch.Tensor, row_code: torch.Tensor,
                            out: torch.Tensor, bits: int, accumulate: bool = True):
    """``out += src.T @ dequantize(packed, params)``: the transposed counterpart."""
    value_T = src.storage.value_T()
    if value_T is None:
        raise RuntimeError("Input mismatch: the sparse matrix has no values")
    if out.size(0) < src.sparse_size(1):
        raise RuntimeError("Input mismatch: out has fewer rows than the sparse matrix has columns")
    _spmm_quantized(src.get_plan_for_transpose(), value_T, packed, params, row_code, out, bits, accumulate,
                    src.sparse_size(0), src.storage.row_T())
    return out, None
