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

from .sparse_tensor import SparseTensor


def _as_f32(value: torch.Tensor, other: torch.Tensor) -> torch.Tensor:
    # reference: value = value.to(other.dtype) (spmm_kernel.py:59-60)
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
