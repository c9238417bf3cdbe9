"""Drop-in for the reference's native module ``computation_ops`` (only ``spmm``; the
quantisation ops of that module serve the MPI exchange, which this build leaves out).

Reference: self_benchmark/a64fx/model/ops/src/spmm.h:3-6, spmm.cpp:327-507, bound at
ops.cpp:23.  Same name, positional order, dtypes and ``(out, None)`` return; ``out`` is
accumulated into in place and returned as the same tensor.
"""
from typing import Optional, Tuple

import torch

from . import _lib


def _require(cond: bool, what: str) -> None:
    # the reference raises c10::Error("Input mismatch") through CHECK_INPUT (utils.h:13)
    if not cond:
        raise RuntimeError(f"Input mismatch: {what}")


def _require_hip(t: torch.Tensor, name: str, device=None) -> None:
    # counterpart of CHECK_CPU (utils.h:12): here every operand must live on the GPU
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU (HIP) tensor; there is no CPU path")
    if device is not None and t.device != device:
        raise RuntimeError(f"{name} is on {t.device}, expected {device}")


def spmm(rowptr: torch.Tensor, col: torch.Tensor, value: Optional[torch.Tensor], mat: torch.Tensor,
         out: torch.Tensor, sparse_rows: int, parallel_row_split: Optional[torch.Tensor] = None,
         parallel_col_split: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, None]:
    """``out[m,:] += sum_e value[e] * mat[col[e],:]`` for the rows of a CSR matrix.

    ``parallel_row_split`` / ``parallel_col_split`` are the reference's per-thread CPU
    work ranges (spmm.cpp:394-395); they carry no meaning on a GPU and are ignored.

    Differences from the reference, all on the side of raising instead of silently
    going on: a missing ``value`` raises (the reference dereferences an empty optional,
    spmm.cpp:377); non-fp32 ``mat``/``value`` raise (the reference prints a message and
    returns ``out`` untouched, spmm.cpp:498-503).
    """
    _require_hip(rowptr, "rowptr")
    dev = rowptr.device
    _require_hip(col, "col", dev)
    _require(value is not None, "value is required")
    _require_hip(value, "value", dev)
    _require_hip(mat, "mat", dev)
    _require_hip(out, "out", dev)
    _require(rowptr.dim() == 1, "rowptr must be 1-D")
    _require(col.dim() == 1, "col must be 1-D")
    _require(value.dim() == 1, "value must be 1-D")
    _require(value.size(0) == col.size(0), "value and col differ in length")
    _require(mat.dim() == 2, "mat must be 2-D")
    _require(rowptr.dtype == torch.int64 and col.dtype == torch.int64, "rowptr/col must be int64")
    _require(mat.dtype == torch.float32 and value.dtype == torch.float32, "mat/value must be float32")
    _require(out.dtype == torch.float32 and out.dim() == 2 and out.is_contiguous(), "out must be contiguous float32 2-D")
    sparse_rows = int(sparse_rows)
    _require(rowptr.size(0) >= sparse_rows + 1, "rowptr shorter than sparse_rows + 1")
    _require(out.size(0) >= sparse_rows and out.size(1) == mat.size(1), "out shape does not match")
    mat = mat.contiguous()
    rowptr = rowptr.contiguous()
    col = col.contiguous()
    value = value.contiguous()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_spmm_csr_f32(_lib.ptr(rowptr), _lib.ptr(col), _lib.ptr(value), _lib.ptr(mat),
                                                  _lib.ptr(out), sparse_rows, mat.size(1), _lib.current_stream(dev)))
    return out, None
