"""A small CSR container with the accessors the aggregation path reads from the
reference's (patched) ``torch_sparse.SparseTensor``.

Reference call sites: construction ``SparseTensor(row=, col=, value=, sparse_sizes=)`` at
self_benchmark/a64fx/data_manager/DataProcessor.py:104-116, :458-502; ``src.csr()``,
``src.storage.colptr()/row_T()/value_T()``, ``src.get/set_work_range[_for_transpose]()``
at model/ops/spmm_kernel.py:46-57, :76-87; ``sparse_size`` at
model/layers/aggregator.py:67, :167.  torch_sparse itself is third party and not in the
reference tree; what is restated here is its documented layout: entries ordered by
(row, col), repeated entries kept, ``rowptr`` by counting.

On a HIP device the format conversions run in libgnnagg; on CPU tensors they run as
plain torch host code (setup-time only -- SpMM itself has no CPU path).
"""
import ctypes
from typing import Optional, Tuple

import torch

from . import _lib


# Tuning values new plans are created with: a dict with any of the keys of ``_lib.PlanOptions`` (long_row_threshold,
# block_row_threshold, rows_per_group, short_rows_per_group, lanes_per_row, loads_per_lane); None or a missing key
# = the library's default.  Results never depend on them.  Tests and sweeps set this; ``SpmmPlan(options=...)``
# overrides it for one plan.
PLAN_OPTIONS: Optional[dict] = None


class SpmmPlan:
    """Cached GPU schedule of one CSR matrix (the counterpart of the per-matrix CPU work
    range the reference caches, model/ops/spmm_kernel.py:48-57)."""

    def __init__(self, rowptr: torch.Tensor, col: torch.Tensor, rows: int, cols: int, options: Optional[dict] = None):
        if not rowptr.is_cuda:
            raise RuntimeError("SpMM plans exist only for matrices on a GPU (HIP) device")
        self.device = rowptr.device
        self.rows, self.cols, self.nnz = int(rows), int(cols), int(col.numel())
        handle = ctypes.c_void_p()
        options = PLAN_OPTIONS if options is None else options
        opt = _lib.PlanOptions(**options) if options else None
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().gnnagg_plan_create_ex(_lib.ptr(rowptr), _lib.ptr(col), self.rows, self.cols, self.nnz,
                                                        None if opt is None else ctypes.byref(opt),
                                                        _lib.current_stream(self.device), ctypes.byref(handle)))
        self._handle = handle

    def info(self) -> dict:
        buf = (ctypes.c_int64 * 12)()
        _lib.check(_lib.lib().gnnagg_plan_info(self._handle, buf))
        keys = ("rows", "cols", "nnz", "huge_rows", "huge_thresh", "empty_rows", "max_row_len", "rows_per_group",
                "short_rows", "short_rows_per_group", "long_rows", "long_thresh")
        return dict(zip(keys, [int(x) for x in buf]))

    @property
    def max_row_len(self) -> int:
        """Stored elements of the matrix's longest row (fixed when the plan was built)."""
        hit = getattr(self, "_max_row_len", None)
        if hit is None:
            hit = self._max_row_len = self.info()["max_row_len"]
        return hit

    def profile(self, enable: bool = True) -> None:
        """Record HIP events around the next SpMM calls (benchmark use)."""
        _lib.check(_lib.lib().gnnagg_plan_profile(self._handle, 1 if enable else 0))

    def profile_read(self):
        """(dominant-kernel ms, whole-call ms) of the most recent profiled call; synchronises."""
        buf = (ctypes.c_double * 2)()
        _lib.check(_lib.lib().gnnagg_plan_profile_read(self._handle, buf))
        return float(buf[0]), float(buf[1])

    def spmm(self, value: torch.Tensor, mat: torch.Tensor, out: torch.Tensor, accumulate: bool = True) -> torch.Tensor:
        """``out (+)= A @ mat``.  ``mat`` and ``out`` may be column blocks of wider row-major
        tensors (unit stride along the features, any row stride): they are used in place."""
        if not (value.is_cuda and mat.is_cuda and out.is_cuda):
            raise RuntimeError("value, mat and out must be GPU (HIP) tensors; there is no CPU path")
        if torch.bfloat16 in (mat.dtype, out.dtype):
            return self._spmm_bf16(value, mat, out, accumulate)
        if value.dtype != torch.float32 or mat.dtype != torch.float32 or out.dtype != torch.float32:
            raise RuntimeError("Input mismatch: value/mat/out must be float32")
        if mat.dim() != 2 or out.dim() != 2 or not _rows_are_dense(out):
            raise RuntimeError("Input mismatch: mat/out must be 2-D and the rows of out contiguous")
        if value.numel() != self.nnz or mat.size(0) < self.cols or out.size(0) < self.rows or out.size(1) != mat.size(1):
            raise RuntimeError("Input mismatch: operand shapes do not match the planned matrix")
        if not _rows_are_dense(mat):
            mat = mat.contiguous()
        value = value.contiguous()
        feat = mat.size(1)
        with torch.cuda.device(self.device):
            if mat.is_contiguous() and out.is_contiguous():
                _lib.check(_lib.lib().gnnagg_plan_spmm_f32(self._handle, _lib.ptr(value), _lib.ptr(mat), _lib.ptr(out),
                                                           feat, 1 if accumulate else 0,
                                                           _lib.current_stream(self.device)))
            else:
                _lib.check(_lib.lib().gnnagg_plan_spmm_strided_f32(
                    self._handle, _lib.ptr(value), _lib.ptr(mat), _row_stride(mat), _lib.ptr(out), _row_stride(out),
                    feat, 1 if accumulate else 0, _lib.current_stream(self.device)))
        return out

    def spmm_two_sources(self, value: torch.Tensor, mat: torch.Tensor, mat2: torch.Tensor, out: torch.Tensor,
                         accumulate: bool = True) -> torch.Tensor:
        """``out (+)= A @ [mat ; mat2]`` with the dense operand in two arrays: column ``c`` reads row ``c`` of ``mat``
        for ``c < mat.size(0)`` and row ``c - mat.size(0)`` of ``mat2`` above.  All float32, rows contiguous (column
        blocks of wider tensors are read and written in place)."""
        tensors = (value, mat, mat2, out)
        if not all(t.is_cuda for t in tensors):
            raise RuntimeError("value, mat, mat2 and out must be GPU (HIP) tensors; there is no CPU path")
        if any(t.dtype != torch.float32 for t in tensors):
            raise RuntimeError("Input mismatch: value/mat/mat2/out must be float32")
        if not all(_rows_are_dense(t) for t in (mat, mat2, out)):
            raise RuntimeError("Input mismatch: mat/mat2/out must be 2-D with contiguous rows")
        feat = out.size(1)
        if (value.numel() != self.nnz or mat.size(0) + mat2.size(0) < self.cols or mat.size(0) > self.cols
                or out.size(0) < self.rows or mat.size(1) != feat or mat2.size(1) != feat):
            raise RuntimeError("Input mismatch: operand shapes do not match the planned matrix")
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().gnnagg_plan_spmm_two_sources_f32(
                self._handle, _lib.ptr(value.contiguous()), _lib.ptr(mat), _row_stride(mat), mat.size(0), _lib.ptr(mat2),
                _row_stride(mat2), _lib.ptr(out), _row_stride(out), feat, 1 if accumulate else 0,
                _lib.current_stream(self.device)))
        return out

    def spmm_dense_then(self, value: torch.Tensor, split: torch.Tensor, mat: torch.Tensor, second, out: torch.Tensor,
                        accumulate: bool = True) -> torch.Tensor:
        """``out (+)= A @ [mat ; second]`` where the rows of the second operand are still in an exchange format: the
        first ``split[r]`` stored elements of row r gather float32 rows of ``mat`` (columns below ``mat.size(0)``), the
        others rows of ``second`` -- a bfloat16 ``[rows, F]`` tensor, or a tuple ``(packed uint8 [packed rows, F],
        params float32 [rows, 2], row_code int32 [rows], bits)`` as ``SPMM_forward_quantized`` takes them."""
        if not all(t.is_cuda for t in (value, split, mat, out)):
            raise RuntimeError("value, split, mat and out must be GPU (HIP) tensors; there is no CPU path")
        feat = out.size(1) if out.dim() == 2 else -1
        if (value.dtype != torch.float32 or mat.dtype != torch.float32 or out.dtype != torch.float32
                or split.dtype != torch.int32 or not split.is_contiguous() or split.numel() != self.rows
                or not _rows_are_dense(mat) or not _rows_are_dense(out) or mat.size(1) != feat
                or value.numel() != self.nnz or out.size(0) < self.rows or mat.size(0) > self.cols):
            raise RuntimeError("Input mismatch: value/mat/out must be float32 with contiguous rows, split int32 [rows], "
                               "shapes matching the planned matrix")
        second_rows = self.cols - mat.size(0)
        L = _lib.lib()
        with torch.cuda.device(self.device):
            if isinstance(second, torch.Tensor):
                if (second.dtype != torch.bfloat16 or not second.is_cuda or not _rows_are_dense(second)
                        or second.size(0) < second_rows or second.size(1) != feat):
                    raise RuntimeError("Input mismatch: the second source must be bfloat16 [rows, F] with contiguous rows")
                _lib.check(L.gnnagg_plan_spmm_dense_then_bf16_f32(
                    self._handle, _lib.ptr(value.contiguous()), _lib.ptr(split), _lib.ptr(mat), _row_stride(mat),
                    mat.size(0), _lib.ptr(second), _row_stride(second), _lib.ptr(out), _row_stride(out), feat,
                    1 if accumulate else 0, _lib.current_stream(self.device)))
            else:
                packed, params, row_code, bits = second
                if (packed.dtype != torch.uint8 or not packed.is_contiguous() or packed.dim() != 2 or packed.size(1) != feat
                        or params.dtype != torch.float32 or not params.is_contiguous() or params.dim() != 2
                        or params.size(0) < second_rows or params.size(1) != 2 or row_code.dtype != torch.int32
                        or not row_code.is_contiguous() or row_code.numel() < second_rows
                        or not all(t.is_cuda for t in (packed, params, row_code))):
                    raise RuntimeError("Input mismatch: quantised second source needs uint8 [packed rows, F] bytes, "
                                       "float32 [rows, 2] parameters and int32 [rows] row codes on the GPU")
                _lib.check_index(row_code, packed.size(0), shift=3, what="row codes of the packed buffer")
                _lib.check(L.gnnagg_plan_spmm_dense_then_quantized_f32(
                    self._handle, _lib.ptr(value.contiguous()), _lib.ptr(split), _lib.ptr(mat), _row_stride(mat),
                    mat.size(0), _lib.ptr(packed), _lib.ptr(params), _lib.ptr(row_code), int(bits), _lib.ptr(out),
                    _row_stride(out), feat, 1 if accumulate else 0, _lib.current_stream(self.device)))
        return out

    def _spmm_bf16(self, value, mat, out, accumulate):
        """The product with bf16 rows on either side (the staging buffers of a 16-bit exchange): a bf16 ``mat`` is
        widened in the gather, a bf16 ``out`` receives the fp32 sums rounded to nearest even -- the same bits as the
        tensor copies around an fp32 product, without the copies."""
        ok = (torch.float32, torch.bfloat16)
        if value.dtype != torch.float32 or mat.dtype not in ok or out.dtype not in ok:
            raise RuntimeError("Input mismatch: value must be float32, mat/out float32 or bfloat16")
        if mat.dim() != 2 or out.dim() != 2 or not _rows_are_dense(out) or not _rows_are_dense(mat):
            raise RuntimeError("Input mismatch: mat/out must be 2-D with contiguous rows")
        if value.numel() != self.nnz or mat.size(0) < self.cols or out.size(0) < self.rows or out.size(1) != mat.size(1):
            raise RuntimeError("Input mismatch: operand shapes do not match the planned matrix")
        if accumulate and out.dtype == torch.bfloat16:
            raise RuntimeError("Input mismatch: a bfloat16 result is written, not accumulated onto")
        feat = mat.size(1)
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().gnnagg_plan_spmm_bf16_f32(
                self._handle, _lib.ptr(value.contiguous()), _lib.ptr(mat), 1 if mat.dtype == torch.bfloat16 else 0,
                _row_stride(mat), _lib.ptr(out), 1 if out.dtype == torch.bfloat16 else 0, _row_stride(out), feat,
                1 if accumulate else 0, _lib.current_stream(self.device)))
        return out

    def __del__(self):
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            try:
                _lib.lib().gnnagg_plan_destroy(h)
            except Exception:  # interpreter shutdown
                pass


def release_plans(device=None) -> None:
    """Free the device memory of the plans dropped so far on ``device`` (default: the current one).  A dropped plan
    only queues its memory, so that a destructor in the middle of a step never synchronises; the queue is emptied by
    the next plan creation on the device -- or here, at a moment the caller knows to be safe (this synchronises the
    device): the end of graph set-up, between epochs."""
    with torch.cuda.device(device):
        _lib.check(_lib.lib().gnnagg_plans_release())


def _rows_are_dense(t: torch.Tensor) -> bool:
    """2-D, unit stride along each row, rows not overlapping (a column block of a row-major tensor)."""
    return t.dim() == 2 and (t.size(1) <= 1 or t.stride(1) == 1) and (t.size(0) <= 1 or t.stride(0) >= t.size(1))


def _row_stride(t: torch.Tensor) -> int:
    return t.stride(0) if t.size(0) > 1 else t.size(1)


def _coo_to_csr_host(row, col, value, rows):
    # stable two-pass sort = order by (row, col), repeated pairs keep their input order
    p1 = torch.sort(col, stable=True).indices
    p2 = torch.sort(row[p1], stable=True).indices
    perm = p1[p2]
    rowptr = torch.zeros(rows + 1, dtype=torch.int64, device=row.device)
    rowptr[1:] = torch.cumsum(torch.bincount(row, minlength=rows), 0)
    return rowptr, col[perm].contiguous(), (None if value is None else value[perm].contiguous())


def _coo_to_csr(row, col, value, rows, cols):
    nnz = int(row.numel())
    if nnz:
        # checked on the device inside libgnnagg for GPU tensors
        if not row.is_cuda and (int(row.min()) < 0 or int(row.max()) >= rows or int(col.min()) < 0 or int(col.max()) >= cols):
            raise RuntimeError("Input mismatch: row/col index outside sparse_sizes")
    if not row.is_cuda:
        return _coo_to_csr_host(row, col, value, rows)
    dev = row.device
    rowptr = torch.empty(rows + 1, dtype=torch.int64, device=dev)
    col_out = torch.empty(nnz, dtype=torch.int64, device=dev)
    value_out = None if value is None else torch.empty(nnz, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_coo_to_csr(_lib.ptr(row), _lib.ptr(col), _lib.ptr(value), nnz, rows, cols,
                                                _lib.ptr(rowptr), _lib.ptr(col_out), _lib.ptr(value_out),
                                                _lib.current_stream(dev)))
    return rowptr, col_out, value_out


class _Storage:
    """``src.storage``: owns the CSR arrays and the lazily built transposed arrays."""

    def __init__(self, rowptr, col, value, sparse_sizes):
        self._rowptr, self._col, self._value = rowptr, col, value
        self._sparse_sizes = (int(sparse_sizes[0]), int(sparse_sizes[1]))
        self._colptr = self._row_T = self._value_T = None

    def rowptr(self):
        return self._rowptr

    def col(self):
        return self._col

    def value(self):
        return self._value

    def row(self):
        counts = self._rowptr[1:] - self._rowptr[:-1]
        return torch.repeat_interleave(torch.arange(self._sparse_sizes[0], device=self._col.device), counts)

    def _build_transposed(self):
        rows, cols = self._sparse_sizes
        nnz = int(self._col.numel())
        if not self._col.is_cuda:
            perm = torch.sort(self._col, stable=True).indices
            self._colptr = torch.zeros(cols + 1, dtype=torch.int64)
            self._colptr[1:] = torch.cumsum(torch.bincount(self._col, minlength=cols), 0)
            self._row_T = self.row()[perm].contiguous()
            self._value_T = None if self._value is None else self._value[perm].contiguous()
            return
        dev = self._col.device
        colptr = torch.empty(cols + 1, dtype=torch.int64, device=dev)
        row_t = torch.empty(nnz, dtype=torch.int64, device=dev)
        value_t = None if self._value is None else torch.empty(nnz, dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            _lib.check(_lib.lib().gnnagg_csr_transpose(_lib.ptr(self._rowptr), _lib.ptr(self._col), _lib.ptr(self._value),
                                                       rows, cols, nnz, _lib.ptr(colptr), _lib.ptr(row_t),
                                                       _lib.ptr(value_t), _lib.current_stream(dev)))
        self._colptr, self._row_T, self._value_T = colptr, row_t, value_t

    def colptr(self):
        if self._colptr is None:
            self._build_transposed()
        return self._colptr

    def row_T(self):
        if self._row_T is None:
            self._build_transposed()
        return self._row_T

    def value_T(self):
        if self._colptr is None:
            self._build_transposed()
        return self._value_T


class SparseTensor:
    def __init__(self, row: Optional[torch.Tensor] = None, rowptr: Optional[torch.Tensor] = None,
                 col: Optional[torch.Tensor] = None, value: Optional[torch.Tensor] = None,
                 sparse_sizes: Optional[Tuple[int, int]] = None, is_sorted: bool = False):
        if col is None:
            raise ValueError("col is required")
        if sparse_sizes is None:
            raise ValueError("sparse_sizes is required")
        rows, cols = int(sparse_sizes[0]), int(sparse_sizes[1])
        col = col.to(torch.int64).contiguous()
        if value is not None:
            value = value.to(torch.float32).contiguous()
            if value.numel() != col.numel():
                raise RuntimeError("Input mismatch: value and col differ in length")
        if rowptr is not None and (is_sorted or row is None):
            rowptr = rowptr.to(torch.int64).contiguous()
            if rowptr.numel() != rows + 1:
                raise RuntimeError("Input mismatch: rowptr length is not rows + 1")
        else:
            if row is None:
                raise ValueError("row or rowptr is required")
            row = row.to(torch.int64).contiguous()
            if row.numel() != col.numel():
                raise RuntimeError("Input mismatch: row and col differ in length")
            rowptr, col, value = _coo_to_csr(row, col, value, rows, cols)
        self.storage = _Storage(rowptr, col, value, (rows, cols))
        empty = torch.empty(0, dtype=torch.int32)
        self._work_range = (empty, empty)
        self._work_range_T = (empty, empty)
        self._plan = None
        self._plan_T = None

    # ---- construction helpers
    @classmethod
    def from_scipy(cls, mat) -> "SparseTensor":
        m = mat.tocsr()
        m.sort_indices()
        return cls(rowptr=torch.from_numpy(m.indptr.astype("int64")), col=torch.from_numpy(m.indices.astype("int64")),
                   value=torch.from_numpy(m.data.astype("float32")), sparse_sizes=m.shape, is_sorted=True)

    def to(self, device) -> "SparseTensor":
        s = self.storage
        out = SparseTensor(rowptr=s._rowptr.to(device), col=s._col.to(device),
                           value=None if s._value is None else s._value.to(device),
                           sparse_sizes=s._sparse_sizes, is_sorted=True)
        return out

    def cuda(self) -> "SparseTensor":
        return self.to("cuda")

    def cpu(self) -> "SparseTensor":
        return self.to("cpu")

    # ---- accessors used by the aggregation path
    def csr(self):
        return self.storage._rowptr, self.storage._col, self.storage._value

    def coo(self):
        return self.storage.row(), self.storage._col, self.storage._value

    def sparse_sizes(self):
        return self.storage._sparse_sizes

    def sparse_size(self, dim: int) -> int:
        return self.storage._sparse_sizes[dim]

    def nnz(self) -> int:
        return int(self.storage._col.numel())

    @property
    def device(self):
        return self.storage._col.device

    def requires_grad_(self, flag: bool = True):
        return self  # no gradient w.r.t. the values is ever produced on this path

    def to_dense(self) -> torch.Tensor:
        """Dense [rows, cols] with repeated entries SUMMED (what the SpMM computes)."""
        row, col, value = self.coo()
        rows, cols = self.sparse_sizes()
        dense = torch.zeros(rows, cols, dtype=torch.float32, device=col.device)
        v = torch.ones(col.numel(), dtype=torch.float32, device=col.device) if value is None else value
        dense.index_put_((row, col), v, accumulate=True)
        return dense

    # ---- cached schedules.  The *_work_range accessors keep the reference's names
    # (model/ops/spmm_kernel.py:48,57,80,87); what is cached on a GPU is the plan.
    def get_work_range(self):
        return self._work_range

    def set_work_range(self, row_splits, col_splits):
        self._work_range = (row_splits, col_splits)

    def get_work_range_for_transpose(self):
        return self._work_range_T

    def set_work_range_for_transpose(self, row_splits, col_splits):
        self._work_range_T = (row_splits, col_splits)

    def get_plan(self) -> SpmmPlan:
        if self._plan is None:
            rowptr, col, _ = self.csr()
            self._plan = SpmmPlan(rowptr, col, self.sparse_size(0), self.sparse_size(1))
        return self._plan

    def get_plan_for_transpose(self) -> SpmmPlan:
        if self._plan_T is None:
            s = self.storage
            self._plan_T = SpmmPlan(s.colptr(), s.row_T(), self.sparse_size(1), self.sparse_size(0))
        return self._plan_T


def side_by_side(left: SparseTensor, right: SparseTensor, transposed: bool = False) -> SparseTensor:
    """``[left | right]`` (``transposed``: ``[left^T | right^T]``) as one CSR: every row holds its elements of
    ``left`` in their order, then its elements of ``right`` in theirs with the column moved up by the columns of
    ``left``.  A product with it over the two dense operands stacked is, row by row, the FMA chain of the product
    with ``left`` continued by the one with ``right``.  Built once per pair and kept on ``left``."""
    cache = left.__dict__.setdefault("_side_by_side", {})
    key = (id(right), bool(transposed))
    hit = cache.get(key)
    if hit is None:
        parts = []
        for m in (left, right):
            row, col, value = m.coo()
            if value is None:
                raise RuntimeError("Input mismatch: the sparse matrix has no values")
            parts.append((col, row, value) if transposed else (row, col, value))
        rows = left.sparse_size(1 if transposed else 0)
        if right.sparse_size(1 if transposed else 0) != rows:
            raise RuntimeError("Input mismatch: the two matrices differ in their number of rows")
        left_cols = left.sparse_size(0 if transposed else 1)
        right_cols = right.sparse_size(0 if transposed else 1)
        # (row, column) order with repeated pairs in input order: inside a row all of left's elements come before
        # right's (their columns are smaller), each part in the order of its own (transposed) CSR
        merged = SparseTensor(row=torch.cat([parts[0][0], parts[1][0]]),
                              col=torch.cat([parts[0][1], parts[1][1] + left_cols]),
                              value=torch.cat([parts[0][2], parts[1][2]]), sparse_sizes=(rows, left_cols + right_cols))
        merged.first_source_rows = left_cols
        # per row: how many of its leading stored elements come from `left`
        ptr = left.storage.colptr() if transposed else left.csr()[0]
        merged.first_counts = (ptr[1:] - ptr[:-1]).to(torch.int32).contiguous()
        if len(cache) >= 4:
            cache.clear()
        hit = cache[key] = (right, merged)   # holding `right` keeps its id its own
    return hit[1]
