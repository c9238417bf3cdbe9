"""TEST INFRASTRUCTURE -- ctypes front end of ``liboracle_spmm.so`` (numpy in/out).

The arithmetic lives in ``oracle/spmm_oracle.c``; every function there cites the
reference lines it restates.  ``load_reference_op()`` returns the reference's own
compiled ``computation_ops`` module when ``oracle/_ref`` holds one.
"""
import ctypes
import glob
import importlib.util
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force: bool = False) -> str:
    """Compile the C restatement with gcc (used by ``__graft_entry__.build``)."""
    path = os.path.join(_HERE, "liboracle_spmm.so")
    if force and os.path.exists(path):
        os.remove(path)
    subprocess.check_call(["make", "-C", _HERE, "liboracle_spmm.so"], stdout=subprocess.DEVNULL)
    return path


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle_spmm.so")
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        i64p = ctypes.POINTER(ctypes.c_int64)
        i32p = ctypes.POINTER(ctypes.c_int32)
        f32p = ctypes.POINTER(ctypes.c_float)
        lib.oracle_divide_work.argtypes = [i32p, ctypes.c_int32, ctypes.c_int32]
        lib.oracle_divide_work.restype = None
        lib.oracle_distribute_work_for_row.argtypes = [i64p, f32p, ctypes.c_int64, ctypes.c_int32, i32p]
        lib.oracle_distribute_work_for_row.restype = None
        lib.oracle_spmm_f32.argtypes = [i64p, i64p, f32p, f32p, f32p, ctypes.c_int64, ctypes.c_int64, i32p,
                                        ctypes.c_int32]
        lib.oracle_spmm_f32.restype = ctypes.c_int
        lib.oracle_max_threads.restype = ctypes.c_int
        lib.oracle_fma_rows_f32.argtypes = [f32p, f32p, f32p, f32p, ctypes.c_int64, ctypes.c_int64]
        lib.oracle_fma_rows_f32.restype = None
        _LIB = lib
    return _LIB


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def fma_rows(q: np.ndarray, scale: np.ndarray, zero_point: np.ndarray) -> np.ndarray:
    """``fmaf(q[r, j], scale[r], zero_point[r])`` for every element, one rounding each."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    zero_point = np.ascontiguousarray(zero_point, dtype=np.float32)
    rows, feat = q.shape
    assert scale.shape == (rows,) and zero_point.shape == (rows,)
    out = np.empty_like(q)
    _lib().oracle_fma_rows_f32(_p(q, ctypes.c_float), _p(scale, ctypes.c_float), _p(zero_point, ctypes.c_float),
                               _p(out, ctypes.c_float), rows, feat)
    return out


def max_threads() -> int:
    return int(_lib().oracle_max_threads())


def divide_work(total_work: int, num_threads: int) -> np.ndarray:
    out = np.zeros(num_threads + 1, dtype=np.int32)
    _lib().oracle_divide_work(_p(out, ctypes.c_int32), int(total_work), int(num_threads))
    return out


def distribute_work_for_row(rowptr: np.ndarray, value: np.ndarray, num_threads: int) -> np.ndarray:
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int64)
    value = np.ascontiguousarray(value, dtype=np.float32)
    out = np.zeros(num_threads + 1, dtype=np.int32)
    _lib().oracle_distribute_work_for_row(_p(rowptr, ctypes.c_int64), _p(value, ctypes.c_float),
                                          rowptr.shape[0] - 1, int(num_threads), _p(out, ctypes.c_int32))
    return out


def spmm(rowptr, col, value, mat, out, row_split=None, num_threads: int = 1) -> np.ndarray:
    """``out += A @ mat`` in place (fp32 FMA chain in CSR order); returns ``out``."""
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int64)
    col = np.ascontiguousarray(col, dtype=np.int64)
    value = np.ascontiguousarray(value, dtype=np.float32)
    mat = np.ascontiguousarray(mat, dtype=np.float32)
    assert out.dtype == np.float32 and out.flags.c_contiguous and out.ndim == 2
    assert mat.ndim == 2 and out.shape[1] == mat.shape[1]
    rows = rowptr.shape[0] - 1
    assert out.shape[0] >= rows
    if col.size:
        assert 0 <= int(col.min()) and int(col.max()) < mat.shape[0], "column index out of range"
    rs = None
    if row_split is not None:
        row_split = np.ascontiguousarray(row_split, dtype=np.int32)
        assert row_split.shape[0] == num_threads + 1
        rs = _p(row_split, ctypes.c_int32)
    rc = _lib().oracle_spmm_f32(_p(rowptr, ctypes.c_int64), _p(col, ctypes.c_int64), _p(value, ctypes.c_float),
                                _p(mat, ctypes.c_float), _p(out, ctypes.c_float), rows, mat.shape[1], rs,
                                int(num_threads))
    if rc != 0:
        raise ValueError("oracle_spmm_f32 rejected its arguments")
    return out


def spmm_transposed(rowptr, col, value, grad, out, num_cols: int, num_threads: int = 1) -> np.ndarray:
    """``out += A.T @ grad`` through the transposed CSR, as SPMM_backward does
    (model/ops/spmm_kernel.py:71-90: the same kernel on colptr/row_T/value_T)."""
    colptr, row_t, value_t = csr_transpose(rowptr, col, value, num_cols)
    return spmm(colptr, row_t, value_t, grad, out, None, num_threads)


def csr_transpose(rowptr, col, value, num_cols: int):
    """(colptr, row_T, value_T): entries grouped by column, rows ascending inside a
    column (stable counting sort) -- the layout torch_sparse's storage hands to
    model/ops/spmm_kernel.py:76-78."""
    rowptr = np.asarray(rowptr, dtype=np.int64)
    col = np.asarray(col, dtype=np.int64)
    value = np.asarray(value, dtype=np.float32)
    rows = rowptr.shape[0] - 1
    row = np.repeat(np.arange(rows, dtype=np.int64), np.diff(rowptr))
    perm = np.argsort(col, kind="stable")
    colptr = np.zeros(num_cols + 1, dtype=np.int64)
    np.cumsum(np.bincount(col, minlength=num_cols), out=colptr[1:])
    return colptr, row[perm], value[perm]


def cpu_has_avx512() -> bool:
    try:
        with open("/proc/cpuinfo") as f:
            txt = f.read()
    except OSError:
        return False
    return all(flag in txt for flag in ("avx512f", "avx512bw", "avx512dq", "avx512vl", "avx512cd"))


def load_reference_op():
    """The reference's own native module built by oracle/build_ref.sh (under the module name
    ``reference_computation_ops``, so that it cannot be mistaken for, or handed out in place of, the product's
    ``computation_ops``: pybind11 keeps one module object per module name in a process), or None."""
    hits = glob.glob(os.path.join(_HERE, "_ref", "reference_computation_ops*.so"))
    if not hits or not cpu_has_avx512():
        return None
    import torch  # noqa: F401  (the module links against libtorch)
    spec = importlib.util.spec_from_file_location("reference_computation_ops", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    if not hasattr(mod, "quantize_tensor"):  # the reference binds its quantisation kernels beside spmm (ops.cpp:11-40)
        raise RuntimeError(f"{hits[0]} did not load as the reference's module")
    return mod
