"""Drop-in for the reference's native module ``computation_ops``.

``spmm``: self_benchmark/a64fx/model/ops/src/spmm.h:3-6, spmm.cpp:327-507, bound at
ops.cpp:23.  Same name, positional order, dtypes and ``(out, None)`` return; ``out`` is
accumulated into in place and returned as the same tensor.

Boundary-buffer codec (ops.cpp:12-18): ``quantize_tensor`` / ``dequantize_tensor`` and
``*_for_all_procs`` with the signatures of the SVE build (quantization_arm.h:5-8, the one
the reference's Python calls, quantizer.py:17, :44, :83-90), ``quantize_tensor_v1`` /
``dequantize_tensor_v1`` (quantization_x86.h:7-8).  All operands are GPU tensors.
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
    # the reference reads mat[col[e]] unchecked (spmm.cpp:38-39); a bad column here would be a GPU memory fault, so
    # the column array is range-checked on the device the first time it is seen (remembered per tensor)
    _lib.check_index(col, mat.size(0), what="col")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_spmm_csr_f32(_lib.ptr(rowptr), _lib.ptr(col), _lib.ptr(value), _lib.ptr(mat),
                                                  _lib.ptr(out), sparse_rows, mat.size(1), _lib.current_stream(dev)))
    return out, None


# ---------------------------------------------------------------- boundary-buffer codec

_PACKED_RANGE_CACHE = {}


def _packed_range(work_range_per_proc: torch.Tensor, bits: int, device) -> Tuple[torch.Tensor, torch.Tensor, int]:
    """Device copies of the per-rank row prefix and of the packed-row prefix derived from it
    (divide_work_v1, quantization_arm.cpp:21-31), cached per range tensor.  The cache entry
    keeps the range tensor alive, so its address cannot be handed to another tensor while the
    entry exists; an in-place change bumps ``_version``."""
    key = (work_range_per_proc.data_ptr(), work_range_per_proc._version, int(work_range_per_proc.numel()), bits,
           str(device))
    hit = _PACKED_RANGE_CACHE.get(key)
    if hit is None:
        host = work_range_per_proc.detach().to("cpu", torch.int64)
        _require(host.dim() == 1 and host.numel() >= 2, "work range must hold num_procs + 1 entries")
        _require(bool((host[1:] >= host[:-1]).all()) and int(host[0]) == 0, "work range must be a prefix sum from 0")
        epb = 8 // bits
        packed = torch.zeros_like(host)
        packed[1:] = torch.cumsum((host[1:] - host[:-1] + epb - 1) // epb, 0)
        hit = (host.to(device, torch.int32), packed.to(device, torch.int32), int(packed[-1]), int(host[-1]),
               work_range_per_proc)
        if len(_PACKED_RANGE_CACHE) > 64:
            _PACKED_RANGE_CACHE.clear()
        _PACKED_RANGE_CACHE[key] = hit
    return hit[:4]


def _check_codec_operands(data_fp32, data_int8, params, bits, params_cols):
    _require(bits in (2, 4, 8), "bits must be 2, 4 or 8")
    _require_hip(data_fp32, "fp32 buffer")
    dev = data_fp32.device
    _require_hip(data_int8, "packed buffer", dev)
    _require_hip(params, "quantisation parameters", dev)
    _require(data_fp32.dtype == torch.float32 and data_fp32.dim() == 2 and data_fp32.is_contiguous(),
             "fp32 buffer must be contiguous float32 2-D")
    _require(data_int8.dtype == torch.uint8 and data_int8.is_contiguous(), "packed buffer must be contiguous uint8")
    _require(params.dtype == torch.float32 and params.is_contiguous() and params.dim() == 2
             and params.size(0) >= data_fp32.size(0) and params.size(1) == params_cols,
             f"parameters must be contiguous float32 [rows, {params_cols}]")
    return dev


def quantize_tensor_for_all_procs(input: torch.Tensor, output: torch.Tensor, quantized_params: torch.Tensor,
                                  work_range_per_proc: torch.Tensor, num_procs: int, bits: int) -> None:
    """Row-packed quantisation of a boundary buffer, every rank's segment on its own
    (quantization_arm.cpp:364-435).  ``quantized_params`` [rows, 2] receives (zero_point,
    scale) per row.  The reference packs 2 bits whatever ``bits`` says (:380-381); here
    ``bits`` is honoured (2, 4 or 8)."""
    dev = _check_codec_operands(input, output, quantized_params, bits, 2)
    _require(work_range_per_proc.numel() == num_procs + 1, "work range must hold num_procs + 1 entries")
    rows_d, packed_d, packed_rows, rows = _packed_range(work_range_per_proc, bits, dev)
    _require(rows == input.size(0), "work range does not cover the buffer's rows")
    _require(output.numel() >= packed_rows * input.size(1), "packed buffer too small")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_quantize_segments_f32(
            _lib.ptr(input), _lib.ptr(output), _lib.ptr(quantized_params), _lib.ptr(rows_d), _lib.ptr(packed_d),
            num_procs, rows, packed_rows, input.size(1), bits, _lib.current_stream(dev)))


def gather_quantize_for_all_procs(src: torch.Tensor, index: torch.Tensor, output: torch.Tensor,
                                  quantized_params: torch.Tensor, work_range_per_proc: torch.Tensor, num_procs: int,
                                  bits: int) -> None:
    """``quantize_tensor_for_all_procs(src[index], output, ...)`` in one pass (aggregator.py:51 then
    communicator.py:281-311): the raw boundary rows are quantised as they are gathered, same bytes and parameters,
    without the gathered fp32 rows being written."""
    _require(bits in (2, 4, 8), "bits must be 2, 4 or 8")
    _require_hip(src, "source rows")
    dev = src.device
    for t, name in ((index, "index"), (output, "packed buffer"), (quantized_params, "quantisation parameters")):
        _require_hip(t, name, dev)
    rows = index.numel()
    _require(src.dtype == torch.float32 and src.dim() == 2 and src.is_contiguous(),
             "source rows must be contiguous float32 2-D")
    _require(index.dtype == torch.int64 and index.is_contiguous(), "index must be contiguous int64")
    _require(output.dtype == torch.uint8 and output.is_contiguous(), "packed buffer must be contiguous uint8")
    _require(quantized_params.dtype == torch.float32 and quantized_params.is_contiguous()
             and quantized_params.dim() == 2 and quantized_params.size(0) >= rows and quantized_params.size(1) == 2,
             "parameters must be contiguous float32 [rows, 2]")
    _require(work_range_per_proc.numel() == num_procs + 1, "work range must hold num_procs + 1 entries")
    rows_d, packed_d, packed_rows, covered = _packed_range(work_range_per_proc, bits, dev)
    _require(covered == rows, "work range does not cover the index list")
    _require(output.numel() >= packed_rows * src.size(1), "packed buffer too small")
    _lib.check_index(index, src.size(0), what="boundary row list (idx_nodes_send_to_others)")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_gather_quantize_segments_f32(
            _lib.ptr(src), src.size(0), _lib.ptr(index), _lib.ptr(output), _lib.ptr(quantized_params), _lib.ptr(rows_d),
            _lib.ptr(packed_d), num_procs, rows, packed_rows, src.size(1), bits, _lib.current_stream(dev)))


def spmm_quantize_for_all_procs(rowptr: torch.Tensor, col: torch.Tensor, value: torch.Tensor, mat: torch.Tensor,
                                output: torch.Tensor, quantized_params: torch.Tensor,
                                work_range_per_proc: torch.Tensor, num_procs: int, bits: int) -> bool:
    """``quantize_tensor_for_all_procs(A @ mat, output, ...)`` in one pass: the rows of the product are quantised out
    of the registers they were summed in, bytes and parameters equal to the two calls' (aggregator.py:44-49 then
    communicator.py:281-311).  ``rowptr`` / ``col`` int64 and ``value`` float32 are A's CSR arrays.  Returns False,
    with nothing done, for operands the one-pass kernel does not take (width no multiple of 4 or above 512, rows of
    ``mat`` off 16-byte boundaries, a matrix without stored elements): the caller then runs the two calls."""
    _require(bits in (2, 4, 8), "bits must be 2, 4 or 8")
    for t, name in ((rowptr, "rowptr"), (col, "col"), (value, "value"), (mat, "dense operand"), (output, "packed buffer"),
                    (quantized_params, "quantisation parameters")):
        _require_hip(t, name, mat.device if mat.is_cuda else None)
    dev = mat.device
    rows = rowptr.numel() - 1
    feat = mat.size(1) if mat.dim() == 2 else -1
    _require(rowptr.dtype == torch.int64 and col.dtype == torch.int64 and value.dtype == torch.float32
             and rowptr.is_contiguous() and col.is_contiguous() and value.is_contiguous()
             and value.numel() == col.numel(), "CSR arrays must be contiguous int64 / int64 / float32")
    _require(mat.dtype == torch.float32 and mat.dim() == 2 and mat.stride(1) == 1 and mat.stride(0) >= feat,
             "dense operand must be float32 2-D with contiguous rows")
    _require(output.dtype == torch.uint8 and output.is_contiguous(), "packed buffer must be contiguous uint8")
    _require(quantized_params.dtype == torch.float32 and quantized_params.is_contiguous()
             and quantized_params.dim() == 2 and quantized_params.size(0) >= rows and quantized_params.size(1) == 2,
             "parameters must be contiguous float32 [rows, 2]")
    _require(work_range_per_proc.numel() == num_procs + 1, "work range must hold num_procs + 1 entries")
    rows_d, packed_d, packed_rows, covered = _packed_range(work_range_per_proc, bits, dev)
    _require(covered == rows, "work range does not cover the product's rows")
    _require(output.numel() >= packed_rows * feat, "packed buffer too small")
    if (feat % 4 != 0 or feat > 512 or mat.stride(0) % 4 != 0 or mat.data_ptr() % 16 != 0 or output.data_ptr() % 4 != 0
            or col.numel() == 0 or rows == 0):
        return False
    _lib.check_index(col, mat.size(0), what="column indices of the sparse matrix")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_spmm_csr_quantize_segments_f32(
            _lib.ptr(rowptr), _lib.ptr(col), _lib.ptr(value), _lib.ptr(mat), mat.stride(0), _lib.ptr(output),
            _lib.ptr(quantized_params), _lib.ptr(rows_d), _lib.ptr(packed_d), num_procs, rows, packed_rows, feat, bits,
            _lib.current_stream(dev)))
    return True


def dequantize_tensor_for_all_procs(input: torch.Tensor, output: torch.Tensor, dequantized_params: torch.Tensor,
                                    work_range_per_proc: torch.Tensor, num_procs: int, bits: int) -> None:
    """Inverse of ``quantize_tensor_for_all_procs`` (quantization_arm.cpp:437-479):
    ``output = q * scale + zero_point`` with one rounding."""
    dev = _check_codec_operands(output, input, dequantized_params, bits, 2)
    _require(work_range_per_proc.numel() == num_procs + 1, "work range must hold num_procs + 1 entries")
    rows_d, packed_d, packed_rows, rows = _packed_range(work_range_per_proc, bits, dev)
    _require(rows == output.size(0), "work range does not cover the buffer's rows")
    _require(input.numel() >= packed_rows * output.size(1), "packed buffer too small")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_dequantize_segments_f32(
            _lib.ptr(input), _lib.ptr(dequantized_params), _lib.ptr(output), _lib.ptr(rows_d), _lib.ptr(packed_d),
            num_procs, rows, packed_rows, output.size(1), bits, _lib.current_stream(dev)))


_ONE_SEGMENT = {}


def _one_segment(rows: int) -> torch.Tensor:
    """The [0, rows] work range of a buffer that is one segment; one tensor per height, so that the device copies
    derived from it (``_packed_range``) are found again on the next call."""
    hit = _ONE_SEGMENT.get(rows)
    if hit is None:
        if len(_ONE_SEGMENT) >= 16:
            _ONE_SEGMENT.clear()
        hit = _ONE_SEGMENT[rows] = torch.tensor([0, rows], dtype=torch.int32)
    return hit


def quantize_tensor(input: torch.Tensor, output: torch.Tensor, quantized_params: torch.Tensor, bits: int) -> None:
    """The whole buffer as one segment (quantization_arm.cpp:302-331)."""
    quantize_tensor_for_all_procs(input, output, quantized_params, _one_segment(input.size(0)), 1, bits)


def dequantize_tensor(input: torch.Tensor, output: torch.Tensor, dequantized_params: torch.Tensor, bits: int) -> None:
    """quantization_arm.cpp:333-362."""
    dequantize_tensor_for_all_procs(input, output, dequantized_params, _one_segment(output.size(0)), 1, bits)


def _raise_on_bad_width(flag: torch.Tensor) -> None:
    if int(flag.item()) != 0:  # the reference prints "Error: unsupported num_bits" and goes on
        raise RuntimeError("Input mismatch: a row's bit width is not 2, 4 or 8")


def quantize_tensor_v1(input: torch.Tensor, output: torch.Tensor, quantized_nodes_feat_range: torch.Tensor,
                       quantized_params: torch.Tensor) -> None:
    """Feature-packed quantisation with a width per row (quantization_x86.cpp:164-243):
    ``quantized_params`` [rows, 3] holds the width in column 0 and receives (zero_point,
    scale) in columns 1-2; row i owns bytes ``range[i]..range[i+1]`` of ``output``.
    Synchronises (the width check is read back)."""
    _require_hip(input, "fp32 buffer")
    dev = input.device
    for t, name in ((output, "packed buffer"), (quantized_nodes_feat_range, "feature range"),
                    (quantized_params, "quantisation parameters")):
        _require_hip(t, name, dev)
    _require(input.dtype == torch.float32 and input.dim() == 2 and input.is_contiguous(),
             "fp32 buffer must be contiguous float32 2-D")
    _require(output.dtype == torch.uint8 and output.is_contiguous(), "packed buffer must be contiguous uint8")
    _require(quantized_nodes_feat_range.dtype == torch.int64 and quantized_nodes_feat_range.is_contiguous()
             and quantized_nodes_feat_range.numel() == input.size(0) + 1, "feature range must be int64 [rows + 1]")
    _require(quantized_params.dtype == torch.float32 and quantized_params.is_contiguous()
             and tuple(quantized_params.shape) == (input.size(0), 3), "parameters must be contiguous float32 [rows, 3]")
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_quantize_mixed_f32(
            _lib.ptr(input), _lib.ptr(output), _lib.ptr(quantized_nodes_feat_range), _lib.ptr(quantized_params),
            input.size(0), input.size(1), _lib.ptr(flag), _lib.current_stream(dev)))
    _raise_on_bad_width(flag)


def dequantize_tensor_v1(input: torch.Tensor, output: torch.Tensor, quantized_nodes_feat_range: torch.Tensor,
                         quantized_params: torch.Tensor) -> None:
    """quantization_x86.cpp:245-305."""
    _require_hip(output, "fp32 buffer")
    dev = output.device
    for t, name in ((input, "packed buffer"), (quantized_nodes_feat_range, "feature range"),
                    (quantized_params, "quantisation parameters")):
        _require_hip(t, name, dev)
    _require(output.dtype == torch.float32 and output.dim() == 2 and output.is_contiguous(),
             "fp32 buffer must be contiguous float32 2-D")
    _require(input.dtype == torch.uint8 and input.is_contiguous(), "packed buffer must be contiguous uint8")
    _require(quantized_nodes_feat_range.dtype == torch.int64 and quantized_nodes_feat_range.is_contiguous()
             and quantized_nodes_feat_range.numel() == output.size(0) + 1, "feature range must be int64 [rows + 1]")
    _require(quantized_params.dtype == torch.float32 and quantized_params.is_contiguous()
             and tuple(quantized_params.shape) == (output.size(0), 3), "parameters must be contiguous float32 [rows, 3]")
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().gnnagg_dequantize_mixed_f32(
            _lib.ptr(input), _lib.ptr(quantized_nodes_feat_range), _lib.ptr(quantized_params), _lib.ptr(output),
            output.size(0), output.size(1), _lib.ptr(flag), _lib.current_stream(dev)))
    _raise_on_bad_width(flag)
