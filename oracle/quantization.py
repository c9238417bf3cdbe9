"""TEST INFRASTRUCTURE -- CPU oracle of the boundary-buffer codec (int2 / int4 / int8).

numpy restatement of the reference's quantisation kernels.  Two layouts exist there:

* ROW-PACKED, per destination rank (the live path of the trainer, int2):
  self_benchmark/a64fx/model/ops/src/quantization_arm.cpp:78-218 (``quantize_tensor_kernel``),
  :220-300 (``dequantize_tensor_kernel``), :364-479 (``*_for_all_procs``); the same packing
  rule for any ``8 % bits == 0`` in quantization_x86.cpp:17-98 / :100-162.  ``8/bits``
  consecutive rows of one rank's segment share one byte per feature column: row k of a
  group sits at bit ``(8/bits - k - 1) * bits``.  Each segment starts a new group, so the
  packed buffer has ``sum_p ceil(rows_p / (8/bits))`` rows of ``F`` bytes.  Parameters per
  row: ``zero_point = min(row)``, ``scale = (max(row) - min(row)) / (2^bits - 1)``,
  ``scale = 1`` when that is 0 (quantization_arm.cpp:104-111), stored as ``[rows, 2]``
  fp32 ``(zero_point, scale)``.  Quantise: ``rint((x - zero_point) / scale)`` to nearest
  even (``svrintn`` :165-168, ``_MM_FROUND_TO_NEAREST_INT`` quantization_x86.cpp:66);
  dequantise: ``q * scale + zero_point`` as ONE fused multiply-add (``svmla`` :263-266).
  The parameters travel as bf16 (communicator.py:297-303): ``params_over_the_wire``.

* FEATURE-PACKED with a bit width per row ("mixed bits", ``*_v1``):
  quantization_x86.cpp:164-243 / :245-305.  ``8/bits`` consecutive features of one row share
  a byte, same shift rule; row i owns bytes ``range[i]..range[i+1]`` with ``range`` from
  ``get_quantized_nodes_feat_range`` (quantizer.py:69-77); parameters ``[rows, 3]`` fp32
  ``(bits, zero_point, scale)``.

Pinning:
* ``quantize_mixed`` / ``dequantize_mixed`` / ``get_quantized_nodes_feat_range``: the
  reference's golden bytes and ranges, tests/test_quantizer.py:29-56, :58-84, :87-114.
* ``quantize_rows`` / ``dequantize_rows`` with given parameters: bit-for-bit against the
  reference's compiled x86 ``quantize_tensor`` / ``dequantize_tensor`` (oracle/_ref) and
  the vectors committed from it (tests/golden/quantization_reference_op_vectors.npz); the
  shift rule is the one the golden bytes above fix.
* The per-segment restart and the in-kernel parameter rule of ``*_for_all_procs`` exist
  only in the SVE source, which cannot be built on x86: PARITY UNPINNED at that level; they
  are pinned by composition (segment p of ``quantize_segments`` == ``quantize_rows`` of
  that segment alone, parameters == the ``*_v1`` rule that the golden vectors fix) and by
  brute force on tiny inputs.
* ``get_splits_for_comm_quantized_data``: tests/test_quantizer.py:10-27.
"""
import numpy as np

from . import spmm as _c


def elems_per_byte(bits: int) -> int:
    if bits not in (1, 2, 4, 8):
        raise ValueError("8 % bits must be 0")  # TORCH_CHECK(8 % bits == 0), quantization_x86.cpp:22
    return 8 // bits


def get_quantized_splits(num_comm_nodes: int, bits: int) -> int:
    """quantizer.py:94-95: packed rows one rank's segment occupies."""
    return -(-int(num_comm_nodes) // elems_per_byte(bits))


def segment_ranges(splits, bits: int):
    """CommBuffer.py:37-43: fp32-row prefix per rank, and the packed-row prefix that
    divide_work_v1 derives from it (quantization_arm.cpp:21-31)."""
    splits = np.asarray(splits, dtype=np.int64)
    rows = np.concatenate(([0], np.cumsum(splits))).astype(np.int32)
    packed = np.concatenate(([0], np.cumsum([get_quantized_splits(s, bits) for s in splits]))).astype(np.int32)
    return rows, packed


def row_params(x: np.ndarray, bits: int) -> np.ndarray:
    """quantization_arm.cpp:90-111: per-row (zero_point, scale) in fp32."""
    x = np.asarray(x, dtype=np.float32)
    if x.shape[0] == 0:
        return np.zeros((0, 2), dtype=np.float32)
    lo = x.min(axis=1)
    hi = x.max(axis=1)
    scale = ((hi - lo).astype(np.float32) / np.float32((1 << bits) - 1)).astype(np.float32)
    scale[scale == 0] = np.float32(1.0)
    return np.stack([lo, scale], axis=1).astype(np.float32)


def _quantize_values(x: np.ndarray, zero_point: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """rint((x - zp) / scale), fp32 arithmetic, ties to even, as int32 (two's complement
    bits are what the shift/or/truncate below works on)."""
    q = np.rint(((x - zero_point[:, None]).astype(np.float32) / scale[:, None]).astype(np.float32))
    return q.astype(np.int64).astype(np.int32)


def quantize_rows(x: np.ndarray, zero_point: np.ndarray, scale: np.ndarray, bits: int) -> np.ndarray:
    """quantization_x86.cpp:17-98 (one segment, parameters given): ``[ceil(rows/epb), F]`` bytes."""
    x = np.asarray(x, dtype=np.float32)
    rows, feat = x.shape
    epb = elems_per_byte(bits)
    q = _quantize_values(x, np.asarray(zero_point, np.float32), np.asarray(scale, np.float32)).astype(np.uint32)
    packed = np.zeros((-(-rows // epb), feat), dtype=np.uint32)
    for k in range(epb):
        part = q[k::epb]
        packed[:part.shape[0]] |= part << np.uint32((epb - k - 1) * bits)
    return (packed & 0xFF).astype(np.uint8)


def dequantize_rows(packed: np.ndarray, zero_point: np.ndarray, scale: np.ndarray, rows: int, bits: int) -> np.ndarray:
    """quantization_x86.cpp:100-162 / quantization_arm.cpp:220-300: q * scale + zero_point, fused."""
    packed = np.asarray(packed, dtype=np.uint8)
    feat = packed.shape[1]
    epb = elems_per_byte(bits)
    mask = (1 << bits) - 1
    q = np.empty((rows, feat), dtype=np.float32)
    for k in range(epb):
        idx = np.arange(k, rows, epb)
        q[idx] = ((packed[:idx.shape[0]] >> ((epb - k - 1) * bits)) & mask).astype(np.float32)
    return _c.fma_rows(q, np.asarray(scale, np.float32), np.asarray(zero_point, np.float32))


def quantize_segments(x: np.ndarray, splits, bits: int):
    """quantize_tensor_for_all_procs (quantization_arm.cpp:364-435): every rank's segment is
    packed on its own.  Returns (packed ``[sum ceil(rows_p/epb), F]`` uint8, params ``[rows, 2]``)."""
    x = np.asarray(x, dtype=np.float32)
    rows, packed_rows = segment_ranges(splits, bits)
    params = row_params(x, bits)
    out = np.zeros((int(packed_rows[-1]), x.shape[1]), dtype=np.uint8)
    for p in range(len(splits)):
        a, b = int(rows[p]), int(rows[p + 1])
        if b > a:
            out[packed_rows[p]:packed_rows[p + 1]] = quantize_rows(x[a:b], params[a:b, 0], params[a:b, 1], bits)
    return out, params


def dequantize_segments(packed: np.ndarray, params: np.ndarray, splits, bits: int) -> np.ndarray:
    """dequantize_tensor_for_all_procs (quantization_arm.cpp:437-479)."""
    rows, packed_rows = segment_ranges(splits, bits)
    out = np.empty((int(rows[-1]), packed.shape[1]), dtype=np.float32)
    for p in range(len(splits)):
        a, b = int(rows[p]), int(rows[p + 1])
        if b > a:
            out[a:b] = dequantize_rows(packed[packed_rows[p]:packed_rows[p + 1]], params[a:b, 0], params[a:b, 1], b - a,
                                       bits)
    return out


def to_bf16_and_back(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (round to nearest even) -> fp32, what ``tensor_bf16.copy_(tensor_fp32)`` and the
    copy back do to the parameters on the wire (communicator.py:297-303)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(nan, 0x7FC00000, rounded)  # c10::BFloat16's scalar conversion; NaN payloads are not pinned
    return (rounded & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(np.shape(x))


def params_over_the_wire(params: np.ndarray) -> np.ndarray:
    return to_bf16_and_back(params)


# ---------------------------------------------------------------- mixed bits (feature-packed)

def get_quantized_nodes_feat_range(num_nodes: int, feat_len: int, nodes_num_bits) -> np.ndarray:
    """quantizer.py:69-77: byte offsets of every row's packed features, ``[num_nodes + 1]`` int64."""
    bits = np.asarray(nodes_num_bits, dtype=np.float32)
    lens = np.ceil(bits * np.float32(feat_len) / np.float32(8.0))
    out = np.zeros(num_nodes + 1, dtype=np.int64)
    out[1:] = np.cumsum(lens[:num_nodes]).astype(np.int64)
    return out


def quantize_mixed(x: np.ndarray, nodes_num_bits, feat_range=None):
    """quantize_tensor_v1 (quantization_x86.cpp:164-243).  Returns (bytes uint8 ``[range[-1]]``,
    params ``[rows, 3]`` = (bits, zero_point, scale))."""
    x = np.asarray(x, dtype=np.float32)
    rows, feat = x.shape
    bits_f = np.asarray(nodes_num_bits, dtype=np.float32)
    if feat_range is None:
        feat_range = get_quantized_nodes_feat_range(rows, feat, bits_f)
    out = np.zeros(int(feat_range[-1]), dtype=np.uint8)
    params = np.zeros((rows, 3), dtype=np.float32)
    for i in range(rows):
        bits = int(bits_f[i])
        epb = elems_per_byte(bits)
        lo, hi = x[i].min(), x[i].max()
        scale = np.float32(np.float32(hi - lo) / np.float32((1 << bits) - 1))
        if scale == 0:
            scale = np.float32(1.0)
        params[i] = (bits, lo, scale)
        q = np.rint((x[i] - lo).astype(np.float32) / scale).astype(np.int64).astype(np.int32).astype(np.uint32)
        nbytes = -(-feat // epb)
        padded = np.zeros(nbytes * epb, dtype=np.uint32)
        padded[:feat] = q
        byte = np.zeros(nbytes, dtype=np.uint32)
        for k in range(epb):
            byte |= padded[k::epb] << np.uint32((epb - k - 1) * bits)
        out[feat_range[i]:feat_range[i] + nbytes] = (byte & 0xFF).astype(np.uint8)
    return out, params


def dequantize_mixed(data: np.ndarray, params: np.ndarray, feat_len: int, feat_range=None) -> np.ndarray:
    """dequantize_tensor_v1 (quantization_x86.cpp:245-305)."""
    params = np.asarray(params, dtype=np.float32)
    rows = params.shape[0]
    if feat_range is None:
        feat_range = get_quantized_nodes_feat_range(rows, feat_len, params[:, 0])
    out = np.empty((rows, feat_len), dtype=np.float32)
    for i in range(rows):
        bits = int(params[i, 0])
        epb = elems_per_byte(bits)
        mask = (1 << bits) - 1
        raw = np.asarray(data[feat_range[i]:feat_range[i + 1]], dtype=np.uint8)
        q = np.stack([(raw >> ((epb - k - 1) * bits)) & mask for k in range(epb)], axis=1).reshape(-1)[:feat_len]
        # ``val * scale + zero_point`` (:287-288) and the 8-bit kernel's mul + add
        # (quantization_kernel_x86.h:58-61) both come out of the reference's build as one fused
        # multiply-add (gcc contracts them), like the SVE kernels' svmla.
        out[i] = _c.fma_rows(q.astype(np.float32)[None, :], params[i, 2:3], params[i, 1:2])[0]
    return out


def get_splits_for_comm_quantized_data(recv_splits, send_splits, dequantized_nodes_feat_range,
                                       quantized_nodes_feat_range):
    """communicator.py:327-381: byte counts per rank of a mixed-bits exchange."""
    def per_rank(splits, feat_range):
        begin = np.concatenate(([0], np.cumsum(np.asarray(splits, dtype=np.int64))))
        return [int(feat_range[begin[r + 1]] - feat_range[begin[r]]) for r in range(len(splits))]

    return (per_rank(recv_splits, np.asarray(dequantized_nodes_feat_range)),
            per_rank(send_splits, np.asarray(quantized_nodes_feat_range)))
