"""Send / receive boundary buffers of one partition, allocated once at the widest layer and
re-shaped per layer (``resize_`` keeps the storage).  Counterpart of
self_benchmark/a64fx/data_manager/CommBuffer.py:4-25 (fp32 / bf16 rows) and :27-49 (the
packed buffers, per-row parameters and per-rank work ranges of the quantised exchange)."""
import torch

from .CommSplits import CommSplits


def _shapes(comm_splits: CommSplits, feat_len: int):
    return (sum(comm_splits.send_splits), feat_len), (sum(comm_splits.recv_splits), feat_len)


class CommBuffer(object):
    def __init__(self, comm_splits: CommSplits, feat_len: int, bits: int, device=None) -> None:
        send_shape, recv_shape = _shapes(comm_splits, feat_len)
        self.send_buf = torch.zeros(send_shape, dtype=torch.float32, device=device)
        self.recv_buf = torch.zeros(recv_shape, dtype=torch.float32, device=device)
        # bf16 staging copies exist only when the exchange itself runs in bf16
        self.send_buf_fp16 = torch.zeros(send_shape, dtype=torch.bfloat16, device=device) if bits == 16 else None
        self.recv_buf_fp16 = torch.zeros(recv_shape, dtype=torch.bfloat16, device=device) if bits == 16 else None

    def resize_buffer(self, comm_splits: CommSplits, feat_len: int, bits: int) -> None:
        send_shape, recv_shape = _shapes(comm_splits, feat_len)
        for buf, shape in ((self.send_buf, send_shape), (self.recv_buf, recv_shape)):
            buf.resize_(shape)
        if bits == 16 and self.send_buf_fp16 is not None:
            self.send_buf_fp16.resize_(send_shape)
            self.recv_buf_fp16.resize_(recv_shape)


def _row_codes(splits, bits: int, device) -> torch.Tensor:
    """For every row of a boundary buffer: (packed row) * 8 + (position inside its byte group), with
    every rank's segment packed on its own -- what a consumer needs to read row i out of the packed
    bytes without unpacking the buffer."""
    per = 8 // bits
    codes, packed_begin = [], 0
    for rows in splits:
        local = torch.arange(int(rows), dtype=torch.int64)
        codes.append((packed_begin + local // per) * 8 + local % per)
        packed_begin += -(-int(rows) // per)
    out = torch.cat(codes) if codes else torch.zeros(0, dtype=torch.int64)
    out = out.to(torch.int32)
    return out.to(device) if device is not None else out


def _prefix(splits, device) -> torch.Tensor:
    out = torch.zeros(len(splits) + 1, dtype=torch.int32)
    out[1:] = torch.tensor(splits, dtype=torch.int32).cumsum(0)
    return out.to(device) if device is not None else out


class CommBufferForQuantization(object):
    """Packed data, (zero_point, scale) per row in fp32 and in the bf16 that travels, and the
    row prefix per peer rank for both directions (CommBuffer.py:27-49).  The reference builds
    these for ``bits == 2`` only; 4 and 8 use the same layout here."""

    def __init__(self, comm_splits: CommSplits, feat_len: int, bits: int, device=None) -> None:
        if bits not in (2, 4, 8):
            raise ValueError("quantised buffers exist for 2, 4 or 8 bits")
        self.bits = bits
        send_rows, recv_rows = sum(comm_splits.send_splits), sum(comm_splits.recv_splits)
        self.quantized_send_data_buf = torch.zeros((sum(comm_splits.send_splits_int2), feat_len), dtype=torch.uint8,
                                                   device=device)
        self.quantized_recv_data_buf = torch.zeros((sum(comm_splits.recv_splits_int2), feat_len), dtype=torch.uint8,
                                                   device=device)
        self.quantized_send_params_buf_fp32 = torch.zeros((send_rows, 2), dtype=torch.float32, device=device)
        self.quantized_recv_params_buf_fp32 = torch.zeros((recv_rows, 2), dtype=torch.float32, device=device)
        self.quantized_send_params_buf_bf16 = torch.zeros((send_rows, 2), dtype=torch.bfloat16, device=device)
        self.quantized_recv_params_buf_bf16 = torch.zeros((recv_rows, 2), dtype=torch.bfloat16, device=device)
        self.quantized_work_range_per_proc = _prefix(comm_splits.send_splits, device)
        self.dequantized_work_range_per_proc = _prefix(comm_splits.recv_splits, device)
        # not in the reference: where each fp32 row sits in the packed bytes, for aggregating
        # straight from them (spmm_kernel.SPMM_forward_quantized)
        self.send_row_code = _row_codes(comm_splits.send_splits, bits, device)
        self.recv_row_code = _row_codes(comm_splits.recv_splits, bits, device)

    def resize_buffer(self, comm_splits: CommSplits, feat_len: int, bits: int) -> None:
        if bits == self.bits:
            self.quantized_send_data_buf.resize_((sum(comm_splits.send_splits_int2), feat_len))
            self.quantized_recv_data_buf.resize_((sum(comm_splits.recv_splits_int2), feat_len))
