"""Send / receive boundary buffers of one partition, allocated once at the widest layer and
re-shaped per layer (``resize_`` keeps the storage).  Counterpart of
self_benchmark/a64fx/data_manager/CommBuffer.py:4-25; the int2 buffers of :27-49 belong to
the quantised exchange and are not built."""
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
