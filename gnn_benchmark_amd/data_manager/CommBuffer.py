"""Send / receive boundary buffers, allocated once at the widest layer and re-shaped per
layer.  Reference: self_benchmark/a64fx/data_manager/CommBuffer.py:4-25."""
import torch

from .CommSplits import CommSplits


class CommBuffer(object):
    def __init__(self, comm_splits: CommSplits, feat_len: int, bits: int, device=None) -> None:
        size_send_buf = (sum(comm_splits.send_splits), feat_len)
        size_recv_buf = (sum(comm_splits.recv_splits), feat_len)
        self.send_buf = torch.zeros(size_send_buf, dtype=torch.float32, device=device)
        self.recv_buf = torch.zeros(size_recv_buf, dtype=torch.float32, device=device)
        self.send_buf_fp16 = None
        self.recv_buf_fp16 = None
        if bits == 16:
            self.send_buf_fp16 = torch.zeros(size_send_buf, dtype=torch.bfloat16, device=device)
            self.recv_buf_fp16 = torch.zeros(size_recv_buf, dtype=torch.bfloat16, device=device)

    def resize_buffer(self, comm_splits: CommSplits, feat_len: int, bits: int) -> None:
        size_send_buf = (sum(comm_splits.send_splits), feat_len)
        size_recv_buf = (sum(comm_splits.recv_splits), feat_len)
        self.send_buf.resize_(size_send_buf)
        self.recv_buf.resize_(size_recv_buf)
        if bits == 16 and self.send_buf_fp16 is not None and self.recv_buf_fp16 is not None:
            self.send_buf_fp16.resize_(size_send_buf)
            self.recv_buf_fp16.resize_(size_recv_buf)
