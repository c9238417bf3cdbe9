"""Per-rank row counts of the boundary exchange.

Reference: self_benchmark/a64fx/data_manager/CommSplits.py:7-19.  Only the fp32/bf16
exchange is in scope; the int2 split lists of the reference (:11-19) belong to the
quantised MPI exchange and are not built (``bits == 2`` raises).
"""


class CommSplits(object):
    def __init__(self, recv_splits: list, send_splits: list, world_size: int, bits: int) -> None:
        if bits not in (32, 16):
            raise NotImplementedError("quantised boundary exchange (bits=%r) is outside this build" % (bits,))
        if len(recv_splits) != world_size or len(send_splits) != world_size:
            raise ValueError("split lists must have one entry per rank")
        self.recv_splits = [int(x) for x in recv_splits]
        self.send_splits = [int(x) for x in send_splits]
