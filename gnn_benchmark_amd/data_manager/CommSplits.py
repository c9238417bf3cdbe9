"""Per-rank row counts of the boundary exchange.

Reference: self_benchmark/a64fx/data_manager/CommSplits.py:7-19.  With a quantised
exchange (``bits`` 2 in the reference; 4 and 8 follow the same rule here) the lists
``recv_splits_int2`` / ``send_splits_int2`` hold the PACKED rows per rank:
``ceil(rows / (8 / bits))``, every rank's segment being packed on its own.
"""


class CommSplits(object):
    def __init__(self, recv_splits: list, send_splits: list, world_size: int, bits: int) -> None:
        if bits not in (32, 16, 8, 4, 2):
            raise NotImplementedError("boundary exchange with bits=%r is not defined" % (bits,))
        if len(recv_splits) != world_size or len(send_splits) != world_size:
            raise ValueError("split lists must have one entry per rank")
        self.recv_splits = [int(x) for x in recv_splits]
        self.send_splits = [int(x) for x in send_splits]
        if bits in (2, 4, 8):
            rows_per_byte = 8 // bits
            self.recv_splits_int2 = [-(-x // rows_per_byte) for x in self.recv_splits]
            self.send_splits_int2 = [-(-x // rows_per_byte) for x in self.send_splits]
