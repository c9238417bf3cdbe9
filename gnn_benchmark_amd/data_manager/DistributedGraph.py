"""Attribute bags the aggregator reads.  Reference:
self_benchmark/a64fx/data_manager/DistributedGraph.py:8-33, :35-59.

One attribute is added to both: ``exchange``, the callable that stands in for the
boundary all-to-all (model/layers/aggregator.py:54-61, :156-163).  ``None`` means a
single-rank world: the aggregator then skips pre-/post-aggregation exactly like the
reference does for ``world_size == 1`` (aggregator.py:47, :100).
"""
from typing import Callable, Optional

from torch import Tensor

from ..sparse_tensor import SparseTensor
from .CommBuffer import CommBuffer
from .CommSplits import CommSplits


class DistributedGraph(object):
    def __init__(self, local_adj_t: SparseTensor, remote_adj_t: SparseTensor, idx_nodes_send_to_others: Tensor,
                 num_nodes_send_to_others: list, num_nodes_recv_from_others: list, in_degrees: Tensor,
                 comm_splits: CommSplits, comm_buf: CommBuffer, comm_buf_for_quantization=None,
                 exchange: Optional[Callable] = None) -> None:
        self.local_adj_t = local_adj_t
        self.remote_adj_t = remote_adj_t
        self.idx_nodes_send_to_others = idx_nodes_send_to_others
        self.num_nodes_send_to_others = num_nodes_send_to_others
        self.num_nodes_recv_from_others = num_nodes_recv_from_others
        self.in_degrees = in_degrees
        self.comm_splits = comm_splits
        self.comm_buf = comm_buf
        self.comm_buf_for_quantization = comm_buf_for_quantization
        self.exchange = exchange
        self._send_scatter_adj_t = None

    def send_scatter_adj_t(self) -> SparseTensor:
        """[N_local, S] selection matrix with a 1 at (idx_nodes_send_to_others[i], i): the
        backward ``index_add_`` (aggregator.py:197-199) as a deterministic SpMM."""
        if self._send_scatter_adj_t is None:
            import torch

            idx = self.idx_nodes_send_to_others
            s = int(idx.numel())
            self._send_scatter_adj_t = SparseTensor(
                row=idx, col=torch.arange(s, dtype=torch.int64, device=idx.device),
                value=torch.ones(s, dtype=torch.float32, device=idx.device),
                sparse_sizes=(self.local_adj_t.sparse_size(0), s))
        return self._send_scatter_adj_t


class DistributedGraphForPre(object):
    def __init__(self, local_adj_t: SparseTensor, adj_t_pre_post_aggr_from: SparseTensor,
                 adj_t_pre_post_aggr_to: SparseTensor, pre_post_aggr_from_splits: list, pre_post_aggr_to_splits: list,
                 in_degrees: Tensor, comm_splits: CommSplits, comm_buf: CommBuffer, comm_buf_for_quantization=None,
                 exchange: Optional[Callable] = None) -> None:
        self.local_adj_t = local_adj_t
        self.adj_t_pre_post_aggr_from = adj_t_pre_post_aggr_from
        self.adj_t_pre_post_aggr_to = adj_t_pre_post_aggr_to
        self.pre_post_aggr_from_splits = pre_post_aggr_from_splits
        self.pre_post_aggr_to_splits = pre_post_aggr_to_splits
        self.in_degrees = in_degrees
        self.comm_splits = comm_splits
        self.comm_buf = comm_buf
        self.comm_buf_for_quantization = comm_buf_for_quantization
        self.exchange = exchange
