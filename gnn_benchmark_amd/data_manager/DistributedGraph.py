"""Attribute bags the aggregator reads: one per partition, holding the CSR matrices, the
split lists and the boundary buffers.  Field names and constructor order are the
reference's (self_benchmark/a64fx/data_manager/DistributedGraph.py:8-33, :35-59), because
``Aggregator`` and the layers address them by name.

Two fields are added to both: ``exchange``, the callable that stands in for the boundary
all-to-all (model/layers/aggregator.py:54-61, :156-163) -- ``None`` means a single-rank
world: the aggregator then skips pre-/post-aggregation exactly like the reference does for
``world_size == 1`` (aggregator.py:47, :100) -- and ``exchange_quantized``, its counterpart
for the packed bytes and per-row parameters of a quantised exchange
(communicator.py:231-325), and ``exchange_bf16`` for the bf16 staging copies of a 16-bit one
(communicator.py:111-137).
"""
from dataclasses import dataclass, field
from typing import Any, Callable, List, Optional

import torch

from ..sparse_tensor import SparseTensor
from .CommBuffer import CommBuffer
from .CommSplits import CommSplits


@dataclass
class DistributedGraph:
    """Raw-halo mode: boundary rows travel as they are."""
    local_adj_t: SparseTensor                  # [N, N]   row = dst, col = src
    remote_adj_t: SparseTensor                 # [N, Rv]  col = halo row in recv_buf
    idx_nodes_send_to_others: torch.Tensor     # [S] local rows gathered into send_buf
    num_nodes_send_to_others: List[int]
    num_nodes_recv_from_others: List[int]
    in_degrees: torch.Tensor                   # fp32 [N, 1]
    comm_splits: CommSplits
    comm_buf: CommBuffer
    comm_buf_for_quantization: Any = None      # CommBufferForQuantization for bits 2 / 4 / 8
    exchange: Optional[Callable] = None
    exchange_quantized: Optional[Callable] = None
    exchange_bf16: Optional[Callable] = None
    in_degrees_folded: bool = False            # the matrices' rows already carry 1 / in_degrees
    _scatter: Optional[SparseTensor] = field(default=None, repr=False)

    def send_scatter_adj_t(self) -> SparseTensor:
        """[N, S] selection matrix with a 1 at (idx_nodes_send_to_others[i], i): turns the
        backward ``index_add_`` (aggregator.py:197-199) into a deterministic SpMM."""
        if self._scatter is None:
            idx = self.idx_nodes_send_to_others
            count = int(idx.numel())
            self._scatter = SparseTensor(
                row=idx, col=torch.arange(count, dtype=torch.int64, device=idx.device),
                value=torch.ones(count, dtype=torch.float32, device=idx.device),
                sparse_sizes=(self.local_adj_t.sparse_size(0), count))
        return self._scatter


@dataclass
class DistributedGraphForPre:
    """Pre/post-aggregation mode: boundary rows travel partly summed."""
    local_adj_t: SparseTensor                  # [N, N]
    adj_t_pre_post_aggr_from: SparseTensor     # [N, Rv]  post-aggregation of received rows
    adj_t_pre_post_aggr_to: SparseTensor       # [S, N]   pre-aggregation into send_buf
    pre_post_aggr_from_splits: List[int]
    pre_post_aggr_to_splits: List[int]
    in_degrees: torch.Tensor
    comm_splits: CommSplits
    comm_buf: CommBuffer
    comm_buf_for_quantization: Any = None
    exchange: Optional[Callable] = None
    exchange_quantized: Optional[Callable] = None
    exchange_bf16: Optional[Callable] = None
    in_degrees_folded: bool = False
