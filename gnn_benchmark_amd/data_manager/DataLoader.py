"""Builds the per-partition graph objects the aggregator consumes.

Reference: self_benchmark/a64fx/data_manager/DataLoader.py:12-61 (the .npy file
contract), :64-122 (``get_distributed_graph``), :125-194
(``get_distributed_graph_for_pre_aggressive``).  Same positional arguments; the
keyword-only arguments are what replaces the reference's process group:

``halo_id_exchange`` / ``graph_exchange``  stand-ins for the setup-time all_to_all calls
    (see DataProcessor); ``None`` behaves like a single-rank world.
``exchange``  the stand-in for the per-layer boundary all-to-all, stored on the graph.
``device``    where the CSR matrices and boundary buffers are placed (the edge lists are
    moved there first, so the maps themselves are built on that device).
"""
import os
from typing import Callable, Optional

import numpy as np
import torch

from .CommBuffer import CommBuffer, CommBufferForQuantization
from .CommSplits import CommSplits
from .DataProcessor import DataProcessor, DataProcessorForPreAggresive
from .DistributedGraph import DistributedGraph, DistributedGraphForPre


def load_graph_structures(input_dir, graph_name, rank):
    """Reads one partition's files: ``p{rank:03d}-{name}_nodes.npy`` int64 [N,2],
    ``..._local_edges.npy`` int64 [2,E_l] (src,dst localised), ``..._remote_edges.npy``
    int64 [2,E_r] (src global, dst localised), ``begin_node_on_each_partition.txt``.
    Reference: DataLoader.py:12-40."""
    prefix = os.path.join(input_dir, "p{:0>3d}-{}".format(rank, graph_name))
    local_nodes_list = np.load(prefix + "_nodes.npy")
    node_idx_begin = local_nodes_list[0][0]
    node_idx_end = local_nodes_list[local_nodes_list.shape[0] - 1][0]
    num_local_nodes = int(node_idx_end - node_idx_begin + 1)
    local_edges_list = np.load(prefix + "_local_edges.npy")
    remote_edges_list = np.load(prefix + "_remote_edges.npy")
    nodes_range_on_each_subgraph = np.loadtxt(os.path.join(input_dir, "begin_node_on_each_partition.txt"),
                                              dtype=np.int64, delimiter=" ")
    return (torch.from_numpy(local_nodes_list), torch.from_numpy(local_edges_list),
            torch.from_numpy(remote_edges_list), torch.from_numpy(nodes_range_on_each_subgraph), num_local_nodes)


def _to_device(edges, device):
    if device is None:
        return edges
    if isinstance(edges, (list, tuple)):
        return [e.to(device) for e in edges]
    return edges.to(device)


def _quantization_buffers(comm_splits, max_feat_len, bits, device):
    # DataLoader.py:105-108, :168-171 (there for bits == 2 only)
    return CommBufferForQuantization(comm_splits, max_feat_len, bits, device=device) if bits in (2, 4, 8) else None


def get_distributed_graph(local_edges_list, remote_edges_list, local_nodes_list, nodes_range_on_each_subgraph,
                          num_local_nodes: int, max_feat_len: int, world_size: int, bits: int, *,
                          halo_id_exchange: Optional[Callable] = None, exchange: Optional[Callable] = None,
                          exchange_quantized: Optional[Callable] = None, exchange_bf16: Optional[Callable] = None,
                          device=None) -> DistributedGraph:
    local_edges_list = _to_device(local_edges_list, device)
    remote_edges_list = _to_device(remote_edges_list, device)
    in_degrees = DataProcessor.get_in_degrees(local_edges_list, remote_edges_list, num_local_nodes)
    remote_edges_list = DataProcessor.sort_remote_edges_list_based_on_remote_nodes(remote_edges_list)
    (remote_nodes_list, range_of_remote_nodes_on_local_graph, remote_nodes_num_from_each_subgraph) = (
        DataProcessor.obtain_remote_nodes_list(remote_edges_list, num_local_nodes, nodes_range_on_each_subgraph,
                                               world_size))
    (local_nodes_required_by_other, num_local_nodes_required_by_other) = (
        DataProcessor.obtain_local_nodes_required_by_other(
            local_nodes_list, remote_nodes_list, range_of_remote_nodes_on_local_graph,
            remote_nodes_num_from_each_subgraph, world_size, halo_id_exchange=halo_id_exchange))
    local_adj_t, remote_adj_t = DataProcessor.transform_edge_index_to_sparse_tensor(
        local_edges_list, remote_edges_list, num_local_nodes, int(remote_nodes_list.size(0)))
    comm_splits = CommSplits(remote_nodes_num_from_each_subgraph.tolist(), num_local_nodes_required_by_other.tolist(),
                             world_size, bits)
    comm_buf = CommBuffer(comm_splits, max_feat_len, bits, device=local_adj_t.device)
    return DistributedGraph(local_adj_t, remote_adj_t, local_nodes_required_by_other,
                            num_local_nodes_required_by_other.tolist(), remote_nodes_num_from_each_subgraph.tolist(),
                            in_degrees, comm_splits, comm_buf,
                            _quantization_buffers(comm_splits, max_feat_len, bits, local_adj_t.device),
                            exchange=exchange, exchange_quantized=exchange_quantized, exchange_bf16=exchange_bf16)


def get_distributed_graph_for_pre_aggressive(local_edges_list, remote_edges_list, nodes_range_on_each_subgraph,
                                             num_local_nodes, max_feat_len, rank, world_size, bits, *,
                                             graph_exchange: Optional[Callable] = None,
                                             exchange: Optional[Callable] = None,
                                             exchange_quantized: Optional[Callable] = None,
                                             exchange_bf16: Optional[Callable] = None,
                                             device=None) -> DistributedGraphForPre:
    local_edges_list = _to_device(local_edges_list, device)
    remote_edges_list = _to_device(remote_edges_list, device)
    in_degrees = DataProcessor.get_in_degrees(local_edges_list, remote_edges_list, num_local_nodes)
    # the dst ids of the remote edges come localised; pre-aggregation needs them global
    # again (DataLoader.py:137-139)
    local_begin = int(nodes_range_on_each_subgraph[rank])
    remote_edges_list[1] += local_begin
    (from_list, to_list, begin_from, begin_to, from_splits, to_splits) = (
        DataProcessorForPreAggresive.divide_remote_edges_list(nodes_range_on_each_subgraph, remote_edges_list,
                                                              world_size, graph_exchange=graph_exchange))
    (local_adj_t, adj_t_pre_post_aggr_from, adj_t_pre_post_aggr_to) = (
        DataProcessorForPreAggresive.transform_edge_index_to_sparse_tensor(
            local_edges_list, from_list, to_list, begin_from, begin_to, num_local_nodes, local_begin))
    comm_splits = CommSplits(from_splits, to_splits, world_size, bits)
    comm_buf = CommBuffer(comm_splits, max_feat_len, bits, device=local_adj_t.device)
    return DistributedGraphForPre(local_adj_t, adj_t_pre_post_aggr_from, adj_t_pre_post_aggr_to, from_splits,
                                  to_splits, in_degrees, comm_splits, comm_buf,
                                  _quantization_buffers(comm_splits, max_feat_len, bits, local_adj_t.device),
                                  exchange=exchange, exchange_quantized=exchange_quantized, exchange_bf16=exchange_bf16)
