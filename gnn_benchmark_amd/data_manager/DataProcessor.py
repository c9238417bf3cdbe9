"""Index maps of one graph partition: in-degrees, halo renumbering, send lists, the
pre/post-aggregation edge split and the CSR matrices the aggregator multiplies with.

Same class / method names, argument meaning, in-place side effects and results as the
reference's self_benchmark/a64fx/data_manager/DataProcessor.py, but every per-edge
Python loop of the reference (:39-53, :238-246, :434-444) is a sort / unique / scan
formulation on whole tensors, so the maps can be built for 10^8 edges and on the GPU
(the tensors stay on whatever device the edge lists live on).  All index results are
int64 and bit-identical to the reference's.

Where the reference calls a setup-time collective (``dist.all_to_all`` at :77, :94,
``dist.all_to_all_single`` at :343, :372) these functions take the received lists from
a caller-supplied callable instead; no process group is needed.

Sorting.  The reference uses ``torch.argsort`` (tie order unspecified); a stable sort
is used here, which reproduces every known-answer vector of the reference's tests.  The
sort, unique and run-numbering steps go through ``device_ops``: libgnnagg's own radix-sort
and run kernels for GPU tensors, torch host ops of the same meaning for CPU tensors.
"""
from typing import Callable, List, Optional

import torch

from ..sparse_tensor import SparseTensor
from . import device_ops
from .device_ops import stable_argsort as _stable_argsort


def _as_i64(x, device=None) -> torch.Tensor:
    return torch.as_tensor(x, dtype=torch.int64, device=device)


class DataProcessor(object):
    def __init__(self) -> None:
        pass

    @staticmethod
    def get_in_degrees(local_edges_list, remote_edges_list, num_local_nodes):
        """fp32 [N,1] number of incoming edges (local + remote), at least 1.
        Reference: DataProcessor.py:12-18."""
        ld, rd = local_edges_list[1], remote_edges_list[1]
        degs = torch.bincount(ld, minlength=num_local_nodes) + torch.bincount(rd, minlength=num_local_nodes)
        return degs.to(torch.float32).clamp(min=1).unsqueeze(-1)

    @staticmethod
    def sort_remote_edges_list_based_on_remote_nodes(remote_edges_list):
        """Order the remote edges by remote src id; rows 0/1 of the argument are
        overwritten and the argument is returned.  Reference: DataProcessor.py:20-26."""
        row, col = remote_edges_list[0], remote_edges_list[1]
        order = _stable_argsort(row)
        remote_edges_list[0] = row[order]
        remote_edges_list[1] = col[order]
        return remote_edges_list

    @staticmethod
    def obtain_remote_nodes_list(remote_edges_list, num_local_nodes, num_nodes_on_each_subgraph, world_size):
        """Halo renumbering of the src-sorted remote edges.  Returns (halo global ids
        [Rv], per-rank halo ranges [W+1], per-rank halo counts [W]) and rewrites the
        src row IN PLACE to ``num_local_nodes + k`` (k = position of the id in the halo
        list).  Reference: DataProcessor.py:28-60."""
        src = remote_edges_list[0]
        dev = src.device
        begins = _as_i64(num_nodes_on_each_subgraph, dev)
        uniq, inverse, _ = device_ops.runs(src, want_counts=False)
        owner = torch.bucketize(uniq, begins[1:world_size + 1].contiguous(), right=True)
        counts = torch.bincount(owner, minlength=world_size)[:world_size].to(torch.int64)
        ranges = torch.zeros(world_size + 1, dtype=torch.int64, device=dev)
        ranges[1:] = torch.cumsum(counts, 0)
        src.copy_(inverse + num_local_nodes)
        return uniq.to(torch.int64), ranges, counts

    @staticmethod
    def obtain_local_nodes_required_by_other(local_nodes_list, remote_nodes_list, range_of_remote_nodes_on_local_graph,
                                             remote_nodes_num_from_each_subgraph, world_size,
                                             halo_id_exchange: Optional[Callable] = None):
        """Which local rows every other rank wants.  ``halo_id_exchange(send_lists)``
        stands in for the two all_to_all calls (DataProcessor.py:76-77, :93-94): it is
        given the per-rank slices of this rank's halo id list and returns the id lists
        the other ranks sent here.  Without it nothing is received (the reference's
        ``world_size == 1`` behaviour).  Returns (row indices [S] = received global ids
        minus this rank's first global id, counts [W]).  Reference: :62-98."""
        r = range_of_remote_nodes_on_local_graph
        send_nodes_list = [remote_nodes_list[int(r[i]):int(r[i + 1])] for i in range(world_size)]
        dev = remote_nodes_list.device
        if halo_id_exchange is not None and world_size != 1:
            recv_nodes_list = [_as_i64(x, dev) for x in halo_id_exchange(send_nodes_list)]
        else:
            recv_nodes_list = [torch.zeros(0, dtype=torch.int64, device=dev) for _ in range(world_size)]
        num_required = _as_i64([int(x.numel()) for x in recv_nodes_list], dev)
        local_node_idx_begin = local_nodes_list[0][0]
        required = torch.cat([x - local_node_idx_begin for x in recv_nodes_list], dim=0)
        return required, num_required

    @staticmethod
    def transform_edge_index_to_sparse_tensor(local_edges_list, remote_edges_list, num_local_nodes, num_remote_nodes):
        """local_adj_t = CSR(row=dst, col=src, 1, [N,N]); remote_adj_t = CSR(row=dst,
        col=src-N, 1, [N,Rv]).  Reference: DataProcessor.py:100-118."""
        dev = local_edges_list[1].device
        local_adj_t = SparseTensor(row=local_edges_list[1], col=local_edges_list[0],
                                   value=torch.ones(local_edges_list[1].shape[0], dtype=torch.float32, device=dev),
                                   sparse_sizes=(num_local_nodes, num_local_nodes))
        tmp_col = remote_edges_list[0] - num_local_nodes
        remote_adj_t = SparseTensor(row=remote_edges_list[1], col=tmp_col,
                                    value=torch.ones(remote_edges_list[1].shape[0], dtype=torch.float32, device=dev),
                                    sparse_sizes=(num_local_nodes, num_remote_nodes))
        return local_adj_t, remote_adj_t


class DataProcessorForPreAggresive(object):
    def __init__(self) -> None:
        pass

    @staticmethod
    def get_degrees(nodes_list):
        """{node id: occurrences}.  Reference: DataProcessor.py:125-131."""
        if nodes_list.is_cuda and nodes_list.numel():
            ordered = nodes_list[_stable_argsort(nodes_list)]
            uniq, _, counts = device_ops.runs(ordered, want_inverse=False)
        else:
            uniq, counts = torch.unique(nodes_list, return_counts=True)
        return dict(zip(uniq.tolist(), counts.tolist()))

    @staticmethod
    def _occurrences_per_entry(nodes: torch.Tensor) -> torch.Tensor:
        return device_ops.occurrences_per_entry(nodes)

    @staticmethod
    def decide_pre_or_post_aggr(src_in_remote_edges, dst_in_remote_edges, is_pre, is_post):
        """POST when out-degree(src) > in-degree(dst), else PRE, degrees counted inside
        the given subset.  Reference: DataProcessor.py:228-248."""
        if src_in_remote_edges.numel() == 0:
            return torch.zeros(0, dtype=torch.int64, device=src_in_remote_edges.device)
        out_deg = DataProcessorForPreAggresive._occurrences_per_entry(src_in_remote_edges)
        in_deg = DataProcessorForPreAggresive._occurrences_per_entry(dst_in_remote_edges)
        flags = torch.where(out_deg > in_deg, int(is_post), int(is_pre))
        return flags.to(torch.int64)

    @staticmethod
    def collect_edges_sent_to_other_subgraphs(src_in_remote_edges, dst_in_remote_edges, pre_aggr_edge_idx,
                                              post_aggr_edge_idx, remote_edges_sent_for_graph_exchange):
        """Appends the packed list told to the src-owning rank: PRE edges (src,dst) and
        one (s,s) per distinct src of a POST edge, ordered by the second component,
        stored as [firsts | seconds].  Reference: DataProcessor.py:252-279."""
        src_in_pre = src_in_remote_edges[pre_aggr_edge_idx]
        dst_in_pre = dst_in_remote_edges[pre_aggr_edge_idx]
        src_in_post = device_ops.unique_sorted(src_in_remote_edges[post_aggr_edge_idx])
        src_to_send = torch.cat((src_in_pre, src_in_post), dim=0)
        dst_to_send = torch.cat((dst_in_pre, src_in_post), dim=0)
        order = _stable_argsort(dst_to_send)
        remote_edges_sent_for_graph_exchange.append(torch.cat((src_to_send[order], dst_to_send[order]), dim=0))

    @staticmethod
    def collect_edges_for_aggregation(src_in_remote_edges, dst_in_remote_edges, pre_aggr_edge_idx, post_aggr_edge_idx,
                                      remote_edges_for_aggr_on_recv, recv_splits_for_data_exchange,
                                      begin_edge_on_each_partition_from, cur_rank):
        """Extends this rank's own post-aggregation edge list: POST edges (src,dst) and
        one (d,d) per distinct dst of a PRE edge, ordered by the first component; the
        receive split of ``cur_rank`` is the number of distinct firsts.
        Reference: DataProcessor.py:283-326."""
        src_in_post = src_in_remote_edges[post_aggr_edge_idx]
        dst_in_post = dst_in_remote_edges[post_aggr_edge_idx]
        pre_dst = device_ops.unique_sorted(dst_in_remote_edges[pre_aggr_edge_idx])
        src_from_recv = torch.cat((src_in_post, pre_dst), dim=0)
        dst_from_recv = torch.cat((dst_in_post, pre_dst), dim=0)
        order = _stable_argsort(src_from_recv)
        src_from_recv = src_from_recv[order]
        dst_from_recv = dst_from_recv[order]
        recv_splits_for_data_exchange.append(
            int(device_ops.runs(src_from_recv, want_inverse=False, want_counts=False)[0].shape[0]))
        remote_edges_for_aggr_on_recv[0] = torch.cat((remote_edges_for_aggr_on_recv[0], src_from_recv), dim=0)
        remote_edges_for_aggr_on_recv[1] = torch.cat((remote_edges_for_aggr_on_recv[1], dst_from_recv), dim=0)
        begin_edge_on_each_partition_from[cur_rank + 1] = (
            begin_edge_on_each_partition_from[cur_rank] + src_from_recv.shape[0])

    @staticmethod
    def split_remote_edges_for_aggr_and_graph_exchange(begin_node_on_each_subgraph, remote_edges_list, world_size):
        """Reference: DataProcessor.py:134-199."""
        all_src, all_dst = remote_edges_list[0], remote_edges_list[1]
        dev = all_src.device
        remote_edges_sent_for_graph_exchange: List[torch.Tensor] = []
        recv_splits_for_data_exchange: List[int] = []
        begin_edge_on_each_partition_from = torch.zeros(world_size + 1, dtype=torch.int64)
        remote_edges_for_aggr_on_recv = [torch.empty(0, dtype=torch.int64, device=dev),
                                         torch.empty(0, dtype=torch.int64, device=dev)]
        begins = [int(x) for x in begin_node_on_each_subgraph]
        is_pre, is_post = 1, 0
        for i in range(world_size):
            edge_idx = (all_src >= begins[i]) & (all_src < begins[i + 1])
            src = all_src[edge_idx]
            dst = all_dst[edge_idx]
            flags = DataProcessorForPreAggresive.decide_pre_or_post_aggr(src, dst, is_pre, is_post)
            pre_idx = flags == is_pre
            post_idx = flags == is_post
            DataProcessorForPreAggresive.collect_edges_sent_to_other_subgraphs(
                src, dst, pre_idx, post_idx, remote_edges_sent_for_graph_exchange)
            DataProcessorForPreAggresive.collect_edges_for_aggregation(
                src, dst, pre_idx, post_idx, remote_edges_for_aggr_on_recv, recv_splits_for_data_exchange,
                begin_edge_on_each_partition_from, i)
        begin_edge_on_each_partition_from[world_size] = remote_edges_for_aggr_on_recv[0].shape[0]
        return (remote_edges_sent_for_graph_exchange, remote_edges_for_aggr_on_recv,
                begin_edge_on_each_partition_from, recv_splits_for_data_exchange)

    @staticmethod
    def split_remote_edges_recv_from_graph_exchange(remote_edges_recv_from_graph_exchange, world_size):
        """Reference: DataProcessor.py:202-225."""
        dev = remote_edges_recv_from_graph_exchange[0].device if world_size else None
        srcs, dsts = [], []
        begin_edge_on_each_partition_to = torch.zeros(world_size + 1, dtype=torch.int64)
        send_splits_for_data_exchange = []
        for i in range(world_size):
            packed = remote_edges_recv_from_graph_exchange[i]
            n = int(packed.shape[0] / 2)
            src, dst = packed[:n], packed[n:]
            send_splits_for_data_exchange.append(int(device_ops.unique_sorted(dst).shape[0]))
            srcs.append(src)
            dsts.append(dst)
            begin_edge_on_each_partition_to[i + 1] = begin_edge_on_each_partition_to[i] + dst.shape[0]
        empty = torch.empty(0, dtype=torch.int64, device=dev)
        remote_edges_for_aggr_for_send = [torch.cat([empty] + srcs, dim=0), torch.cat([empty] + dsts, dim=0)]
        begin_edge_on_each_partition_to[world_size] = remote_edges_for_aggr_for_send[0].shape[0]
        return remote_edges_for_aggr_for_send, begin_edge_on_each_partition_to, send_splits_for_data_exchange

    @staticmethod
    def divide_remote_edges_list(begin_node_on_each_subgraph, remote_edges_list, world_size,
                                 graph_exchange: Optional[Callable] = None):
        """``graph_exchange(sent_lists) -> received_lists`` stands in for the two
        all_to_all_single calls (DataProcessor.py:329-382): it is given the W packed
        lists this rank addresses to the others and returns the W packed lists
        addressed to this rank.  Without it nothing is received.  Reference: :385-427."""
        (sent, aggr_on_recv, begin_from, recv_splits) = (
            DataProcessorForPreAggresive.split_remote_edges_for_aggr_and_graph_exchange(
                begin_node_on_each_subgraph, remote_edges_list, world_size))
        dev = remote_edges_list[0].device
        if graph_exchange is not None and world_size != 1:
            received = [_as_i64(x, dev) for x in graph_exchange(sent)]
        else:
            received = [torch.empty(0, dtype=torch.int64, device=dev) for _ in range(world_size)]
        (for_send, begin_to, send_splits) = (
            DataProcessorForPreAggresive.split_remote_edges_recv_from_graph_exchange(received, world_size))
        return aggr_on_recv, for_send, begin_from, begin_to, recv_splits, send_splits

    @staticmethod
    def remap_remote_nodes_id(remote_nodes_list, begin_edge_on_each_partition):
        """Inside each rank segment of a sorted id list, equal neighbours share one
        buffer-row index; the index keeps counting across segments and equality is not
        carried over a segment boundary.  Rewrites the list IN PLACE, returns the
        number of buffer rows.  Reference: DataProcessor.py:432-445."""
        n = int(remote_nodes_list.shape[0])
        if n == 0:
            return 0
        dev = remote_nodes_list.device
        starts = _as_i64(begin_edge_on_each_partition, dev)[:-1]
        values, new_ids, _ = device_ops.runs(remote_nodes_list, forced_starts=starts, want_counts=False)
        remote_nodes_list.copy_(new_ids)
        return int(values.shape[0])

    @staticmethod
    def transform_edge_index_to_sparse_tensor(local_edges_list, remote_edges_list_pre_post_aggr_from,
                                              remote_edges_list_pre_post_aggr_to, begin_edge_on_each_partition_from,
                                              begin_edge_on_each_partition_to, num_local_nodes, local_node_begin_idx):
        """Reference: DataProcessor.py:448-508.  local_adj_t [N,N]; adj_t_pre_post_aggr_from
        = CSR(row = dst - begin, col = buffer row of src, [N,Rv]); adj_t_pre_post_aggr_to =
        CSR(row = buffer row of dst, col = src - begin, [S,N]).  The two remote lists are
        rewritten in place like the reference's."""
        dev = local_edges_list[1].device
        ones = lambda n: torch.ones(n, dtype=torch.float32, device=dev)  # noqa: E731
        local_adj_t = SparseTensor(row=local_edges_list[1], col=local_edges_list[0],
                                   value=ones(local_edges_list[1].shape[0]),
                                   sparse_sizes=(num_local_nodes, num_local_nodes))

        f = remote_edges_list_pre_post_aggr_from
        f[1] -= local_node_begin_idx
        num_from = DataProcessorForPreAggresive.remap_remote_nodes_id(f[0], begin_edge_on_each_partition_from)
        adj_t_pre_post_aggr_from = SparseTensor(row=f[1], col=f[0], value=ones(f[1].shape[0]),
                                                sparse_sizes=(num_local_nodes, num_from))

        t = remote_edges_list_pre_post_aggr_to
        t[0] -= local_node_begin_idx
        num_to = DataProcessorForPreAggresive.remap_remote_nodes_id(t[1], begin_edge_on_each_partition_to)
        adj_t_pre_post_aggr_to = SparseTensor(row=t[1], col=t[0], value=ones(t[1].shape[0]),
                                              sparse_sizes=(num_to, num_local_nodes))
        return local_adj_t, adj_t_pre_post_aggr_from, adj_t_pre_post_aggr_to
