"""The on-disk form of one partition, on the side that FEEDS the index-map builders.

The reference produces these files offline (self_benchmark/a64fx/graph_partition_scripts/
postprocess_graph_multi_proc.py:10-44, :63-139, :273-282) and reads them in
data_manager/DataLoader.py:12-61.  Only the contract is restated here -- which edges are
local or remote and how their ids are localised, and the file names / dtypes -- so that a
partitioned edge list (or a synthetic partition) can be handed to
``load_graph_structures`` and the builders.
"""
import os
from typing import Tuple

import numpy as np
import torch


def divide_edges_into_local_and_remote(edges_list: torch.Tensor, node_idx_begin: int,
                                       node_idx_end: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Split the edges whose dst this partition owns.  ``edges_list`` is int64 [E, 2] of
    (src, dst) GLOBAL ids with every dst in [node_idx_begin, node_idx_end] (END INCLUSIVE,
    like the reference).  Returns (local_edges [2, E_l] with src and dst localised,
    remote_edges [2, E_r] with src still global and dst localised), edge order preserved.
    Reference: postprocess_graph_multi_proc.py:10-44."""
    src, dst = edges_list[:, 0], edges_list[:, 1]
    if dst.numel() and (int(dst.min()) < node_idx_begin or int(dst.max()) > node_idx_end):
        raise AssertionError("a dst id lies outside this partition's node range")
    is_local = (src >= node_idx_begin) & (src <= node_idx_end)
    local = torch.stack((src[is_local] - node_idx_begin, dst[is_local] - node_idx_begin))
    remote = torch.stack((src[~is_local], dst[~is_local] - node_idx_begin))
    return local, remote


def save_partition_files(output_dir: str, graph_name: str, rank: int, begins, local_edges: torch.Tensor,
                         remote_edges: torch.Tensor) -> None:
    """Writes ``p{rank:03d}-{name}_nodes.npy`` (int64 [N, 2]: partition-contiguous id, original
    id), ``..._local_edges.npy``, ``..._remote_edges.npy`` and
    ``begin_node_on_each_partition.txt`` the way DataLoader.py:12-40 expects to read them."""
    os.makedirs(output_dir, exist_ok=True)
    begins = np.asarray(begins, dtype=np.int64)
    ids = np.arange(begins[rank], begins[rank + 1], dtype=np.int64)
    prefix = os.path.join(output_dir, "p{:0>3d}-{}".format(rank, graph_name))
    np.save(prefix + "_nodes.npy", np.stack((ids, ids), axis=1))
    np.save(prefix + "_local_edges.npy", local_edges.cpu().numpy().astype(np.int64))
    np.save(prefix + "_remote_edges.npy", remote_edges.cpu().numpy().astype(np.int64))
    np.savetxt(os.path.join(output_dir, "begin_node_on_each_partition.txt"), begins.reshape(1, -1), fmt="%d",
               delimiter=" ")
