"""TEST INFRASTRUCTURE -- CPU oracle for the index maps of the aggregation path.

A numpy / plain-loop restatement of the reference's graph pre-processing, written to
be read next to the reference: one function per reference function, same argument
meaning, same in-place side effects where the reference has them.  Small inputs only
(the loops are per-edge Python, like the reference's).  Paths are relative to
/root/reference/self_benchmark/a64fx/.

Pinning status (what fixes each function's answers independently of this file):
  get_in_degrees .......................... tests/test_data_preprocessor.py:96-102 vector
  sort_remote_edges_list_based_on_remote_nodes ... :11-14 vector
  obtain_remote_nodes_list ................ :16-27 and :64-74 vectors
  transform_edge_index_to_sparse_tensor ... :42-93 dense-equality vectors
  build_csr (torch_sparse.SparseTensor, third-party, not in the tree) ...
        pinned through the two dense-equality vectors above and scipy's coo->csr
        with sorted indices; duplicates are kept (no coalescing)
  get_degrees ............................. tests/test_data_preprocessor_pre_aggr.py:12-31
  decide_pre_or_post_aggr ................. :33-62 (4 cases)
  collect_edges_sent_to_other_subgraphs ... :64-109 (3 cases)
  collect_edges_for_aggregation ........... :111-182 (3 cases)
  split_remote_edges_for_aggr_and_graph_exchange ... :184-227 (4-rank worked example)
  split_remote_edges_recv_from_graph_exchange ...... :230-292 (3 cases)
  remap_remote_nodes_id ................... :294-358 (8 cases)
  obtain_local_nodes_required_by_other .... the reference's test is commented out
        (tests/test_data_preprocessor.py:29-40) and it needs a process group:
        PARITY UNPINNED beyond its closed form (ids requested by rank r, minus the
        local begin) and the all-ranks invariant in tests/test_pipeline_invariant.py
  divide_edges_into_local_and_remote ...... tests/test_postprocess_graph_data.py:10-40 (3 vectors)
  simulate_* helpers ...................... no reference counterpart: they replace the
        setup-time all_to_all calls (DataProcessor.py:76-98, :329-382) by moving the
        lists between simulated ranks in one process

Tie order: the reference sorts with ``torch.argsort`` (not guaranteed stable).  Every
reference vector above agrees with a STABLE sort, which is what is used here; the
final CSR matrices and split lists do not depend on the tie order.
"""
import numpy as np

I64 = np.int64


# --------------------------------------------------------------------------- A7
def build_csr(row, col, value, num_rows):
    """CSR arrays of a COO list the way ``SparseTensor(row=, col=, value=,
    sparse_sizes=)`` lays them out (call sites data_manager/DataProcessor.py:104-116,
    :458-502): entries ordered by (row, col), duplicates kept, ``rowptr`` by counting."""
    row = np.asarray(row, dtype=I64)
    col = np.asarray(col, dtype=I64)
    value = np.asarray(value, dtype=np.float32)
    perm = np.lexsort((col, row))  # stable: last key is primary
    rowptr = np.zeros(num_rows + 1, dtype=I64)
    for r in row:
        rowptr[r + 1] += 1
    np.cumsum(rowptr, out=rowptr)
    return rowptr, col[perm].copy(), value[perm].copy()


def csr_to_dense(rowptr, col, value, num_cols):
    rows = rowptr.shape[0] - 1
    dense = np.zeros((rows, num_cols), dtype=np.float64)
    for r in range(rows):
        for e in range(rowptr[r], rowptr[r + 1]):
            dense[r, col[e]] += value[e]
    return dense


# --------------------------------------------------------------------------- A5
def get_in_degrees(local_edges_list, remote_edges_list, num_local_nodes):
    """data_manager/DataProcessor.py:12-18: fp32 [N,1] count of incoming edges over the
    local and remote lists (row 1 = localised dst), clamped to at least 1."""
    degs = np.zeros(num_local_nodes, dtype=np.float32)
    for d in np.asarray(local_edges_list[1], dtype=I64):
        degs[d] += 1.0
    for d in np.asarray(remote_edges_list[1], dtype=I64):
        degs[d] += 1.0
    return np.maximum(degs, 1.0).reshape(-1, 1)


def sort_remote_edges_list_based_on_remote_nodes(remote_edges_list):
    """DataProcessor.py:20-26: order the remote edges by their (remote) src id;
    writes rows 0 and 1 of the argument and returns it."""
    src = np.asarray(remote_edges_list[0], dtype=I64)
    dst = np.asarray(remote_edges_list[1], dtype=I64)
    order = np.argsort(src, kind="stable")
    remote_edges_list[0] = src[order]
    remote_edges_list[1] = dst[order]
    return remote_edges_list


def obtain_remote_nodes_list(remote_edges_list, num_local_nodes, num_nodes_on_each_subgraph, world_size):
    """DataProcessor.py:28-60: scan the src-sorted remote edges; every new src id is a
    halo node, appended to the halo list and given the next local id starting at
    ``num_local_nodes`` (src row rewritten IN PLACE, :53); per owning rank the halo
    range [W+1] and count [W] are accumulated (:44-51, :55-56)."""
    begins = [int(x) for x in num_nodes_on_each_subgraph]
    remote_nodes_list = []
    ranges = np.zeros(world_size + 1, dtype=I64)
    counts = np.zeros(world_size, dtype=I64)
    src = remote_edges_list[0]
    part_idx = 0
    local_node_idx = num_local_nodes - 1
    prev_node = -1
    for i in range(len(src)):
        cur_node = int(src[i])
        if cur_node != prev_node:
            remote_nodes_list.append(cur_node)
            local_node_idx += 1
            while cur_node >= begins[part_idx + 1]:
                part_idx += 1
                ranges[part_idx + 1] = ranges[part_idx]
            ranges[part_idx + 1] += 1
            counts[part_idx] += 1
        prev_node = cur_node
        src[i] = local_node_idx
    for i in range(part_idx + 1, world_size):
        ranges[i + 1] = ranges[i]
    return np.asarray(remote_nodes_list, dtype=I64), ranges, counts


def obtain_local_nodes_required_by_other(local_node_begin, recv_nodes_list):
    """DataProcessor.py:62-98 after its two all_to_all calls: ``recv_nodes_list[r]`` holds
    the global ids rank r asked this rank for; the send index list is their
    concatenation minus this rank's first global id (:95-97), the counts one per rank."""
    num = np.asarray([len(x) for x in recv_nodes_list], dtype=I64)
    parts = [np.asarray(x, dtype=I64) - int(local_node_begin) for x in recv_nodes_list]
    idx = np.concatenate(parts) if parts else np.zeros(0, dtype=I64)
    return idx.astype(I64), num


def transform_edge_index_to_sparse_tensor(local_edges_list, remote_edges_list, num_local_nodes, num_remote_nodes):
    """DataProcessor.py:100-118: ``local_adj_t`` = CSR(row=dst, col=src, 1, [N,N]) and
    ``remote_adj_t`` = CSR(row=dst, col=src - N, 1, [N,Rv]).  Returns two
    (rowptr, col, value, (rows, cols)) tuples."""
    ls, ld = np.asarray(local_edges_list[0], dtype=I64), np.asarray(local_edges_list[1], dtype=I64)
    rs, rd = np.asarray(remote_edges_list[0], dtype=I64), np.asarray(remote_edges_list[1], dtype=I64)
    local = build_csr(ld, ls, np.ones(ld.shape[0], np.float32), num_local_nodes) + ((num_local_nodes, num_local_nodes),)
    remote = build_csr(rd, rs - num_local_nodes, np.ones(rd.shape[0], np.float32), num_local_nodes) + (
        (num_local_nodes, num_remote_nodes),)
    return local, remote


# --------------------------------------------------------------------------- A6
def get_degrees(nodes_list):
    """DataProcessor.py:125-131: {node id: number of occurrences}."""
    degrees = {}
    for n in np.asarray(nodes_list, dtype=I64):
        degrees[int(n)] = degrees.get(int(n), 0) + 1
    return degrees


def decide_pre_or_post_aggr(src, dst, is_pre=1, is_post=0):
    """DataProcessor.py:228-248: an edge is POST-aggregated when the out-degree of its
    src exceeds the in-degree of its dst (degrees counted inside this src-rank subset),
    otherwise PRE-aggregated."""
    src = np.asarray(src, dtype=I64)
    dst = np.asarray(dst, dtype=I64)
    out_deg = get_degrees(src)
    in_deg = get_degrees(dst)
    flags = np.zeros(src.shape[0], dtype=I64)
    for e in range(src.shape[0]):
        flags[e] = is_post if out_deg[int(src[e])] > in_deg[int(dst[e])] else is_pre
    return flags


def _take(a, idx):
    """Index with either a boolean mask or an integer index list (the reference's
    tests pass index lists, its own caller passes masks)."""
    a = np.asarray(a, dtype=I64)
    idx = np.asarray(idx)
    if idx.dtype == np.bool_:
        return a[idx]
    return a[idx.astype(I64)]


def collect_edges_sent_to_other_subgraphs(src, dst, pre_idx, post_idx, sent_lists):
    """DataProcessor.py:252-279: what this rank tells the src-owning rank: its PRE edges
    (src,dst) plus one (s,s) pair per distinct src of a POST edge, ordered by the second
    component, packed as [all firsts | all seconds] and appended to ``sent_lists``."""
    src_in_pre = _take(src, pre_idx)
    dst_in_pre = _take(dst, pre_idx)
    src_in_post = np.unique(_take(src, post_idx))
    src_to_send = np.concatenate((src_in_pre, src_in_post))
    dst_to_send = np.concatenate((dst_in_pre, src_in_post))
    order = np.argsort(dst_to_send, kind="stable")
    sent_lists.append(np.concatenate((src_to_send[order], dst_to_send[order])).astype(I64))


def collect_edges_for_aggregation(src, dst, pre_idx, post_idx, aggr_on_recv, recv_splits, begin_edge_from, cur_rank):
    """DataProcessor.py:283-326: what this rank aggregates itself after the exchange:
    its POST edges (src,dst) plus one (d,d) pair per distinct dst of a PRE edge, ordered
    by the first component; appended to the two running lists.  The receive split of
    ``cur_rank`` is the number of distinct firsts; the running edge offset goes to
    ``begin_edge_from[cur_rank + 1]``."""
    src_in_post = _take(src, post_idx)
    dst_in_post = _take(dst, post_idx)
    pre_dst_unique = np.unique(_take(dst, pre_idx))
    src_from_recv = np.concatenate((src_in_post, pre_dst_unique))
    dst_from_recv = np.concatenate((dst_in_post, pre_dst_unique))
    order = np.argsort(src_from_recv, kind="stable")
    src_from_recv = src_from_recv[order]
    dst_from_recv = dst_from_recv[order]
    recv_splits.append(int(np.unique(src_from_recv).shape[0]))
    aggr_on_recv[0] = np.concatenate((np.asarray(aggr_on_recv[0], dtype=I64), src_from_recv))
    aggr_on_recv[1] = np.concatenate((np.asarray(aggr_on_recv[1], dtype=I64), dst_from_recv))
    begin_edge_from[cur_rank + 1] = begin_edge_from[cur_rank] + src_from_recv.shape[0]


def split_remote_edges_for_aggr_and_graph_exchange(begin_node_on_each_subgraph, remote_edges_list, world_size):
    """DataProcessor.py:134-199: per src-owning rank i, take the remote edges whose src
    lies in [begin_i, begin_{i+1}), classify them PRE/POST, and build (a) the packed list
    sent to rank i and (b) this rank's own post-aggregation edge list + receive splits."""
    begins = [int(x) for x in begin_node_on_each_subgraph]
    sent = []
    recv_splits = []
    begin_edge_from = np.zeros(world_size + 1, dtype=I64)
    aggr_on_recv = [np.zeros(0, dtype=I64), np.zeros(0, dtype=I64)]
    all_src = np.asarray(remote_edges_list[0], dtype=I64)
    all_dst = np.asarray(remote_edges_list[1], dtype=I64)
    for i in range(world_size):
        mask = (all_src >= begins[i]) & (all_src < begins[i + 1])
        src = all_src[mask]
        dst = all_dst[mask]
        flags = decide_pre_or_post_aggr(src, dst, 1, 0)
        pre = flags == 1
        post = flags == 0
        collect_edges_sent_to_other_subgraphs(src, dst, pre, post, sent)
        collect_edges_for_aggregation(src, dst, pre, post, aggr_on_recv, recv_splits, begin_edge_from, i)
    begin_edge_from[world_size] = aggr_on_recv[0].shape[0]
    return sent, aggr_on_recv, begin_edge_from, recv_splits


def split_remote_edges_recv_from_graph_exchange(recv_lists, world_size):
    """DataProcessor.py:202-225: unpack what the other ranks sent ([firsts | seconds]
    halves), concatenate in rank order, send split of rank i = distinct seconds."""
    for_send = [np.zeros(0, dtype=I64), np.zeros(0, dtype=I64)]
    begin_edge_to = np.zeros(world_size + 1, dtype=I64)
    send_splits = []
    for i in range(world_size):
        packed = np.asarray(recv_lists[i], dtype=I64)
        n = int(packed.shape[0] / 2)
        src = packed[:n]
        dst = packed[n:]
        send_splits.append(int(np.unique(dst).shape[0]))
        for_send[0] = np.concatenate((for_send[0], src))
        for_send[1] = np.concatenate((for_send[1], dst))
        begin_edge_to[i + 1] = begin_edge_to[i] + dst.shape[0]
    begin_edge_to[world_size] = for_send[0].shape[0]
    return for_send, begin_edge_to, send_splits


def remap_remote_nodes_id(remote_nodes_list, begin_edge_on_each_partition):
    """DataProcessor.py:432-445: inside each rank segment of a sorted id list give
    consecutive-equal ids one buffer-row index; the index keeps counting across
    segments, and equality is NOT carried over a segment boundary (prev reset, :435).
    Rewrites the list IN PLACE and returns the number of buffer rows."""
    local_node_idx = -1
    for rank in range(len(begin_edge_on_each_partition) - 1):
        prev_node = -1
        begin = int(begin_edge_on_each_partition[rank])
        num = int(begin_edge_on_each_partition[rank + 1]) - begin
        for i in range(num):
            cur = int(remote_nodes_list[begin + i])
            if cur != prev_node:
                local_node_idx += 1
            prev_node = cur
            remote_nodes_list[begin + i] = local_node_idx
    return local_node_idx + 1


def transform_edge_index_to_sparse_tensor_for_pre(local_edges_list, from_list, to_list, begin_edge_from,
                                                  begin_edge_to, num_local_nodes, local_node_begin_idx):
    """DataProcessor.py:448-508.  Returns three (rowptr, col, value, (rows, cols)) tuples:
    local_adj_t [N,N]; adj_t_pre_post_aggr_from = CSR(row = dst - begin, col = remapped
    src, [N,Rv]); adj_t_pre_post_aggr_to = CSR(row = remapped dst, col = src - begin,
    [S,N]).  ``from_list`` / ``to_list`` are rewritten in place as in the reference."""
    ls, ld = np.asarray(local_edges_list[0], dtype=I64), np.asarray(local_edges_list[1], dtype=I64)
    n = num_local_nodes
    local = build_csr(ld, ls, np.ones(ld.shape[0], np.float32), n) + ((n, n),)

    from_list[1] = np.asarray(from_list[1], dtype=I64) - int(local_node_begin_idx)
    from_list[0] = np.asarray(from_list[0], dtype=I64).copy()
    num_from = remap_remote_nodes_id(from_list[0], begin_edge_from)
    a_from = build_csr(from_list[1], from_list[0], np.ones(from_list[1].shape[0], np.float32), n) + ((n, num_from),)

    to_list[0] = np.asarray(to_list[0], dtype=I64) - int(local_node_begin_idx)
    to_list[1] = np.asarray(to_list[1], dtype=I64).copy()
    num_to = remap_remote_nodes_id(to_list[1], begin_edge_to)
    a_to = build_csr(to_list[1], to_list[0], np.ones(to_list[1].shape[0], np.float32), num_to) + ((num_to, n),)
    return local, a_from, a_to


# ------------------------------------------------- single-process stand-ins for the setup collectives
def simulate_graph_exchange(sent_lists_per_rank):
    """Stand-in for DataProcessor.py:329-382 (all_to_all_single of the packed edge
    lists): ``result[r][i]`` is what rank i sent to rank r."""
    world = len(sent_lists_per_rank)
    return [[np.asarray(sent_lists_per_rank[i][r], dtype=I64) for i in range(world)] for r in range(world)]


def simulate_halo_id_exchange(remote_nodes_list_per_rank, ranges_per_rank):
    """Stand-in for DataProcessor.py:76-94 (all_to_all of the halo id lists):
    ``result[r][i]`` is the slice of rank i's halo list owned by rank r."""
    world = len(remote_nodes_list_per_rank)
    return [[np.asarray(remote_nodes_list_per_rank[i][int(ranges_per_rank[i][r]):int(ranges_per_rank[i][r + 1])],
                        dtype=I64) for i in range(world)] for r in range(world)]


# ------------------------------------------------- file contract on the input side
def divide_edges_into_local_and_remote(edges_list, node_idx_begin, node_idx_end):
    """graph_partition_scripts/postprocess_graph_multi_proc.py:10-44: edges [E,2] of global
    (src, dst) whose dst lies in [begin, end] (end inclusive); local edges have both ids
    localised, remote edges keep the global src.  Pinned by
    tests/test_postprocess_graph_data.py:10-40 (3 vectors)."""
    local_s, local_d, remote_s, remote_d = [], [], [], []
    for s, d in np.asarray(edges_list, dtype=I64).reshape(-1, 2):
        assert node_idx_begin <= d <= node_idx_end
        if node_idx_begin <= s <= node_idx_end:
            local_s.append(s - node_idx_begin)
            local_d.append(d - node_idx_begin)
        else:
            remote_s.append(s)
            remote_d.append(d - node_idx_begin)
    return (np.asarray([local_s, local_d], dtype=I64).reshape(2, -1),
            np.asarray([remote_s, remote_d], dtype=I64).reshape(2, -1))
