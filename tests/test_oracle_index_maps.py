"""Pins oracle/index_maps.py against the known-answer vectors the reference's own unit
tests hold (tests/golden/reference_index_map_vectors.json names file:line of each)."""
import numpy as np

from oracle import index_maps as om


def A(x):
    return np.asarray(x, dtype=np.int64)


def test_sort_remote_edges(golden):
    for c in golden["sort_remote_edges"]:
        edges = [A(c["edges"][0]), A(c["edges"][1])]
        out = om.sort_remote_edges_list_based_on_remote_nodes(edges)
        assert np.array_equal(np.stack(out), A(c["expected"]))


def test_obtain_remote_nodes_list(golden):
    for c in golden["obtain_remote_nodes_list"]:
        edges = [A(c["edges"][0]), A(c["edges"][1])]
        edges = om.sort_remote_edges_list_based_on_remote_nodes(edges)
        nodes, ranges, counts = om.obtain_remote_nodes_list(edges, c["num_local_nodes"], c["begins"], c["world_size"])
        assert np.array_equal(np.stack(edges), A(c["expected_edges"]))  # src row rewritten in place
        assert np.array_equal(nodes, A(c["expected_remote_nodes"]))
        assert np.array_equal(ranges, A(c["expected_ranges"]))
        assert np.array_equal(counts, A(c["expected_counts"]))


def _coo_dense(coo):
    d = np.zeros(coo["size"])
    d[coo["row"], coo["col"]] = coo["val"]  # assignment, like the SparseTensor.to_dense() the reference compares
    return d


def test_transform_edge_index_to_sparse_tensor(golden):
    for c in golden["transform_edge_index_to_sparse_tensor"]:
        local, remote = om.transform_edge_index_to_sparse_tensor(
            [A(c["local_edges"][0]), A(c["local_edges"][1])], [A(c["remote_edges"][0]), A(c["remote_edges"][1])],
            c["num_local_nodes"], c["num_remote_nodes"])
        for got, key, edges in ((local, "expected_local_coo", c["local_edges"]),
                                (remote, "expected_remote_coo", c["remote_edges"])):
            rowptr, col, val, shape = got
            assert list(shape) == c[key]["size"]
            dense = om.csr_to_dense(rowptr, col, val, shape[1])
            assert np.array_equal(dense > 0, _coo_dense(c[key]) > 0)  # orientation row=dst, col=src(-N)
            assert col.shape[0] == len(edges[0]) and dense.sum() == len(edges[0])  # repeated edges kept
            assert np.all(val == 1.0)
            for r in range(shape[0]):  # columns ascending inside a row
                assert np.all(np.diff(col[rowptr[r]:rowptr[r + 1]]) >= 0)


def test_build_csr_equals_scipy_with_duplicates():
    import scipy.sparse as sp

    rng = np.random.default_rng(0)
    row, col = rng.integers(0, 40, 600), rng.integers(0, 30, 600)
    val = rng.standard_normal(600).astype(np.float32)
    rowptr, c, v = om.build_csr(row, col, val, 40)
    assert rowptr[-1] == 600
    ref = sp.coo_matrix((val.astype(np.float64), (row, col)), shape=(40, 30)).toarray()
    assert np.allclose(om.csr_to_dense(rowptr, c, v, 30), ref)


def test_get_in_degrees(golden):
    for c in golden["get_in_degrees"]:
        got = om.get_in_degrees([A(x) for x in c["local_edges"]], [A(x) for x in c["remote_edges"]],
                                c["num_local_nodes"])
        assert got.dtype == np.float32 and np.array_equal(got, np.asarray(c["expected"], dtype=np.float32))


def test_get_degrees(golden):
    for c in golden["get_degrees"]:
        assert om.get_degrees(A(c["nodes"])) == {int(k): v for k, v in c["expected"].items()}
    rng = np.random.default_rng(1)
    nodes = rng.integers(0, 100, 10000)  # tests/test_data_preprocessor_pre_aggr.py:28-31
    assert om.get_degrees(nodes) == {int(n): int((nodes == n).sum()) for n in np.unique(nodes)}


def test_decide_pre_or_post_aggr(golden):
    for c in golden["decide_pre_or_post_aggr"]:
        got = om.decide_pre_or_post_aggr(A(c["src"]), A(c["dst"]), c["is_pre"], c["is_post"])
        assert np.array_equal(got, A(c["expected"])), c["source"]


def test_collect_edges_sent_to_other_subgraphs(golden):
    for c in golden["collect_edges_sent_to_other_subgraphs"]:
        sent = []
        om.collect_edges_sent_to_other_subgraphs(A(c["src"]), A(c["dst"]), A(c["pre_idx"]), A(c["post_idx"]), sent)
        n = len(c["expected_src_to_send"])
        assert np.array_equal(sent[0][:n], A(c["expected_src_to_send"])), c["source"]
        assert np.array_equal(sent[0][n:], A(c["expected_dst_to_send"])), c["source"]


def test_collect_edges_for_aggregation(golden):
    for c in golden["collect_edges_for_aggregation"]:
        lists, splits, begin = [A([]), A([])], [], np.zeros(2, dtype=np.int64)
        om.collect_edges_for_aggregation(A(c["src"]), A(c["dst"]), A(c["pre_idx"]), A(c["post_idx"]), lists, splits,
                                         begin, 0)
        assert np.array_equal(lists[0], A(c["expected_src"])), c["source"]
        assert np.array_equal(lists[1], A(c["expected_dst"])), c["source"]
        assert splits == c["expected_splits"] and np.array_equal(begin, A(c["expected_begin_edge"]))


def test_split_remote_edges_for_aggr_and_graph_exchange(golden):
    for c in golden["split_remote_edges_for_aggr_and_graph_exchange"]:
        sent, aggr, begin_from, recv_splits = om.split_remote_edges_for_aggr_and_graph_exchange(
            c["begins"], [A(c["edges"][0]), A(c["edges"][1])], c["world_size"])
        assert len(sent) == len(c["expected_sent"])
        for got, exp in zip(sent, c["expected_sent"]):
            assert np.array_equal(got, A(exp))
        assert np.array_equal(aggr[0], A(c["expected_aggr_on_recv"][0]))
        assert np.array_equal(aggr[1], A(c["expected_aggr_on_recv"][1]))
        assert np.array_equal(begin_from, A(c["expected_begin_edge_from"]))
        assert recv_splits == c["expected_recv_splits"]


def test_split_remote_edges_recv_from_graph_exchange(golden):
    for c in golden["split_remote_edges_recv_from_graph_exchange"]:
        lists, begin_to, splits = om.split_remote_edges_recv_from_graph_exchange(
            [A(x) for x in c["recv_lists"]], c["world_size"])
        assert np.array_equal(lists[0], A(c["expected_lists"][0])) and np.array_equal(lists[1], A(c["expected_lists"][1]))
        assert np.array_equal(begin_to, A(c["expected_begin_edge_to"])) and splits == c["expected_send_splits"]


def test_remap_remote_nodes_id(golden):
    for c in golden["remap_remote_nodes_id"]:
        nodes = A(c["nodes"]).copy()
        assert om.remap_remote_nodes_id(nodes, A(c["begins"])) == c["expected_count"], c["source"]
        assert np.array_equal(nodes, A(c["expected_nodes"])), c["source"]


def test_divide_edges_into_local_and_remote(golden):
    for c in golden["divide_edges_into_local_and_remote"]:
        local, remote = om.divide_edges_into_local_and_remote(A(c["edges"]).T, c["begin"], c["end"])
        assert np.array_equal(local, A(c["expected_local"]).reshape(2, -1)), c["source"]
        assert np.array_equal(remote, A(c["expected_remote"]).reshape(2, -1)), c["source"]
