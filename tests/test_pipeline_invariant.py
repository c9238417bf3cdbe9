"""All-ranks invariant of the pre/post-aggregation index maps, at oracle level (CPU).

Every rank of a small partitioned graph is simulated in one process with the oracle's
index-map builders; the setup-time exchanges are replaced by moving the lists between
the simulated ranks.  Then for any X

    out_r = A_local_r X_r + A_from_r * exchange_r( A_to_i X_i for all i )

must equal rows [begin_r, end_r) of the plain global product A X, and the same with all
matrices transposed for the gradient direction.  A wrong orientation, a send/recv row
mismatch, a dropped (s,s)/(d,d) identity pair or a wrong PRE/POST rule fails it.  The
raw-halo (non-pre) maps are checked the same way, which also pins
obtain_local_nodes_required_by_other (the reference's own test for it is commented out)."""
import numpy as np
import pytest

from oracle import aggregator as oagg
from oracle import index_maps as om
from tests.world_sim import World


def build_pre_world(w: World):
    """Per-rank dict of oracle matrices and splits, pre/post mode."""
    W = w.world
    split = []
    for r in range(W):
        local, remote = w.partition(r)
        remote_g = [remote[0].copy(), remote[1] + w.begins[r]]
        split.append((local, om.split_remote_edges_for_aggr_and_graph_exchange(w.begins, remote_g, W)))
    received = om.simulate_graph_exchange([s[1][0] for s in split])
    ranks = []
    for r in range(W):
        local, (sent, aggr_on_recv, begin_from, recv_splits) = split[r]
        for_send, begin_to, send_splits = om.split_remote_edges_recv_from_graph_exchange(received[r], W)
        mats = om.transform_edge_index_to_sparse_tensor_for_pre(
            local, [aggr_on_recv[0].copy(), aggr_on_recv[1].copy()], [for_send[0].copy(), for_send[1].copy()],
            begin_from, begin_to, int(w.sizes[r]), int(w.begins[r]))
        ranks.append(dict(local=mats[0], a_from=mats[1], a_to=mats[2], recv_splits=recv_splits,
                          send_splits=send_splits))
    return ranks


def exchange(send_bufs, send_splits, recv_splits):
    """all_to_all_single with uneven row splits: rank r receives, in rank order, the slice
    of every peer's send buffer addressed to r (communicator.py:85-109)."""
    W = len(send_bufs)
    offs = [np.concatenate(([0], np.cumsum(s))) for s in send_splits]
    recv = []
    for r in range(W):
        parts = [send_bufs[i][offs[i][r]:offs[i][r + 1]] for i in range(W)]
        for i in range(W):
            assert parts[i].shape[0] == recv_splits[r][i], "send rows of i->r do not match recv split of r<-i"
        recv.append(np.concatenate(parts, axis=0))
    return recv


@pytest.mark.parametrize("seed,sizes", [(0, (30, 45, 25)), (1, (60, 1, 40, 33)), (2, (50, 0, 50)), (3, (20, 20, 20, 20, 20))])
def test_pre_post_pipeline_equals_global_product(seed, sizes):
    w = World(seed, sizes)
    ranks = build_pre_world(w)
    W, F = w.world, 7
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((w.n, F)).astype(np.float32)
    xs = [x[w.begins[r]:w.begins[r + 1]] for r in range(W)]
    for r in range(W):
        assert ranks[r]["a_from"][3] == (sizes[r], sum(ranks[r]["recv_splits"]))
        assert ranks[r]["a_to"][3] == (sum(ranks[r]["send_splits"]), sizes[r])
    send = [oagg.forward_send(ranks[r]["a_to"], np.ascontiguousarray(xs[r])) for r in range(W)]
    recv = exchange(send, [k["send_splits"] for k in ranks], [k["recv_splits"] for k in ranks])
    want = w.global_product(x)
    for r in range(W):
        out = oagg.forward_out(ranks[r]["local"], ranks[r]["a_from"], np.ascontiguousarray(xs[r]), recv[r])
        assert np.allclose(out, want[w.begins[r]:w.begins[r + 1]], rtol=1e-5, atol=1e-5)

    # gradient direction: buffers swap roles (aggregator.py:141, :186; communicator.py:91-95)
    g = rng.standard_normal((w.n, F)).astype(np.float32)
    gs = [np.ascontiguousarray(g[w.begins[r]:w.begins[r + 1]]) for r in range(W)]
    back = [oagg.backward_recv(ranks[r]["a_from"], gs[r]) for r in range(W)]
    incoming = exchange(back, [k["recv_splits"] for k in ranks], [k["send_splits"] for k in ranks])
    want_t = w.global_product(g, transposed=True)
    for r in range(W):
        dx = oagg.backward_out(ranks[r]["local"], ranks[r]["a_to"], gs[r], incoming[r])
        assert np.allclose(dx, want_t[w.begins[r]:w.begins[r + 1]], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("seed,sizes", [(4, (30, 45, 25)), (5, (60, 1, 40, 33)), (6, (50, 0, 50))])
def test_raw_halo_pipeline_equals_global_product(seed, sizes):
    w = World(seed, sizes)
    W, F = w.world, 5
    per = []
    for r in range(W):
        local, remote = w.partition(r)
        edges = [remote[0].copy(), remote[1].copy()]
        om.sort_remote_edges_list_based_on_remote_nodes(edges)
        nodes, ranges, counts = om.obtain_remote_nodes_list(edges, int(sizes[r]), w.begins, W)
        per.append(dict(local_e=local, remote_e=edges, nodes=nodes, ranges=ranges, counts=counts))
    asked = om.simulate_halo_id_exchange([p["nodes"] for p in per], [p["ranges"] for p in per])
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((w.n, F)).astype(np.float32)
    g = rng.standard_normal((w.n, F)).astype(np.float32)
    send, back = [], []
    for r in range(W):
        p = per[r]
        p["idx"], p["num_send"] = om.obtain_local_nodes_required_by_other(w.begins[r], asked[r])
        p["local"], p["remote"] = om.transform_edge_index_to_sparse_tensor(p["local_e"], p["remote_e"], int(sizes[r]),
                                                                          len(p["nodes"]))
        assert p["idx"].size == 0 or (p["idx"].min() >= 0 and p["idx"].max() < sizes[r])
        send.append(oagg.forward_send_raw(p["idx"], x[w.begins[r]:w.begins[r + 1]]))
        back.append(oagg.backward_recv(p["remote"], np.ascontiguousarray(g[w.begins[r]:w.begins[r + 1]])))
    send_splits = [p["num_send"].tolist() for p in per]
    recv_splits = [p["counts"].tolist() for p in per]
    recv = exchange(send, send_splits, recv_splits)
    incoming = exchange(back, recv_splits, send_splits)
    want, want_t = w.global_product(x), w.global_product(g, transposed=True)
    for r in range(W):
        p = per[r]
        sl = slice(w.begins[r], w.begins[r + 1])
        out = oagg.forward_out(p["local"], p["remote"], np.ascontiguousarray(x[sl]), recv[r])
        assert np.allclose(out, want[sl], rtol=1e-5, atol=1e-5)
        dx = oagg.backward_out_raw(p["local"], p["idx"], np.ascontiguousarray(g[sl]), incoming[r])
        assert np.allclose(dx, want_t[sl], rtol=1e-5, atol=1e-5)
