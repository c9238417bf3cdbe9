"""Host-side pieces of the row-restricted last layer (no GPU): the matrices the restricted aggregation runs on are
checked against dense arithmetic, and the restricted view of a graph against the graph it reads from."""
import numpy as np
import pytest
import torch

from gnn_benchmark_amd.aggregator import SparseTensor, _RowRestrictedGraph, restricted_transpose, select_rows


def _random_matrix(rows, cols, density, seed, with_values=True):
    gen = torch.Generator().manual_seed(seed)
    dense = (torch.rand(rows, cols, generator=gen) < density).float()
    if with_values:
        dense = dense * (torch.rand(rows, cols, generator=gen) + 0.5)
    r, c = dense.nonzero(as_tuple=True)
    m = SparseTensor(row=r, col=c, value=dense[r, c] if with_values else None, sparse_sizes=(rows, cols))
    return dense, m


def _to_dense(m):
    rowptr, col, value = m.csr()
    out = torch.zeros(m.sparse_size(0), m.sparse_size(1))
    counts = rowptr[1:] - rowptr[:-1]
    row = torch.repeat_interleave(torch.arange(m.sparse_size(0)), counts)
    out[row, col] = torch.ones(col.numel()) if value is None else value
    return out


@pytest.mark.parametrize("with_values", [True, False])
def test_select_rows_is_the_dense_row_selection(with_values):
    dense, m = _random_matrix(40, 23, 0.2, 1, with_values)
    gen = torch.Generator().manual_seed(2)
    for rows in (torch.randperm(40, generator=gen)[:9], torch.tensor([39, 0, 0, 17]), torch.zeros(0, dtype=torch.int64)):
        picked = select_rows(m, rows)
        assert picked.sparse_sizes() == (rows.numel(), 23)
        assert torch.equal(_to_dense(picked), dense[rows])
        rowptr, col, _ = picked.csr()
        for i in range(rows.numel()):  # entries of a row keep their (ascending-column) order
            assert np.all(np.diff(col[rowptr[i]:rowptr[i + 1]].numpy()) > 0)


def test_select_rows_handles_empty_rows_and_an_empty_matrix():
    dense = torch.zeros(6, 4)
    dense[1, 2] = 3.0
    r, c = dense.nonzero(as_tuple=True)
    m = SparseTensor(row=r, col=c, value=dense[r, c], sparse_sizes=(6, 4))
    assert torch.equal(_to_dense(select_rows(m, torch.tensor([0, 1, 5]))), dense[[0, 1, 5]])
    assert select_rows(m, torch.tensor([0, 3])).nnz() == 0


@pytest.mark.parametrize("with_values", [True, False])
def test_restricted_transpose_drops_exactly_the_unset_rows(with_values):
    dense, m = _random_matrix(31, 17, 0.25, 3, with_values)
    gen = torch.Generator().manual_seed(4)
    for kept in (torch.randperm(31, generator=gen)[:5], torch.arange(31), torch.zeros(0, dtype=torch.int64)):
        mask = torch.zeros(31, dtype=torch.bool)
        mask[kept] = True
        t = restricted_transpose(m, mask)
        assert t.sparse_sizes() == (17, 31)
        assert torch.equal(_to_dense(t), (dense * mask[:, None].float()).t())
        # against a gradient that is zero outside the kept rows, the restricted transpose is the whole transpose
        g = torch.randn(31, 6, generator=gen) * mask[:, None].float()
        assert torch.allclose(_to_dense(t) @ g, dense.t() @ g, rtol=0, atol=0)


def test_restricted_view_reads_everything_else_from_its_graph():
    class Graph:
        pass

    graph = Graph()
    graph.local_adj_t, graph.in_degrees, graph.comm_buf = "full matrix", "all degrees", "buffers"
    view = _RowRestrictedGraph(graph, {"local_adj_t": "some rows", "in_degrees": "their degrees", "remote_adj_t": None})
    assert (view.local_adj_t, view.in_degrees, view.remote_adj_t) == ("some rows", "their degrees", None)
    assert view.comm_buf == "buffers"
    graph.exchange = "attached after the view was made"
    assert view.exchange == "attached after the view was made"
    assert getattr(view, "never_set", None) is None
    view.scratch = 1  # what is set on the view stays on the view
    assert not hasattr(graph, "scratch")
