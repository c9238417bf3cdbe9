"""Pins the CPU oracle of the SpMM operator (oracle/spmm_oracle.c) against things that
do not share its code: scipy / dense fp64 products on the recipe of the reference's own
test (self_benchmark/a64fx/tests/test_spmm.py:70-115), the accumulate invariant, a
feature-width sweep across the reference's 16- and 64-float block edges, closed forms
of the work splitters, and -- where oracle/_ref is built -- the reference's compiled
operator itself, bit for bit."""
import numpy as np
import pytest
import scipy.sparse as sp

from oracle import spmm as ospmm


def _recipe(rows=20020, cols=1020, density=0.0007, feat=128, seed=0):
    a = sp.rand(rows, cols, density=density, format="csr", dtype=np.float32, random_state=seed)
    a.sort_indices()
    rng = np.random.default_rng(seed)
    x = rng.random((cols, feat), dtype=np.float32)
    return a, x


def test_forward_matches_scipy_and_dense_fp64_on_reference_recipe():
    a, x = _recipe()
    out = np.zeros((a.shape[0], x.shape[1]), dtype=np.float32)
    ospmm.spmm(a.indptr, a.indices, a.data, x, out)
    dense = a.toarray().astype(np.float64) @ x.astype(np.float64)
    # tolerance of the reference's own assertion (tests/test_spmm.py:113)
    assert np.allclose(out, dense, atol=1e-5)
    assert np.allclose(out, a @ x, atol=1e-5)


def test_backward_matches_transposed_product_on_reference_recipe():
    a, _ = _recipe()
    rng = np.random.default_rng(1)
    g = rng.standard_normal((a.shape[0], 128)).astype(np.float32)
    out = np.zeros((a.shape[1], 128), dtype=np.float32)
    ospmm.spmm_transposed(a.indptr, a.indices, a.data, g, out, a.shape[1])
    ref = a.T.toarray().astype(np.float64) @ g.astype(np.float64)
    assert np.allclose(out, ref, rtol=1e-5, atol=1e-5)


def test_transposed_arrays_equal_scipy_csc():
    a, _ = _recipe(rows=500, cols=300, density=0.02)
    colptr, row_t, val_t = ospmm.csr_transpose(a.indptr, a.indices, a.data, a.shape[1])
    c = a.tocsc()
    c.sort_indices()
    assert np.array_equal(colptr, c.indptr) and np.array_equal(row_t, c.indices) and np.array_equal(val_t, c.data)


@pytest.mark.parametrize("feat", [1, 15, 16, 17, 47, 63, 64, 65, 100, 128, 130, 602])
def test_accumulates_into_out_for_every_block_shape(feat):
    # widths straddle the reference's vector (16) and main-block (64) edges, spmm.cpp:452-479
    a, x = _recipe(rows=257, cols=190, density=0.05, feat=feat, seed=feat)
    rng = np.random.default_rng(feat)
    out0 = rng.standard_normal((a.shape[0], feat)).astype(np.float32)
    out = out0.copy()
    ospmm.spmm(a.indptr, a.indices, a.data, x, out)
    expect = out0.astype(np.float64) + a.toarray().astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(out, expect, rtol=1e-5, atol=1e-5)
    # a dropped "load out first" would fail this: zero matrix leaves out untouched
    z = sp.csr_matrix((a.shape[0], a.shape[1]), dtype=np.float32)
    out = out0.copy()
    ospmm.spmm(z.indptr, z.indices, z.data, x, out)
    assert np.array_equal(out, out0)


def test_one_hot_rows_copy_dense_rows_exactly():
    # A with one unit entry per row is a row gather: a wrong index or a transposed operand fails
    rng = np.random.default_rng(3)
    cols, rows, feat = 50, 80, 33
    pick = rng.integers(0, cols, rows)
    rowptr = np.arange(rows + 1, dtype=np.int64)
    x = rng.standard_normal((cols, feat)).astype(np.float32)
    out = np.zeros((rows, feat), dtype=np.float32)
    ospmm.spmm(rowptr, pick.astype(np.int64), np.ones(rows, np.float32), x, out)
    assert np.array_equal(out, x[pick])


def test_threads_and_row_splits_do_not_change_results():
    a, x = _recipe(rows=3000, cols=700, density=0.01)
    base = np.zeros((a.shape[0], x.shape[1]), dtype=np.float32)
    ospmm.spmm(a.indptr, a.indices, a.data, x, base)
    for t in (2, 5):
        out = np.zeros_like(base)
        ospmm.spmm(a.indptr, a.indices, a.data, x, out, None, t)
        assert np.array_equal(out, base)
        rs = ospmm.distribute_work_for_row(a.indptr, np.ones_like(a.data), t)
        out = np.zeros_like(base)
        ospmm.spmm(a.indptr, a.indices, a.data, x, out, rs, t)
        assert np.array_equal(out, base)


@pytest.mark.parametrize("total,threads", [(0, 1), (1, 4), (10, 3), (12, 4), (1000, 7), (5, 8)])
def test_divide_work_closed_form(total, threads):
    got = ospmm.divide_work(total, threads)
    # brute force: hand out ceil(remaining / threads_left) one thread at a time
    expect, remain = [0], total
    for i in range(threads):
        chunk = -(-remain // (threads - i))
        expect.append(expect[-1] + chunk)
        remain -= chunk
    expect[-1] = total
    assert got.tolist() == expect
    assert got[0] == 0 and got[-1] == total and np.all(np.diff(got) >= 0)
    assert np.diff(got).max() - np.diff(got).min() <= 1


def test_distribute_work_for_row_hand_worked():
    # row weights (sum of values, all 1.0): [3, 1, 1, 3, 2, 2]; total 12; 3 threads -> target 4
    # running sum: 3, 4, 5>4 -> bound at row 2, restart at 1; 4, 6>4 -> bound at row 4, restart 2; 4
    rowptr = np.array([0, 3, 4, 5, 8, 10, 12], dtype=np.int64)
    val = np.ones(12, dtype=np.float32)
    assert ospmm.distribute_work_for_row(rowptr, val, 3).tolist() == [0, 2, 4, 6]
    # one thread: the running sum never exceeds the total -> [0, rows]
    assert ospmm.distribute_work_for_row(rowptr, val, 1).tolist() == [0, 6]
    # more threads than work: unset bounds stay at num_rows
    assert ospmm.distribute_work_for_row(np.array([0, 1, 2], dtype=np.int64), np.ones(2, np.float32), 4).tolist()[-1] == 2


# ---------------------------------------------------------------- against the reference's compiled op
@pytest.mark.parametrize("feat", [16, 47, 64, 100, 128, 256, 602])
def test_oracle_is_bit_identical_to_reference_op(reference_op, feat):
    import torch

    a, x = _recipe(rows=4099, cols=911, density=0.01, feat=feat, seed=100 + feat)
    rng = np.random.default_rng(feat)
    out0 = rng.standard_normal((a.shape[0], feat)).astype(np.float32)
    mine = out0.copy()
    ospmm.spmm(a.indptr, a.indices, a.data, x, mine)

    threads = torch.get_num_threads()
    rs = torch.from_numpy(ospmm.divide_work(a.shape[0], threads))
    cs = torch.tensor([0, feat], dtype=torch.int32)
    theirs = torch.from_numpy(out0.copy())
    ret = reference_op.spmm(torch.from_numpy(a.indptr.astype(np.int64)), torch.from_numpy(a.indices.astype(np.int64)),
                            torch.from_numpy(a.data), torch.from_numpy(x), theirs, a.shape[0], rs, cs)
    assert ret[1] is None and ret[0].data_ptr() == theirs.data_ptr()
    assert np.array_equal(mine, theirs.numpy())


def test_oracle_backward_is_bit_identical_to_reference_op(reference_op):
    import torch

    a, _ = _recipe(rows=3001, cols=1200, density=0.01, seed=7)
    rng = np.random.default_rng(8)
    g = rng.standard_normal((a.shape[0], 128)).astype(np.float32)
    colptr, row_t, val_t = ospmm.csr_transpose(a.indptr, a.indices, a.data, a.shape[1])
    mine = np.zeros((a.shape[1], 128), dtype=np.float32)
    ospmm.spmm(colptr, row_t, val_t, g, mine)
    threads = torch.get_num_threads()
    rs = torch.from_numpy(ospmm.divide_work(a.shape[1], threads))
    theirs = torch.zeros(a.shape[1], 128)
    reference_op.spmm(torch.from_numpy(colptr), torch.from_numpy(row_t), torch.from_numpy(val_t), torch.from_numpy(g),
                      theirs, a.shape[1], rs, torch.tensor([0, 128], dtype=torch.int32))
    assert np.array_equal(mine, theirs.numpy())


# ---------------------------------------------------------------- against committed reference outputs
def _golden_cases():
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "spmm_reference_op_vectors.npz")
    z = np.load(path)
    n = len({k.split("_")[0] for k in z.files})
    return [{name: z[f"c{i}_{name}"] for name in ("rowptr", "col", "val", "x", "out0", "out")} for i in range(n)]


def test_oracle_reproduces_committed_reference_outputs_bit_for_bit():
    # outputs of the reference's compiled operator (tests/golden/make_spmm_reference_vectors.py)
    for c in _golden_cases():
        got = c["out0"].copy()
        ospmm.spmm(c["rowptr"], c["col"], c["val"], c["x"], got)
        assert np.array_equal(got, c["out"])
