"""The hand-written set-up kernels of csrc/sort.hip through the C ABI: stable radix argsort and the run structure of
a list, against torch's host ops; and the index-map steps built on them (``data_manager.device_ops``)."""
import numpy as np
import pytest
import torch

from gnn_benchmark_amd.data_manager import device_ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 255, 256, 257, 2047, 2048, 2049, 4097, 8191, 8192, 8193, 16385, 65_537,
                               100_003, 1_000_003])
@pytest.mark.parametrize("span", [1, 5, 300, 70_000, 1 << 33, (1 << 62) + 12345])
def test_argsort_is_the_stable_ascending_order(n, span):
    """Few distinct keys (long runs of equal keys: stability), keys of 1 .. 8 radix passes, sizes around the tile and
    round boundaries of the scatter kernel."""
    rng = np.random.default_rng(n + span % 1000)
    x = torch.from_numpy(rng.integers(0, span, n, dtype=np.int64))
    want = torch.sort(x, stable=True).indices
    got = device_ops.stable_argsort(x.cuda())
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), want)


def test_argsort_takes_sorted_reversed_and_constant_input_and_refuses_negative_keys():
    n = 300_000
    for x in (torch.arange(n), torch.arange(n).flip(0), torch.zeros(n, dtype=torch.int64),
              torch.full((n,), (1 << 40) + 7, dtype=torch.int64), torch.arange(n) // 7):
        assert torch.equal(device_ops.stable_argsort(x.cuda()).cpu(), torch.sort(x, stable=True).indices)
    with pytest.raises(RuntimeError, match="non-negative"):
        device_ops.stable_argsort(torch.tensor([3, -1, 2]).cuda())


@pytest.mark.parametrize("n", [1, 2, 255, 2048, 2049, 100_003, 3_000_001])
@pytest.mark.parametrize("distinct", [1, 3, 1000, 10 ** 9])
def test_runs_equal_unique_consecutive(n, distinct):
    rng = np.random.default_rng(n % 977 + distinct % 13)
    x = torch.from_numpy(np.sort(rng.integers(0, distinct, n, dtype=np.int64)))
    values, inverse, counts = torch.unique_consecutive(x, return_inverse=True, return_counts=True)
    got = device_ops.runs(x.cuda())
    assert torch.equal(got[0].cpu(), values) and torch.equal(got[1].cpu(), inverse) and torch.equal(got[2].cpu(), counts)
    # unsorted input: runs of equal neighbours, not distinct values
    y = torch.from_numpy(rng.integers(0, 3, n, dtype=np.int64))
    values, inverse, counts = torch.unique_consecutive(y, return_inverse=True, return_counts=True)
    got = device_ops.runs(y.cuda())
    assert torch.equal(got[0].cpu(), values) and torch.equal(got[1].cpu(), inverse) and torch.equal(got[2].cpu(), counts)
    only = device_ops.runs(y.cuda(), want_inverse=False, want_counts=False)
    assert only[1] is None and only[2] is None and torch.equal(only[0].cpu(), values)


def test_runs_with_forced_starts_equal_the_host_form():
    """Segments across which equality is not carried (the per-rank restart of remap_remote_nodes_id)."""
    rng = np.random.default_rng(3)
    x = torch.from_numpy(np.sort(rng.integers(0, 50, 5000, dtype=np.int64)))
    starts = torch.tensor([0, 17, 17, 2500, 4999, 5000, -3, 99999])
    want = device_ops.runs(x, forced_starts=starts)          # host tensors: the torch form
    got = device_ops.runs(x.cuda(), forced_starts=starts)
    for a, b in zip(got, want):
        assert torch.equal(a.cpu(), b)
    assert int(want[0].shape[0]) > int(torch.unique_consecutive(x).shape[0])


@pytest.mark.parametrize("n", [1, 1000, 250_000])
def test_unique_and_occurrences_equal_torch(n):
    rng = np.random.default_rng(n)
    x = torch.from_numpy(rng.integers(0, max(2, n // 5), n, dtype=np.int64))
    assert torch.equal(device_ops.unique_sorted(x.cuda()).cpu(), torch.unique(x, sorted=True))
    _, inverse, counts = torch.unique(x, return_inverse=True, return_counts=True)
    assert torch.equal(device_ops.occurrences_per_entry(x.cuda()).cpu(), counts[inverse])


def test_calls_without_a_workspace_allocate_their_own_and_a_short_workspace_is_refused():
    import ctypes

    from gnn_benchmark_amd import _lib

    L = _lib.lib()
    n = 50_001
    x = torch.from_numpy(np.random.default_rng(5).integers(0, 900, n, dtype=np.int64)).cuda()
    perm, ordered = torch.empty_like(x), torch.empty_like(x)
    stream = _lib.current_stream(x.device)
    _lib.check(L.gnnagg_argsort_i64(_lib.ptr(x), n, _lib.ptr(perm), _lib.ptr(ordered), None, 0, stream))
    assert torch.equal(perm, device_ops.stable_argsort(x)) and torch.equal(ordered, x[perm])
    values, counts = torch.empty_like(x), torch.empty_like(x)
    found = ctypes.c_int64(0)
    _lib.check(L.gnnagg_runs_i64(_lib.ptr(ordered), n, None, 0, _lib.ptr(values), None, _lib.ptr(counts),
                                 ctypes.byref(found), None, 0, stream))
    want_values, want_counts = torch.unique_consecutive(ordered, return_counts=True)
    k = int(found.value)
    assert k == want_values.numel()
    assert torch.equal(values[:k], want_values) and torch.equal(counts[:k], want_counts)
    short = torch.empty(int(L.gnnagg_argsort_workspace_bytes(n)) - 256, dtype=torch.uint8, device="cuda")
    with pytest.raises(_lib.GnnAggError, match="workspace"):
        _lib.check(L.gnnagg_argsort_i64(_lib.ptr(x), n, _lib.ptr(perm), None, _lib.ptr(short), short.numel(), stream))
    with pytest.raises(_lib.GnnAggError, match="workspace"):
        _lib.check(L.gnnagg_runs_i64(_lib.ptr(ordered), n, None, 0, _lib.ptr(values), None, None, ctypes.byref(found),
                                     _lib.ptr(short), 64, stream))


@pytest.mark.parametrize("n,distinct", [(50_000_000, 1_000_003), (120_000_000, 1 << 46)])
def test_argsort_at_the_size_of_a_partitions_edge_list_is_sorted_stable_and_a_permutation(n, distinct):
    """Size-independent properties at the scale of config 4's edge lists (10^8 keys): the keys come out in
    non-decreasing order, equal keys in their input order, and every position occurs exactly once."""
    gen = torch.Generator(device="cuda").manual_seed(n % 1000)
    x = torch.randint(0, distinct, (n,), device="cuda", generator=gen, dtype=torch.int64)
    perm = device_ops.stable_argsort(x)
    ordered = x[perm]
    step = ordered[1:] - ordered[:-1]
    assert bool((step >= 0).all())
    assert bool((perm[1:][step == 0] > perm[:-1][step == 0]).all())          # stable
    del step, ordered
    seen = torch.zeros(n, dtype=torch.int8, device="cuda")
    seen[perm] = 1
    assert int(seen.sum(dtype=torch.int64)) == n and int(perm.min()) == 0 and int(perm.max()) == n - 1
