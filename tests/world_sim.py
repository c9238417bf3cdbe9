"""Test helper (not collected): a small partitioned world held in one process.

Builds a seeded undirected graph, cuts it into W contiguous partitions with the file
contract of the reference (local edges localised; remote edges with global src and
localised dst; ``begins`` prefix array), and provides the global matrix for the
all-ranks invariant."""
import numpy as np


class World:
    def __init__(self, seed, sizes, mean_deg=5.0, hub_frac=0.05, self_loops=True):
        rng = np.random.default_rng(seed)
        self.sizes = np.asarray(sizes, dtype=np.int64)
        self.world = len(sizes)
        self.begins = np.concatenate(([0], np.cumsum(self.sizes))).astype(np.int64)
        n = int(self.begins[-1])
        self.n = n
        e = int(n * mean_deg / 2)
        # a few hubs so that both PRE and POST edges occur between every pair of ranks
        hubs = rng.choice(n, max(1, int(n * hub_frac)), replace=False)
        src = np.where(rng.random(e) < 0.5, rng.choice(hubs, e), rng.integers(0, n, e))
        dst = rng.integers(0, n, e)
        s = np.concatenate((src, dst, np.arange(n) if self_loops else np.zeros(0, np.int64)))
        d = np.concatenate((dst, src, np.arange(n) if self_loops else np.zeros(0, np.int64)))
        key = np.unique(d.astype(np.int64) * n + s.astype(np.int64))
        self.dst = key // n   # row
        self.src = key % n    # col
        self.owner = np.searchsorted(self.begins, np.arange(n), side="right") - 1

    def partition(self, rank):
        """(local_edges [2,El], remote_edges [2,Er]) of one rank: edges whose dst it owns."""
        b, e = self.begins[rank], self.begins[rank + 1]
        mine = (self.dst >= b) & (self.dst < e)
        s, d = self.src[mine], self.dst[mine] - b
        is_local = (s >= b) & (s < e)
        local = np.stack((s[is_local] - b, d[is_local])).astype(np.int64)
        remote = np.stack((s[~is_local], d[~is_local])).astype(np.int64)
        return local, remote

    def global_product(self, x, transposed=False):
        """A @ x (or A.T @ x) in fp64 with unit values, A[dst, src] = 1."""
        out = np.zeros((self.n, x.shape[1]), dtype=np.float64)
        if transposed:
            np.add.at(out, self.src, x[self.dst].astype(np.float64))
        else:
            np.add.at(out, self.dst, x[self.src].astype(np.float64))
        return out
