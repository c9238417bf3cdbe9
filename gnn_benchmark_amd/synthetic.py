"""Seeded synthetic graphs of the shapes the aggregation path is measured on.

There are no datasets on the box, so every workload is generated: random numbers come
from ``numpy.random.default_rng(seed)`` on the host (identical on every machine), the
heavy lifting (symmetrising, de-duplicating, sorting into CSR, the partition index
maps) runs on ``device`` with torch ops and libgnnagg.

Shapes follow the reference trainer's data: matrices are ``row = dst, col = src``
(self_benchmark/a64fx/data_manager/DataProcessor.py:104-116); a partition is described
by localised local edges, remote edges with global src / localised dst and the
``begin_node_on_each_partition`` prefix array (data_manager/DataLoader.py:12-40).
"""
from dataclasses import dataclass
from typing import Callable, List, Optional

import numpy as np
import torch

from .data_manager import (CommBuffer, DataProcessorForPreAggresive, get_distributed_graph,
                           get_distributed_graph_for_pre_aggressive)
from .sparse_tensor import SparseTensor


@dataclass
class SyntheticGraph:
    adj: SparseTensor
    num_nodes: int
    nnz: int
    max_degree: int
    description: str


def truncated_zipf(rng: np.random.Generator, n: int, s: float, kmax: int) -> np.ndarray:
    """n samples of P(k) ~ k^-s on {1..kmax} (inverse-CDF sampling)."""
    k = np.arange(1, kmax + 1, dtype=np.float64)
    cdf = np.cumsum(k ** (-s))
    cdf /= cdf[-1]
    return (np.searchsorted(cdf, rng.random(n), side="left") + 1).astype(np.int64)


def zipf_out_degrees(rng: np.random.Generator, n: int, s: float, mean: float, kmax: int) -> np.ndarray:
    """Zipf(s) out-degrees rescaled to the requested mean (stochastic rounding) and
    clipped to [0, kmax]."""
    z = truncated_zipf(rng, n, s, kmax).astype(np.float64)
    scaled = z * (mean / z.mean())
    deg = np.floor(scaled + rng.random(n)).astype(np.int64)
    return np.clip(deg, 0, kmax)


def _directed_edges(rng: np.random.Generator, out_deg: np.ndarray, num_targets: int, device):
    src = torch.repeat_interleave(torch.arange(out_deg.shape[0], dtype=torch.int64, device=device),
                                  torch.from_numpy(out_deg).to(device))
    dst = torch.from_numpy(rng.integers(0, num_targets, int(out_deg.sum()), dtype=np.int64)).to(device)
    return src, dst


def _csr_from_sorted_keys(keys: torch.Tensor, num_rows: int, num_cols: int):
    row = torch.div(keys, num_cols, rounding_mode="floor")
    col = keys - row * num_cols
    rowptr = torch.zeros(num_rows + 1, dtype=torch.int64, device=keys.device)
    rowptr[1:] = torch.cumsum(torch.bincount(row, minlength=num_rows), 0)
    return rowptr, row, col


def power_law_graph(num_nodes: int, mean_out_degree: float, zipf_s: float, max_degree: int, seed: int,
                    device="cuda", normalize: str = "gcn") -> SyntheticGraph:
    """Power-law graph: Zipf(s) out-degrees with the given mean, uniform endpoints,
    symmetrised, self-loops added, duplicates removed.  ``normalize="gcn"`` stores
    D^-1/2 (A+I) D^-1/2, ``"unit"`` stores ones (the reference's own matrices)."""
    rng = np.random.default_rng(seed)
    out_deg = zipf_out_degrees(rng, num_nodes, zipf_s, mean_out_degree, max_degree)
    src, dst = _directed_edges(rng, out_deg, num_nodes, device)
    loops = torch.arange(num_nodes, dtype=torch.int64, device=device)
    keys = torch.cat((dst * num_nodes + src, src * num_nodes + dst, loops * num_nodes + loops))
    del src, dst
    keys = torch.unique(keys)  # sorted: (row, col) order
    rowptr, row, col = _csr_from_sorted_keys(keys, num_nodes, num_nodes)
    del keys
    deg = rowptr[1:] - rowptr[:-1]
    if normalize == "gcn":
        value = (deg[row].double() * deg[col].double()).rsqrt().float()
    else:
        value = torch.ones(col.numel(), dtype=torch.float32, device=device)
    del row
    adj = SparseTensor(rowptr=rowptr, col=col, value=value, sparse_sizes=(num_nodes, num_nodes), is_sorted=True)
    return SyntheticGraph(adj, num_nodes, int(col.numel()), int(deg.max()),
                          f"power-law N={num_nodes} zipf_s={zipf_s} mean_out={mean_out_degree} seed={seed} {normalize}")


def dense_degree_graph(num_nodes: int, mu: float, sigma: float, seed: int, device="cuda") -> SyntheticGraph:
    """Load-balance stress: in-degrees ~ lognormal(mu, sigma), sources uniform, duplicates
    removed, row-normalised values (mean aggregation)."""
    rng = np.random.default_rng(seed)
    deg = np.clip(np.rint(rng.lognormal(mu, sigma, num_nodes)), 1, num_nodes).astype(np.int64)
    row, col = _directed_edges(rng, deg, num_nodes, device)
    keys = torch.unique(row * num_nodes + col)
    del row, col
    rowptr, row, col = _csr_from_sorted_keys(keys, num_nodes, num_nodes)
    del keys
    d = (rowptr[1:] - rowptr[:-1]).clamp(min=1)
    value = (1.0 / d[row].double()).float()
    del row
    adj = SparseTensor(rowptr=rowptr, col=col, value=value, sparse_sizes=(num_nodes, num_nodes), is_sorted=True)
    return SyntheticGraph(adj, num_nodes, int(col.numel()), int(d.max()),
                          f"lognormal({mu},{sigma}) in-degrees N={num_nodes} seed={seed} row-normalised")


# --------------------------------------------------------------------------- one partition of a partitioned graph
@dataclass
class PartitionData:
    """The in-memory form of one partition's files."""
    rank: int
    world_size: int
    begins: torch.Tensor          # [W+1] first global id of every partition (host)
    num_local_nodes: int
    local_edges: torch.Tensor     # [2, E_l] src, dst localised
    remote_edges: torch.Tensor    # [2, E_r] src global (other partitions), dst localised


def partition_edges(num_local_nodes: int, world_size: int, rank: int, local_mean_out_degree: float, zipf_s: float,
                    max_degree: int, num_halo_nodes: int, num_remote_edges: int, seed: int,
                    device="cuda") -> PartitionData:
    """One rank's share of a power-law graph split ``world_size`` ways, every partition
    ``num_local_nodes`` wide.  Local edges: symmetrised power-law graph with self-loops.
    Remote edges: ``num_halo_nodes`` distinct remote ids drawn uniformly over the other
    partitions; every remote edge picks a halo node and a local dst uniformly."""
    rng = np.random.default_rng(seed)
    n = num_local_nodes
    begins = torch.arange(world_size + 1, dtype=torch.int64) * n
    out_deg = zipf_out_degrees(rng, n, zipf_s, local_mean_out_degree, max_degree)
    src, dst = _directed_edges(rng, out_deg, n, device)
    loops = torch.arange(n, dtype=torch.int64, device=device)
    keys = torch.unique(torch.cat((dst * n + src, src * n + dst, loops * n + loops)))
    del src, dst
    l_dst = torch.div(keys, n, rounding_mode="floor")
    l_src = keys - l_dst * n
    del keys
    local_edges = torch.stack((l_src, l_dst))
    del l_src, l_dst

    # halo ids: uniform over the (W-1)*n remote ids, distinct
    others = (world_size - 1) * n
    halo = np.unique(rng.integers(0, others, int(num_halo_nodes * 1.02) + 16, dtype=np.int64))
    if halo.shape[0] > num_halo_nodes:
        halo = np.sort(rng.choice(halo, num_halo_nodes, replace=False))
    halo = np.where(halo >= rank * n, halo + n, halo)  # skip this rank's own id range
    pick = rng.integers(0, halo.shape[0], num_remote_edges, dtype=np.int64)
    r_src = torch.from_numpy(halo[pick]).to(device)
    r_dst = torch.from_numpy(rng.integers(0, n, num_remote_edges, dtype=np.int64)).to(device)
    rkeys = torch.unique(r_dst * (world_size * n) + r_src)  # no repeated remote edge
    r_dst = torch.div(rkeys, world_size * n, rounding_mode="floor")
    r_src = rkeys - r_dst * (world_size * n)
    remote_edges = torch.stack((r_src, r_dst))
    return PartitionData(rank, world_size, begins, n, local_edges, remote_edges)


def mirrored_graph_exchange(part: PartitionData) -> Callable[[List[torch.Tensor]], List[torch.Tensor]]:
    """Stand-in for the setup-time exchange of edge lists when only ONE partition exists.

    The graph is undirected, so peer i holds the reverse of every remote edge this rank
    holds from i.  What peer i would address to this rank is therefore computable here:
    run the reference's own classification (POST when out-degree(src) > in-degree(dst),
    data_manager/DataProcessor.py:228-248) and packing (:252-279) on the reversed edges
    from the peer's point of view."""
    begins = part.begins
    local_begin = int(begins[part.rank])

    def exchange(_sent_lists):
        g_src = part.remote_edges[0]                 # peer-owned global ids
        g_dst = part.remote_edges[1] + local_begin   # this rank's global ids
        received = []
        for i in range(part.world_size):
            sel = (g_src >= int(begins[i])) & (g_src < int(begins[i + 1]))
            # reversed: the peer aggregates INTO its node g_src FROM our node g_dst
            p_src, p_dst = g_dst[sel], g_src[sel]
            flags = DataProcessorForPreAggresive.decide_pre_or_post_aggr(p_src, p_dst, 1, 0)
            out: List[torch.Tensor] = []
            DataProcessorForPreAggresive.collect_edges_sent_to_other_subgraphs(p_src, p_dst, flags == 1, flags == 0, out)
            received.append(out[0])
        return received

    return exchange


class SeededHaloExchange:
    """Stand-in for the per-layer boundary all-to-all: on "forward" the receive buffer is
    filled with seeded N(0,1) rows generated on the device, on "backward" the send
    buffer is (those are the rows a real exchange would have delivered).  The fill is
    enqueued on the current stream; ``wait()`` is a no-op.  ``std`` / ``backward_std`` scale the
    rows (feature rows and gradient rows live on very different scales in a real run)."""

    def __init__(self, seed: int = 0, std: float = 1.0, backward_std: Optional[float] = None):
        self.seed = seed
        self.std = std
        self.backward_std = std if backward_std is None else backward_std
        self._gen = None
        self.calls: List[str] = []

    def __call__(self, comm_splits, comm_buf, tag: str, direction: str):
        buf = comm_buf.recv_buf if direction == "forward" else comm_buf.send_buf
        if self._gen is None or self._gen.device != buf.device:
            self._gen = torch.Generator(device=buf.device)
        # one reproducible stream of numbers per (layer tag)
        self._gen.manual_seed(self.seed * 1000003 + sum(ord(c) * (i + 1) for i, c in enumerate(tag)))
        buf.normal_(0.0, self.std if direction == "forward" else self.backward_std, generator=self._gen)
        self.calls.append(tag)
        return None


class _DeliveredInPlaceCommBuffer(CommBuffer):
    """A ``CommBuffer`` whose ``send_buf`` / ``recv_buf`` an exchange may point at rows that were delivered into
    memory of its own (a zero-copy receive).  ``resize_buffer`` -- the first thing the aggregator does in either
    direction (self_benchmark/a64fx/model/layers/aggregator.py:34, :133) -- hands the buffer's own tensors back, so
    whatever the aggregator writes goes to those and delivered rows are only ever read."""

    def __init__(self, inner: CommBuffer):
        self.__dict__.update(inner.__dict__)
        self._own = (inner.send_buf, inner.recv_buf, inner.send_buf_fp16, inner.recv_buf_fp16)

    def resize_buffer(self, comm_splits, feat_len: int, bits: int) -> None:
        self.send_buf, self.recv_buf, self.send_buf_fp16, self.recv_buf_fp16 = self._own
        super().resize_buffer(comm_splits, feat_len, bits)


class PregeneratedHaloExchange(SeededHaloExchange):
    """The same seeded rows as ``SeededHaloExchange``, drawn ONCE per (tag, shape) and kept on the device; a call
    points the receiving buffer at them (``attach`` gives the graph a buffer object that allows it).  Nothing is
    enqueued inside a timed step: no random-number kernels, no copy -- the stand-in for an exchange whose rows have
    arrived in their own memory by the time the aggregator waits for them."""

    def __init__(self, seed: int = 0, std: float = 1.0, backward_std: Optional[float] = None):
        super().__init__(seed, std, backward_std)
        self._rows = {}

    @staticmethod
    def attach(graph):
        if not isinstance(graph.comm_buf, _DeliveredInPlaceCommBuffer):
            graph.comm_buf = _DeliveredInPlaceCommBuffer(graph.comm_buf)
        return graph

    def __call__(self, comm_splits, comm_buf, tag: str, direction: str):
        if not isinstance(comm_buf, _DeliveredInPlaceCommBuffer):
            raise RuntimeError("PregeneratedHaloExchange needs PregeneratedHaloExchange.attach(graph) first")
        buf = comm_buf.recv_buf if direction == "forward" else comm_buf.send_buf
        key = (tag, tuple(buf.shape), str(buf.device))
        rows = self._rows.get(key)
        if rows is None:
            super().__call__(comm_splits, comm_buf, tag, direction)   # fills buf with the seeded rows
            rows = self._rows[key] = buf.clone()
        else:
            self.calls.append(tag)
        if direction == "forward":
            comm_buf.recv_buf = rows
        else:
            comm_buf.send_buf = rows
        return None


class SeededQuantizedHaloExchange:
    """Quantised counterpart of SeededHaloExchange: the packed rows and the (zero_point, scale)
    rows a real exchange would have delivered are seeded random bytes and seeded parameters
    (already rounded through bf16, as they are on the wire), generated on the device."""

    def __init__(self, seed: int = 0):
        self.seed = seed
        self._gen = None
        self.calls: List[str] = []

    def __call__(self, comm_splits, qbuf, tag: str, direction: str):
        data = qbuf.quantized_recv_data_buf if direction == "forward" else qbuf.quantized_send_data_buf
        params = qbuf.quantized_recv_params_buf_fp32 if direction == "forward" else qbuf.quantized_send_params_buf_fp32
        if self._gen is None or self._gen.device != data.device:
            self._gen = torch.Generator(device=data.device)
        self._gen.manual_seed(self.seed * 1000003 + 7 + sum(ord(c) * (i + 1) for i, c in enumerate(tag)))
        data.random_(0, 256, generator=self._gen)
        params.normal_(generator=self._gen)
        params[:, 1].abs_().add_(0.05)
        params.copy_(params.to(torch.bfloat16))
        self.calls.append(tag)
        return None


class PregeneratedQuantizedHaloExchange(SeededQuantizedHaloExchange):
    """The same seeded packed rows and parameters, drawn once per (tag, shape) and kept on the device; a later call
    copies them into the receiving buffers (a device copy of the packed bytes, 1/16 of the fp32 rows at 2 bits) instead
    of running the random-number kernels inside a timed step."""

    def __init__(self, seed: int = 0):
        super().__init__(seed)
        self._kept = {}

    def __call__(self, comm_splits, qbuf, tag: str, direction: str):
        data = qbuf.quantized_recv_data_buf if direction == "forward" else qbuf.quantized_send_data_buf
        params = qbuf.quantized_recv_params_buf_fp32 if direction == "forward" else qbuf.quantized_send_params_buf_fp32
        key = (tag, tuple(data.shape), tuple(params.shape), str(data.device))
        kept = self._kept.get(key)
        if kept is None:
            super().__call__(comm_splits, qbuf, tag, direction)
            self._kept[key] = (data.clone(), params.clone())
        else:
            data.copy_(kept[0])
            params.copy_(kept[1])
            self.calls.append(tag)
        return None


class SeededBf16HaloExchange:
    """bf16 counterpart of SeededHaloExchange: fills the bf16 staging copy the aggregator widens."""

    def __init__(self, seed: int = 0):
        self.seed = seed
        self._gen = None
        self.calls: List[str] = []

    def __call__(self, comm_splits, comm_buf, tag: str, direction: str):
        target = comm_buf.recv_buf_fp16 if direction == "forward" else comm_buf.send_buf_fp16
        if self._gen is None or self._gen.device != target.device:
            self._gen = torch.Generator(device=target.device)
        self._gen.manual_seed(self.seed * 1000003 + 11 + sum(ord(c) * (i + 1) for i, c in enumerate(tag)))
        target.normal_(generator=self._gen)
        self.calls.append(tag)
        return None


class PregeneratedBf16HaloExchange(SeededBf16HaloExchange):
    """bf16 counterpart of ``PregeneratedHaloExchange``: the seeded bf16 rows are drawn once per (tag, shape) and a
    call points the receiving staging buffer at them, so nothing is enqueued inside a timed step."""

    def __init__(self, seed: int = 0):
        super().__init__(seed)
        self._rows = {}

    def __call__(self, comm_splits, comm_buf, tag: str, direction: str):
        if not isinstance(comm_buf, _DeliveredInPlaceCommBuffer):
            raise RuntimeError("PregeneratedBf16HaloExchange needs PregeneratedHaloExchange.attach(graph) first")
        buf = comm_buf.recv_buf_fp16 if direction == "forward" else comm_buf.send_buf_fp16
        key = (tag, tuple(buf.shape), str(buf.device))
        rows = self._rows.get(key)
        if rows is None:
            super().__call__(comm_splits, comm_buf, tag, direction)
            rows = self._rows[key] = buf.clone()
        else:
            self.calls.append(tag)
        if direction == "forward":
            comm_buf.recv_buf_fp16 = rows
        else:
            comm_buf.send_buf_fp16 = rows
        return None


def build_partition_graph(part: PartitionData, max_feat_len: int, is_pre_delay: bool,
                          exchange: Optional[Callable] = None, bits: int = 32, device="cuda",
                          exchange_quantized: Optional[Callable] = None, exchange_bf16: Optional[Callable] = None):
    """DistributedGraphForPre (pre/post-aggregation) or DistributedGraph (raw halo rows) of
    one synthetic partition."""
    local_edges = part.local_edges.clone()
    remote_edges = part.remote_edges.clone()
    if isinstance(exchange, PregeneratedHaloExchange):
        built = build_partition_graph(part, max_feat_len, is_pre_delay, None, bits, device, exchange_quantized,
                                      exchange_bf16)
        built.exchange = exchange
        return PregeneratedHaloExchange.attach(built)
    if is_pre_delay:
        return get_distributed_graph_for_pre_aggressive(
            local_edges, remote_edges, part.begins, part.num_local_nodes, max_feat_len, part.rank, part.world_size,
            bits, graph_exchange=mirrored_graph_exchange(part), exchange=exchange,
            exchange_quantized=exchange_quantized, exchange_bf16=exchange_bf16, device=device)
    begin = int(part.begins[part.rank])
    local_nodes_list = torch.stack((torch.arange(begin, begin + part.num_local_nodes), ) * 2, dim=1)

    def halo_id_exchange(_send_lists):
        # undirected graph: peer i asks for exactly the local nodes adjacent to its nodes
        g_src, l_dst = part.remote_edges[0], part.remote_edges[1]
        out = []
        for i in range(part.world_size):
            sel = (g_src >= int(part.begins[i])) & (g_src < int(part.begins[i + 1]))
            out.append(torch.unique(l_dst[sel]) + begin)
        return out

    return get_distributed_graph(local_edges, remote_edges, local_nodes_list, part.begins, part.num_local_nodes,
                                 max_feat_len, part.world_size, bits, halo_id_exchange=halo_id_exchange,
                                 exchange=exchange, exchange_quantized=exchange_quantized, exchange_bf16=exchange_bf16,
                                 device=device)
