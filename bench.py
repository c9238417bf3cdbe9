#!/usr/bin/env python3
"""Benchmark of the aggregation hot path on ONE MI355X.

Headline workload ("c2"): standalone CSR SpMM forward A @ X plus the transposed backward
A^T @ G on a seeded power-law graph of 2.45 M nodes / ~122 M stored elements with
GCN-normalised fp32 values and a 2.45 M x 100 fp32 dense operand.  One "step" is one
forward plus one backward, with every input already resident in HBM.

Prints ONE compact JSON line on stdout (a few KB), last.  ``value`` is the FLOP rate of the whole
step (2 * nnz * F per product).  ``roofline`` prices the dominant kernel (the forward's row
kernel) against the 8 TB/s HBM peak with the no-reuse gather byte model
    bytes = nnz*(8+4) + (rows+1)*8 + nnz*F*4 + 2*rows*F*4
over the rows / stored elements that launch covers, divided by its duration measured
with HIP events on the launch stream inside the timed region.  ``cpu_baseline`` is the
reference's own compiled operator (or the C port of it when that cannot run on the
host) timed on this machine's cores on the same matrices.  ``parity`` is the gate in front of
the number: the GPU results of the headline operands (and, when c4 runs, of a seeded row sample
of the partition's pipeline) against that CPU operator, rel 1e-5 / abs 1e-6; a failure exits
non-zero and prints no value.  ``targets`` summarises the partition workload: the six products of
the pipeline as a fraction of the HBM peak, and the train steps.

The other workloads run after the timed headline: c1 (the single-rank 2-layer GCN forward +
backward, with the same step on the host cores beside it), c2 at other widths, c3 (dense-degree
mean aggregation, F=602/256), c4 (one partition of a 16-way split: pre-aggregation, local SpMM,
post-aggregation, F=128) and c5 (3-layer GCN train step and the reference's 3-layer SAGE model
on the c4 partition).  Their full reports do not go into the stdout line: each is written, as
soon as its workload has finished, as one JSON line to stderr and into the side file
``--extra-out`` (default bench_out/bench_extra.json), so a late failure loses nothing.
``--only headline`` skips them.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
MAX_LINE_BYTES = 6000   # the stdout line stays a few KB: everything else goes to the side file and stderr


def _finite(obj):
    """`obj` with non-finite floats replaced by their names (strict JSON has no NaN / Infinity)."""
    if isinstance(obj, float):
        return obj if obj == obj and abs(obj) != float("inf") else str(obj)
    if isinstance(obj, dict):
        return {k: _finite(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [_finite(v) for v in obj]
    return obj


class ExtraSink:
    """Full reports of the workloads besides the headline: each goes to stderr as one JSON line and into the side
    file (rewritten whole, atomically) the moment its workload has finished."""

    def __init__(self, path):
        self.path, self.data, self.keys, self.failed = path, {}, [], None

    def put(self, key, value):
        value = _finite(value)
        self.data[key] = value
        self.keys.append(key)
        print(json.dumps({"extra": key, "report": value}, allow_nan=False), file=sys.stderr, flush=True)
        if self.path:
            try:
                os.makedirs(os.path.dirname(os.path.abspath(self.path)), exist_ok=True)
                with open(self.path + ".tmp", "w") as f:
                    json.dump(self.data, f, allow_nan=False, indent=1)
                os.replace(self.path + ".tmp", self.path)
            except OSError as e:  # a read-only tree: stderr still has everything
                self.failed = str(e)
        return value

    def where(self):
        if not self.path or self.failed:
            return "stderr only" + (f" ({self.failed})" if self.failed else "")
        return os.path.relpath(self.path, ROOT)


def c4_targets(c4):
    """The compact summary of the partition workload for the stdout line: per product of the pipeline, as the
    Aggregator runs it, [ms, fraction of the HBM peak on the model bytes, the same on the measured bytes (or null)];
    and the whole autograd.Function."""
    short = {"pre-aggregation A_to@X -> send_buf": "pre", "local A_local@X -> out": "local",
             "post-aggregation A_from@recv_buf -> out": "post", "pre-aggregation transposed": "pre_T",
             "local transposed": "local_T", "post-aggregation transposed": "post_T"}
    products = {}
    for op in c4["ops"]:
        if op.get("as_run_by_aggregator") is not True:
            continue
        name = next((v for k, v in short.items() if op["op"].startswith(k)), None)
        if name is not None:
            products[name] = [op["ms"], op["frac_model"], op.get("frac_measured")]
    out = {"products_ms_fracmodel_fracmeasured": products, "feat": c4["feat"],
           "min_frac_model": min((v[1] for v in products.values()), default=None)}
    for k in ("aggregator_forward_ms", "aggregator_forward_backward_ms", "aggregator_forward_ms_one_launch",
              "aggregator_forward_backward_ms_one_launch", "aggregator_forward_backward_ms_int2_exchange",
              "aggregator_forward_backward_ms_int2_exchange_one_launch"):
        if k in c4:
            out[k] = c4[k]
    return out

# HBM-side traffic of ONE launch, measured with rocprofv3 --pmc on this file's own workloads (default sizes and
# seed): bytes read = 32 / 64 / 128-byte read requests of the L2 to the memory side, counted by size
# (TCC_EA0_RDREQ_32B / _64B / _128B; on this GPU practically all are 128-byte requests), bytes written =
# WRITE_SIZE.  "Memory side" is what lies behind the L2: HBM and the 256 MB memory-side cache in front of it, which
# these counters cannot tell apart.  (workload, op, F) -> (bytes read, bytes written,
# the summary under profiles/ that holds the counter readings and the commands).  These are constants taken from
# those profile runs, not something a timed run can produce (the counters need the profiler): the JSON labels
# them "profile".  Any other size or seed: no entry, and the measured fields are left out.
_P = "profiles/spmm_memory_traffic_c2_c3_c4.md"
MEASURED_TRAFFIC = {
    ("c2", "A@X", 100): (5.68207e+10, 1.01207e+09, _P), ("c2", "A^T@G", 100): (5.68207e+10, 1.01207e+09, _P),
    ("c2", "A@X", 128): (5.71924e+10, 1.25440e+09, _P), ("c2", "A^T@G", 128): (5.71924e+10, 1.25440e+09, _P),
    ("c2", "A@X", 256): (1.18675e+11, 2.50880e+09, _P), ("c2", "A^T@G", 256): (1.18675e+11, 2.50880e+09, _P),
    ("c2", "A@X", 172): (9.10710e+10, 1.73200e+09, _P), ("c2", "A^T@G", 172): (9.10710e+10, 1.73200e+09, _P),
    ("c2", "A@X", 40): (2.72050e+10, 4.00000e+08, _P), ("c2", "A^T@G", 40): (2.72050e+10, 4.00000e+08, _P),
    ("c2", "A@X", 47): (3.31340e+10, 5.38000e+08, _P), ("c2", "A^T@G", 47): (3.31340e+10, 5.38000e+08, _P),
    # (c3: the block-per-row kernel's share, 0.8 / 0.3 GB, is included in the forward figures)
    ("c3", "A@X", 602): (2.94247e+11, 5.82812e+08, _P), ("c3", "A^T@G", 602): (2.85891e+11, 5.91882e+08, _P),
    ("c3", "A@X", 256): (1.18438e+11, 2.38592e+08, _P), ("c3", "A^T@G", 256): (1.12242e+11, 2.38592e+08, _P),
    ("c4", "pre", 128): (1.22851e+10, 1.53568e+09, _P), ("c4", "pre_overwrite", 128): (1.07445e+10, 1.53568e+09, _P),
    ("c4", "pre_T", 128): (1.43904e+10, 3.37825e+09, _P), ("c4", "pre_T_overwrite", 128): (1.10097e+10, 3.58400e+09, _P),
    ("c4", "local", 128): (5.48747e+10, 3.58400e+09, _P), ("c4", "local_overwrite", 128): (5.12406e+10, 3.58400e+09, _P),
    ("c4", "local_T", 128): (5.48742e+10, 3.58400e+09, _P), ("c4", "local_T_overwrite", 128): (5.12387e+10, 3.58400e+09, _P),
    ("c4", "post", 128): (1.43898e+10, 3.37825e+09, _P), ("c4", "post_overwrite", 128): (1.10093e+10, 3.58400e+09, _P),
    ("c4", "post_T", 128): (1.22983e+10, 1.55268e+09, _P), ("c4", "post_T_overwrite", 128): (1.07407e+10, 1.55268e+09, _P),
    ("c4", "local_planless", 128): (5.50780e+10, 3.58400e+09, _P),
    ("c4", "local+post", 128): (6.22570e+10, 3.58400e+09, _P), ("c4", "local_T+pre_T", 128): (6.22570e+10, 3.58400e+09, _P),
}


def measured_traffic(args, workload, op, feat):
    """(read bytes, written bytes, source) of one launch from MEASURED_TRAFFIC, or None when the run's sizes are
    not the ones the profiles were taken at."""
    if (args.nodes, args.mean_out_degree, args.c4_nodes, args.seed) != (2_450_000, 25.0, 7_000_000, 0):
        return None
    return MEASURED_TRAFFIC.get((workload, op, feat))


def host_cpu():
    """(model name, physical cores, logical CPUs) of the host, from /proc/cpuinfo."""
    model, cores, logical = "unknown", set(), 0
    try:
        with open("/proc/cpuinfo") as f:
            phys = core = None
            for line in f:
                key, _, val = line.partition(":")
                key, val = key.strip(), val.strip()
                if key == "processor":
                    logical += 1
                elif key == "model name":
                    model = val
                elif key == "physical id":
                    phys = val
                elif key == "core id":
                    core = val
                elif not key and phys is not None:
                    cores.add((phys, core))
                    phys = core = None
            if phys is not None:
                cores.add((phys, core))
    except OSError:
        pass
    return model, (len(cores) or logical), logical


def cpu_median_seconds(run, warmups=2, reps=5):
    """Median wall time of `run` over `reps` calls after `warmups` untimed ones."""
    for _ in range(warmups):
        run()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2]


def b_alg(nnz: int, rows: int, feat: int, overwrite_rows: int = None) -> float:
    """Algorithmic bytes of one call (no-reuse gather model).  out += A @ X over `rows` visited rows: per stored
    element an int64 column index, an fp32 value and one F-wide fp32 row; per row its rowptr entry and the read and
    write of its output row.  With `overwrite_rows` (out = A @ X: nothing is read from out, and every one of those
    rows is written, the ones without stored elements as zeros) the output side is one write per row."""
    if overwrite_rows is not None:
        return nnz * 12.0 + (overwrite_rows + 1) * 8.0 + nnz * feat * 4.0 + overwrite_rows * feat * 4.0
    return nnz * 12.0 + (rows + 1) * 8.0 + nnz * feat * 4.0 + 2.0 * rows * feat * 4.0


def b_min(nnz: int, rows: int, cols: int, feat: int) -> float:
    """Compulsory floor: the dense operand read once."""
    return nnz * 12.0 + (rows + 1) * 8.0 + cols * feat * 4.0 + 2.0 * rows * feat * 4.0


def time_plan(plan, value, x, out, steps, warmup, accumulate=True):
    """Mean dominant-kernel and whole-call durations (ms) over `steps` calls, HIP events."""
    plan.profile(True)
    k_ms, c_ms = [], []
    for i in range(warmup + steps):
        plan.spmm(value, x, out, accumulate=accumulate)
        k, c = plan.profile_read()
        if i >= warmup:
            k_ms.append(k)
            c_ms.append(c)
    plan.profile(False)
    return sum(k_ms) / len(k_ms), sum(c_ms) / len(c_ms)


def op_report(name, nnz, rows, cols, feat, ms, empty_rows=0, accumulate=True, measured=None):
    """Rates of one call.  `frac_model` prices the MODEL bytes (no-reuse gather: every stored element fetches a
    whole dense row) against the 8 TB/s HBM peak; where gathered rows are re-read out of L2 or the 256 MB
    memory-side cache the model counts bytes HBM never moved, so it can exceed 1 and is not an HBM fraction.
    `frac_measured` prices the traffic the counters saw on the memory side of the L2 (`measured`: bytes read,
    bytes written, profile) in the time measured here.  Accumulate calls neither read nor write rows without
    stored elements; overwrite calls write every row."""
    rows_total, rows = rows, rows - empty_rows
    model = b_alg(nnz, rows, feat) if accumulate else b_alg(nnz, rows, feat, overwrite_rows=rows_total)
    gbs = model / (ms * 1e-3) / 1e9
    r = {"op": name, "rows": rows_total, "rows_visited": rows if accumulate else rows_total, "cols": cols, "nnz": nnz,
         "feat": feat, "accumulate": bool(accumulate), "ms": round(ms, 4),
         "gflops": round(2.0 * nnz * feat / (ms * 1e-3) / 1e9, 1), "bytes_model": model, "gbs_model": round(gbs, 1),
         "frac_model": round(gbs / HBM_PEAK_GBS, 4),
         "gbs_floor": round(b_min(nnz, rows, cols, feat) / (ms * 1e-3) / 1e9, 1)}
    if measured is not None:
        rd, wr, source = measured
        r["traffic_measured"] = {"read_bytes": rd, "written_bytes": wr, "kind": "profile", "source": source}
        r["gbs_measured"] = round((rd + wr) / (ms * 1e-3) / 1e9, 1)
        r["frac_measured"] = round((rd + wr) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    return r


def cpu_operator(threads):
    """``run(rowptr, col, val, x, out, row_split)`` doing one out += A @ x on the host cores: the reference's own
    compiled operator when oracle/_ref holds it and the host has AVX-512 (kind "reference"), else the C port of it
    (kind "port")."""
    import torch

    from oracle import spmm as ospmm

    ref = ospmm.load_reference_op()
    if ref is not None:
        torch.set_num_threads(threads)

        def run(rowptr, col, val, x, out, row_split):
            t = torch.from_numpy
            ref.spmm(t(rowptr), t(col), t(val), t(x), t(out), rowptr.shape[0] - 1, t(row_split),
                     torch.tensor([0, x.shape[1]], dtype=torch.int32))

        return run, "reference"

    def run(rowptr, col, val, x, out, row_split):
        ospmm.spmm(rowptr, col, val, x, out, row_split, threads)

    return run, "port"


def cpu_description(kind, threads):
    model, physical, logical = host_cpu()
    return {"kind": kind, "cores": int(threads), "threads": int(threads), "host_physical_cores": physical,
            "host_logical_cpus": logical, "cpu_model": model,
            "protocol": "median of 5 timed calls after 2 warm-ups, OpenMP threads = the host share given to this job"}


PARITY_REL, PARITY_ABS = 1e-5, 1e-6  # the gate's tolerance: |gpu - cpu| <= ABS + REL * |cpu|


def parity_excess(got, want):
    """(worst |got - want| - (ABS + REL * |want|), bit-identical?) of two fp32 arrays, in slabs."""
    import numpy as np

    assert got.shape == want.shape, (got.shape, want.shape)
    worst, same = -PARITY_ABS, True
    step = max(1, (1 << 24) // max(1, got.shape[1]))
    for lo in range(0, got.shape[0], step):
        a, b = got[lo:lo + step].astype(np.float64), want[lo:lo + step].astype(np.float64)
        if not np.isfinite(a).all():
            return float("inf"), False
        worst = max(worst, float((np.abs(a - b) - (PARITY_ABS + PARITY_REL * np.abs(b))).max(initial=-1.0)))
        same = same and bool(np.array_equal(got[lo:lo + step], want[lo:lo + step]))
    return worst, same


class ParityGate:
    """Collects the comparisons of GPU results with the CPU operator; `record` exits the process (status 4, nothing
    on stdout) on the first one outside the tolerance -- no number is printed for results that differ."""

    def __init__(self, enabled):
        self.enabled, self.cases, self.kind = enabled, {}, None

    def record(self, name, got, want, what):
        excess, same = parity_excess(got, want)
        self.cases[name] = {"what": what, "max_excess": float(f"{excess:.3e}"), "bit_identical": same,
                            "pass": excess <= 0.0}
        print(json.dumps({"parity": name, **self.cases[name]}), file=sys.stderr, flush=True)
        if not excess <= 0.0:
            print(f"bench.py: parity gate FAILED for {name} ({what}): worst excess over abs {PARITY_ABS} + rel "
                  f"{PARITY_REL} is {excess:.3e}; no number is reported", file=sys.stderr, flush=True)
            sys.exit(4)

    def report(self):
        if not self.enabled:
            return {"checked": False}
        return {"checked": bool(self.cases), "tolerance": f"abs {PARITY_ABS} + rel {PARITY_REL}",
                "against": f"CPU operator ({self.kind})",
                "max_excess": max((c["max_excess"] for c in self.cases.values()), default=None),
                "bit_identical": all(c["bit_identical"] for c in self.cases.values()),
                "cases": {k: [c["max_excess"], c["bit_identical"]] for k, c in self.cases.items()}}


def cpu_baseline_spmm(src, x_host, g_host, gate=None, gpu_results=None, timed=True):
    """Forward + transposed backward of the headline workload on the host cores.  The first, fresh pair of results
    (onto zeros) is what the parity gate compares the GPU's `gpu_results` = (A @ X, A^T @ G) with, as the reference's
    own test does (tests/test_spmm.py:93-115); the timed calls follow."""
    import numpy as np

    from oracle import spmm as ospmm

    threads = ospmm.max_threads()
    run, kind = cpu_operator(threads)
    rowptr, col, val = [t.cpu().numpy() for t in src.csr()]
    colptr = src.storage.colptr().cpu().numpy()
    row_t = src.storage.row_T().cpu().numpy()
    val_t = src.storage.value_T().cpu().numpy()
    rows, cols = src.sparse_sizes()
    feat = x_host.shape[1]
    # the reference balances its threads on per-row work (model/ops/spmm_kernel.py:7-28); unit weights = nnz
    rs_f = ospmm.distribute_work_for_row(rowptr, np.ones(col.shape[0], np.float32), threads)
    rs_b = ospmm.distribute_work_for_row(colptr, np.ones(col.shape[0], np.float32), threads)
    out_f = np.zeros((rows, feat), dtype=np.float32)
    out_b = np.zeros((cols, feat), dtype=np.float32)

    def step():
        run(rowptr, col, val, x_host, out_f, rs_f)
        run(colptr, row_t, val_t, g_host, out_b, rs_b)

    if gate is not None and gate.enabled:
        step()
        gate.kind = f"{kind}, {threads} threads"
        gate.record("c2_forward", gpu_results[0], out_f, f"A@X, all {rows} rows, F={feat}")
        gate.record("c2_backward", gpu_results[1], out_b, f"A^T@G, all {cols} rows, F={feat}")
    if not timed:
        return None
    sec = cpu_median_seconds(step)
    flops = 2 * 2.0 * col.shape[0] * feat
    r = {"value": round(flops / sec / 1e9, 3), "unit": "GFLOP/s"}
    r.update(cpu_description(kind, threads))
    r["sample"] = f"the whole workload: 1 forward + 1 transposed backward per step, F={feat} (7 steps, about 2 s)"
    r["ms_per_step"] = round(sec * 1e3, 2)
    return r


def parity_rows_of_pipeline(gate, graph, x, out, recv_buf, n_sample, seed):
    """Gate for the partition workload: rows of `out` = A_local @ x + A_from @ recv_buf (the Aggregator's forward)
    for a seeded sample of rows plus the 64 longest, against the CPU operator run on those rows' own slices of the
    two matrices -- local elements first, then the received ones, the order the reference accumulates in
    (model/layers/aggregator.py:67-104)."""
    import numpy as np
    import torch

    from oracle import spmm as ospmm

    threads = ospmm.max_threads()
    run, kind = cpu_operator(threads)
    gate.kind = gate.kind or f"{kind}, {threads} threads"
    rp_l = graph.local_adj_t.csr()[0]
    deg = (rp_l[1:] - rp_l[:-1]).cpu().numpy()
    n = deg.shape[0]
    pick = np.unique(np.concatenate([np.argsort(deg)[-64:], np.random.default_rng(seed).integers(0, n, n_sample)]))
    want = np.zeros((pick.shape[0], x.shape[1]), dtype=np.float32)
    for m, operand in ((graph.local_adj_t, x), (graph.adj_t_pre_post_aggr_from, recv_buf)):
        rowptr, col, val = m.csr()
        rp = rowptr.cpu().numpy()
        lens = rp[pick + 1] - rp[pick]
        take = torch.from_numpy(np.concatenate([np.arange(rp[r], rp[r + 1]) for r in pick] + [np.zeros(0, np.int64)]))
        take = take.to(col.device)
        sub_ptr = np.concatenate(([0], np.cumsum(lens))).astype(np.int64)
        sub_col, sub_val = col[take].cpu().numpy(), val[take].cpu().numpy()
        # only the operand rows the sample touches travel to the host
        used, inverse = np.unique(sub_col, return_inverse=True)
        operand_host = operand[torch.from_numpy(used).to(operand.device)].cpu().numpy()
        rs = ospmm.distribute_work_for_row(sub_ptr, np.ones(sub_col.shape[0], np.float32), threads)
        run(sub_ptr, inverse.astype(np.int64), sub_val, operand_host, want, rs)
    got = out[torch.from_numpy(pick).to(out.device)].cpu().numpy()
    gate.record("c4_aggregator_forward_rows", got, want,
                f"A_local@X + A_from@recv_buf, {pick.shape[0]} sampled rows incl. the 64 longest, F={x.shape[1]}")


def cpu_time_product(rowptr, col, val, x_host, rows):
    """Median seconds of one out += A @ x on the host cores, which operator ran, and the thread count."""
    import numpy as np

    from oracle import spmm as ospmm

    threads = ospmm.max_threads()
    run, kind = cpu_operator(threads)
    rs = ospmm.distribute_work_for_row(rowptr, np.ones(col.shape[0], np.float32), threads)
    out = np.zeros((rows, x_host.shape[1]), dtype=np.float32)
    return cpu_median_seconds(lambda: run(rowptr, col, val, x_host, out, rs)), kind, threads


def time_planless(src, x, out, steps, warmup=2):
    """Mean ms of ``computation_ops.spmm`` of the compiled extension module -- the literal export of the reference's
    op (ops.cpp:23): rows in their natural order, int64 column indices, no cached plan -- on the launch stream."""
    import torch

    from gnn_benchmark_amd import ext

    computation_ops = ext.load()  # the compiled pybind11 module, as the reference's wrapper would import it
    rowptr, col, val = src.csr()
    empty = torch.empty(0, dtype=torch.int32, device=x.device)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(warmup + steps):
        if i == warmup:
            e0.record()
        computation_ops.spmm(rowptr, col, val, x, out, src.sparse_size(0), empty, empty)
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / steps


def spmm_pair(src, feat, steps, warmup, gen, args=None, workload=None, planless=False):
    """Times `steps` (forward + transposed backward) steps; returns (report, x, g)."""
    import torch

    rows, cols = src.sparse_sizes()
    nnz = src.nnz()
    dev = src.device
    plan_f, plan_b = src.get_plan(), src.get_plan_for_transpose()
    val, val_t = src.csr()[2], src.storage.value_T()
    x = torch.randn(cols, feat, device=dev, generator=gen)
    g = torch.randn(rows, feat, device=dev, generator=gen)
    out = torch.zeros(rows, feat, device=dev)
    dx = torch.zeros(cols, feat, device=dev)
    for _ in range(warmup):
        plan_f.spmm(val, x, out, True)
        plan_b.spmm(val_t, g, dx, True)
    plan_f.profile(True)
    k_ms = []
    torch.cuda.synchronize()
    t_begin = time.perf_counter()
    for _ in range(steps):
        plan_f.spmm(val, x, out, True)
        plan_b.spmm(val_t, g, dx, True)
        k_ms.append(plan_f.profile_read()[0])
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t_begin) * 1e3 / steps
    plan_f.profile(False)
    kern_ms = sum(k_ms) / len(k_ms)
    info = plan_f.info()
    bytes_launch = b_alg(nnz, rows - info["empty_rows"], feat)  # empty rows are not visited
    _, fwd_ms = time_plan(plan_f, val, x, out, max(3, steps // 2), 1)
    _, bwd_ms = time_plan(plan_b, val_t, g, dx, max(3, steps // 2), 1)
    m_f = measured_traffic(args, workload, "A@X", feat) if args is not None else None
    m_b = measured_traffic(args, workload, "A^T@G", feat) if args is not None else None
    r = {"feat": feat, "steps": steps, "ms_per_step": round(ms_step, 4),
         "gflops": round(2 * 2.0 * nnz * feat / (ms_step * 1e-3) / 1e9, 2),
         "forward": op_report("A@X", nnz, rows, cols, feat, fwd_ms, info["empty_rows"], measured=m_f),
         "backward": op_report("A^T@G", nnz, cols, rows, feat, bwd_ms, plan_b.info()["empty_rows"], measured=m_b),
         "kernel_ms": round(kern_ms, 4), "kernel_ms_median": round(sorted(k_ms)[len(k_ms) // 2], 4),
         "kernel_ms_min": round(min(k_ms), 4), "kernel_bytes": bytes_launch}
    if planless:
        ms = time_planless(src, x, out, max(3, steps // 2))
        r["forward_without_plan"] = op_report("A@X through computation_ops.spmm (no plan: natural row order, int64 "
                                              "column indices)", nnz, rows, cols, feat, ms, info["empty_rows"])
        # that kernel reads the int64 column array itself: 8 more bytes per stored element than the model counts
        r["forward_without_plan"]["ms_with_plan"] = round(fwd_ms, 4)
    return r, x, g


def spmm_kernel_name(feat, planned=True):
    """The instance of the row kernel a contiguous, 16-byte aligned operand of this width runs in."""
    vec = 4 if feat % 4 == 0 else (2 if feat % 2 == 0 else 1)
    shapes = [(32, 1), (64, 1), (64, 2), (64, 3), (64, 4), (64, 5), (64, 6), (64, 8)]
    lpr, nch = next(((l, n) for l, n in shapes if vec * l * n >= feat), shapes[-1])
    return f"gnnagg::spmm_tasks_kernel<{vec},{lpr},{nch},{'int' if planned else 'long'},{1 if planned else 0},0>"


def run_c2(args, gate, sink):
    import torch

    from gnn_benchmark_amd import synthetic

    dev = "cuda:0"
    t0 = time.perf_counter()
    g = synthetic.power_law_graph(num_nodes=args.nodes, mean_out_degree=args.mean_out_degree, zipf_s=1.8,
                                  max_degree=15000, seed=args.seed, device=dev)
    src = g.adj
    info = src.get_plan().info()
    src.get_plan_for_transpose()
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    r, x, gr = spmm_pair(src, args.feat, args.steps, args.warmup, gen, args, "c2", planless="c2" in args.extras)
    achieved = r["kernel_bytes"] / (r["kernel_ms"] * 1e-3) / 1e9
    m = measured_traffic(args, "c2", "A@X", args.feat)
    line = {
        "metric": "spmm_fwd_bwd_gflops", "value": r["gflops"], "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"c2: CSR SpMM forward A@X + transposed backward A^T@G, power-law graph "
                               f"{g.num_nodes} nodes / {g.nnz} nnz (Zipf s=1.8, longest row {g.max_degree}), "
                               f"GCN-normalised fp32, dense operand {g.num_nodes}x{args.feat} fp32",
                   "nodes": g.num_nodes, "nnz": g.nnz, "feat": args.feat, "seed": args.seed,
                   "huge_rows": info["huge_rows"], "max_row_len": info["max_row_len"], "setup_s": round(setup_s, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": None if m is None else m[0] + m[1],
                     "traffic_kind": None if m is None else "constant from a rocprofv3 --pmc run of this workload "
                                                            "(not produced by this run): " + m[2],
                     "kernel": spmm_kernel_name(args.feat) + " (forward A@X, one launch over all rows)",
                     "kernel_ms": r["kernel_ms"], "kernel_ms_median": r["kernel_ms_median"],
                     "kernel_ms_min": r["kernel_ms_min"], "bytes_per_launch": r["kernel_bytes"]},
    }
    sink.put("c2_headline", r)
    # the gate (and the CPU baseline) on the headline operands themselves: one fresh product each way
    gpu_results = None
    if gate.enabled:
        rows, cols = src.sparse_sizes()
        fresh_f = torch.zeros(rows, args.feat, device=dev)
        fresh_b = torch.zeros(cols, args.feat, device=dev)
        src.get_plan().spmm(src.csr()[2], x, fresh_f, True)
        src.get_plan_for_transpose().spmm(src.storage.value_T(), gr, fresh_b, True)
        gpu_results = (fresh_f.cpu().numpy(), fresh_b.cpu().numpy())
        del fresh_f, fresh_b
    line["cpu_baseline"] = None
    if gate.enabled or not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_spmm(src, x.cpu().numpy(), gr.cpu().numpy(), gate, gpu_results,
                                                 timed=not args.no_cpu_baseline)
    del gpu_results
    if "c2" in args.extras:
        # the hidden widths of c4 / c5, c5's class count (172) and two narrow widths whose rows are not whole
        # 16-byte vectors or 64-byte multiples (class counts 40 and 47)
        widths = [r]
        for f in (128, 256, 172, 40, 47):
            if f != args.feat:
                widths.append(spmm_pair(src, f, max(3, args.steps // 4), 2, gen, args, "c2")[0])
        # a width that is no multiple of 4 (4-byte loads) against the same rows padded by one zero column to 48
        # (16-byte loads): the aggregation of a 47-class layer kept in 48-float rows; the first 47 columns of the
        # result are the same bits
        dev_rows, plan, val = src.sparse_size(0), src.get_plan(), src.csr()[2]
        x48 = torch.zeros(dev_rows, 48, device=dev)
        x48[:, :47].normal_(generator=gen)
        o48 = torch.zeros(dev_rows, 48, device=dev)
        x47, o47 = x48[:, :47].contiguous(), torch.zeros(dev_rows, 47, device=dev)
        _, ms47 = time_plan(plan, val, x47, o47, 5, 2, accumulate=False)
        _, ms48 = time_plan(plan, val, x48, o48, 5, 2, accumulate=False)
        widths.append({"feat": 47, "padded_to": 48, "forward_ms": round(ms47, 4), "forward_ms_padded": round(ms48, 4),
                       "same_bits": bool(torch.equal(o48[:, :47], o47))})
        del x48, o48, x47, o47
        sink.put("c2", widths)
    return line


def run_c1(args):
    """The single-rank case: 2-layer GCN forward + backward (no halo, no exchange) on a power-law graph of 100 000
    nodes, Zipf(2.0) out-degrees with mean 16, symmetrised with self-loops, values D^-1/2 (A+I) D^-1/2; features
    N(0,1) F=128, hidden 128, 16 classes, uniform labels.  The same step on the host cores beside it: the
    aggregations through the reference's compiled operator (forward through the CSR, backward through the
    transposed CSR, as its wrappers do), the dense parts by torch on the CPU."""
    import numpy as np
    import torch
    import torch.nn.functional as F

    from gnn_benchmark_amd import gcn, synthetic
    from gnn_benchmark_amd.data_manager import CommBuffer, CommSplits, DistributedGraphForPre

    dev = "cuda:0"
    n, feat, hidden, classes = 100_000, 128, 128, 16
    g = synthetic.power_law_graph(n, 16, 2.0, 20_000, seed=args.seed + 1, device=dev)
    splits = CommSplits([0], [0], 1, 32)
    graph = DistributedGraphForPre(g.adj, None, None, [0], [0], torch.ones(n, 1, device=dev), splits,
                                   CommBuffer(splits, feat, 32, device=dev), None, exchange=None)
    gen = torch.Generator(device=dev).manual_seed(args.seed + 2)
    x = torch.randn(n, feat, device=dev, generator=gen)
    labels = torch.randint(0, classes, (n,), device=dev, generator=gen)
    torch.manual_seed(args.seed + 3)
    model = gcn.GCN([feat, hidden, classes], dropout=0.0).to(dev)
    model.train()

    def step():
        model.zero_grad(set_to_none=True)
        loss = F.nll_loss(model(graph, x, True, None), labels)
        loss.backward()
        return loss

    steps = max(10, args.steps)
    for _ in range(3):
        loss = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    plan = g.adj.get_plan()
    out_buf = torch.zeros(n, feat, device=dev)
    _, spmm_ms = time_plan(plan, g.adj.csr()[2], x, out_buf, steps, 2, accumulate=False)
    r = {"workload": f"c1: single rank, 2-layer GCN forward + backward, {n} nodes / {g.nnz} nnz (longest row "
                     f"{g.max_degree}), F={feat}, hidden {hidden}, {classes} classes",
         "forward_backward_ms": round(ms, 3), "loss": round(float(loss.detach()), 5), "steps": steps,
         "aggregation": op_report("A@X (overwriting)", g.nnz, n, n, feat, spmm_ms, plan.info()["empty_rows"], False)}
    if args.no_cpu_baseline:
        return r
    from oracle import spmm as ospmm

    threads = ospmm.max_threads()
    run, kind = cpu_operator(threads)
    csr = [t.cpu().numpy() for t in g.adj.csr()]
    csc = [g.adj.storage.colptr().cpu().numpy(), g.adj.storage.row_T().cpu().numpy(),
           g.adj.storage.value_T().cpu().numpy()]
    ones = np.ones(csr[1].shape[0], np.float32)
    rs_f = ospmm.distribute_work_for_row(csr[0], ones, threads)
    rs_b = ospmm.distribute_work_for_row(csc[0], ones, threads)

    class HostAggregate(torch.autograd.Function):
        @staticmethod
        def forward(ctx, t):
            out = np.zeros((n, t.shape[1]), dtype=np.float32)
            run(csr[0], csr[1], csr[2], np.ascontiguousarray(t.detach().numpy()), out, rs_f)
            return torch.from_numpy(out)

        @staticmethod
        def backward(ctx, grad):
            out = np.zeros((n, grad.shape[1]), dtype=np.float32)
            run(csc[0], csc[1], csc[2], np.ascontiguousarray(grad.numpy()), out, rs_b)
            return torch.from_numpy(out)

    w = [p.detach().cpu().clone().requires_grad_() for p in model.parameters()]  # W1, b1, W2, b2
    x_host, labels_host = x.cpu(), labels.cpu()

    def host_step():
        for p in w:
            p.grad = None
        h = torch.relu(HostAggregate.apply(x_host) @ w[0] + w[1])
        z = HostAggregate.apply(h) @ w[2] + w[3]
        host_loss = F.nll_loss(F.log_softmax(z, dim=1), labels_host)
        host_loss.backward()
        return host_loss

    sec = cpu_median_seconds(host_step)
    r["cpu"] = {"forward_backward_ms": round(sec * 1e3, 2), "loss": round(float(host_step().detach()), 5)}
    r["cpu"].update(cpu_description(kind, threads))
    return r


def load_probes():
    """ctypes handle of bench_probes/libbenchprobes.so (built by __graft_entry__.build(); built here when missing)."""
    import ctypes
    import subprocess

    here = os.path.join(ROOT, "bench_probes")
    path = os.path.join(here, "libbenchprobes.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", here, "libbenchprobes.so"], stdout=subprocess.DEVNULL)
    L = ctypes.CDLL(path)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.bench_probe_memory.restype = i32
    L.bench_probe_memory.argtypes = [i32, vp, vp, vp, i64, i64, i64, vp]
    L.bench_probe_issue.restype = i32
    L.bench_probe_issue.argtypes = [i32, i32, vp, vp]
    return L


def run_ceilings(args):
    """What the memory system delivers, in this run, for plain kernels with the access mixes of the aggregation
    path (bench_probes/libbenchprobes.so, `bench_probe_memory`; asked for with `--only ceilings`): streams, uniformly random 512-byte row gathers with nothing written, and the
    same gathers mixed with the row writes / row read-modify-writes of the boundary products (7 gathers per row
    written: the pre-aggregation's mix; 3 per row read and written: the post-aggregation's; 15: the local product's
    on a graph without hub rows).  Sizes of the c4 partition at F=128: 7 M source rows, 20 M gathers."""
    import torch

    from gnn_benchmark_amd import _lib

    dev = torch.device("cuda:0")
    rows, feat, gathers = args.c4_nodes, 128, int(args.c4_nodes * 20 / 7)
    gen = torch.Generator(device=dev).manual_seed(args.seed + 9)
    src = torch.randn(rows, feat, device=dev, generator=gen)
    dst = torch.zeros(rows, feat, device=dev)
    index = torch.randint(0, rows, (gathers,), device=dev, generator=gen, dtype=torch.int32)
    L = load_probes()
    stream = _lib.current_stream(dev)

    def check(rc):
        if rc != 0:
            raise RuntimeError(f"libbenchprobes returned {rc} (1 bad argument, 2 HIP error, 3 unsupported row width)")

    def timed(kind, count, per_row, nbytes, reps=10):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(reps + 2):
            if i == 2:
                e0.record()
            check(L.bench_probe_memory(kind, _lib.ptr(src), _lib.ptr(index), _lib.ptr(dst), count, feat, per_row, stream))
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1) / reps
        return {"ms": round(ms, 4), "bytes": nbytes, "gbs": round(nbytes / ms / 1e6, 1),
                "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}

    n = rows * feat
    row_b = feat * 4.0
    out = {"sizes": f"{rows} rows x {feat} fp32, {gathers} gathers through uniformly random int32 row numbers",
           "stream_read": timed(0, n, 1, n * 4.0), "stream_write": timed(1, n, 1, n * 4.0),
           "stream_copy": timed(2, n, 1, n * 8.0)}
    for name, kind, per_row in (("gather_only", 3, 8), ("gather_7_per_row_written", 4, 7),
                                ("gather_3_per_row_read_and_written", 5, 3),
                                ("gather_15_per_row_read_and_written", 5, 15), ("gather_15_per_row_written", 4, 15)):
        results = gathers // per_row
        nbytes = results * per_row * (row_b + 4.0) + (results * row_b if kind >= 4 else 0) + (results * row_b if kind == 5 else 0)
        out[name] = timed(kind, results, per_row, nbytes)

    # matrix pipe and vector ALU of a SIMD, fed by different waves (`bench_probe_issue`): alone and together
    def issue(mfma_rounds, valu_rounds, reps=5):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(reps + 2):
            if i == 2:
                e0.record()
            check(L.bench_probe_issue(mfma_rounds, valu_rounds, _lib.ptr(dst), stream))
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / reps

    rounds = 5000
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    m, v, both = issue(rounds, 0), issue(0, rounds), issue(rounds, rounds)
    out["matrix_pipe_and_vector_alu"] = {
        "what": f"one block of 8 waves per compute unit; waves 0-3 issue {8 * rounds} independent v_mfma_f32_32x32x16_bf16 "
                f"each, waves 4-7 run {8 * rounds} rounds of the fp32 -> bf16-pieces cutting sequence each",
        "mfma_alone_ms": round(m, 4), "vector_alone_ms": round(v, 4), "together_ms": round(both, 4),
        "sum_of_the_two_ms": round(m + v, 4),
        "mfma_alone_tflops": round(2.0 * 32 * 32 * 16 * 8 * rounds * 4 * cus / m / 1e9, 1),
        "reading": "together = max of the two: the pipes overlap; together = their sum: they take turns"}
    return out


def run_c3(args):
    import torch

    from gnn_benchmark_amd import synthetic

    dev = "cuda:0"
    g = synthetic.dense_degree_graph(num_nodes=233_000, mu=5.5, sigma=1.2, seed=args.seed, device=dev)
    gen = torch.Generator(device=dev).manual_seed(args.seed + 3)
    out = {"graph": g.description, "nodes": g.num_nodes, "nnz": g.nnz, "max_row_len": g.max_degree, "runs": []}
    for f in (602, 256):
        r, x, _g = spmm_pair(g.adj, f, max(3, args.steps // 4), 2, gen, args, "c3")
        if not args.no_cpu_baseline and f == 602:
            rowptr, col, val = [t.cpu().numpy() for t in g.adj.csr()]
            sec, kind, threads = cpu_time_product(rowptr, col, val, x.cpu().numpy(), g.num_nodes)
            r["forward"]["cpu_ms"] = round(sec * 1e3, 1)
            r["forward"]["cpu"] = f"{kind} operator, {threads} threads"
        out["runs"].append(r)
        del x, _g
    return out


def build_c4(args):
    import torch

    from gnn_benchmark_amd import synthetic

    dev = "cuda:0"
    t0 = time.perf_counter()
    part = synthetic.partition_edges(num_local_nodes=args.c4_nodes, world_size=16, rank=3,
                                     local_mean_out_degree=6.8, zipf_s=1.8, max_degree=15000,
                                     num_halo_nodes=int(args.c4_nodes * 3 / 7),
                                     num_remote_edges=int(args.c4_nodes * 20 / 7), seed=args.seed + 4, device=dev)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    # stand-in rows on the scale of real ones: features O(0.1), gradients of a mean loss O(1e-7)
    # (the seeded rows are drawn once per layer and direction and kept on the device; a step points the boundary
    # buffers at them -- no random-number work, and no other work of the stand-in, inside a timed step)
    exchange = synthetic.PregeneratedHaloExchange(args.seed + 4, std=0.1, backward_std=1e-7)
    graph = synthetic.build_partition_graph(part, 256, True, exchange=exchange, device=dev)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for m in (graph.local_adj_t, graph.adj_t_pre_post_aggr_from, graph.adj_t_pre_post_aggr_to):
        m.get_plan()
        m.get_plan_for_transpose()
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    # what the set-up time is made of: the synthetic edge lists (not part of the path), the index-map builders with
    # the three matrices and the buffers (the reference's DataProcessor loops), the six degree-ordered plans with the
    # transposed arrays behind three of them
    setup = {"total": round(t3 - t0, 3), "synthetic_edge_lists": round(t1 - t0, 3),
             "index_maps_matrices_buffers": round(t2 - t1, 3), "plans_and_transposed_arrays": round(t3 - t2, 3)}
    return part, graph, setup


def run_c4(args, graph, setup_s, gate=None):
    import torch

    from gnn_benchmark_amd import Aggregator

    dev = "cuda:0"
    n, feat = graph.local_adj_t.sparse_size(0), 128
    steps = max(5, args.steps // 2)
    gen = torch.Generator(device=dev).manual_seed(args.seed + 5)
    x = torch.randn(n, feat, device=dev, generator=gen)
    g = torch.randn(n, feat, device=dev, generator=gen)
    graph.comm_buf.resize_buffer(graph.comm_splits, feat, 32)
    send_buf, recv_buf = graph.comm_buf.send_buf, graph.comm_buf.recv_buf
    recv_buf.normal_(generator=gen)
    out = torch.zeros(n, feat, device=dev)
    ops = []
    # Each product is timed the way Aggregator runs it (`as_run`): the pre-aggregation OVERWRITES the send buffer and
    # the local product OVERWRITES the fresh output (no read of the old rows, every row written), the post-aggregation
    # accumulates onto the output; in the gradient direction A_from^T @ G overwrites the receive buffer, A_local^T @ G
    # overwrites the fresh gradient and A_to^T @ send_buf accumulates onto it.  The other mode of each is timed too.
    for key, name, m, src_x, dst, fwd_overwrites, bwd_overwrites in (
            ("pre", "pre-aggregation A_to@X -> send_buf", graph.adj_t_pre_post_aggr_to, x, send_buf, True, False),
            ("local", "local A_local@X -> out", graph.local_adj_t, x, out, True, True),
            ("post", "post-aggregation A_from@recv_buf -> out", graph.adj_t_pre_post_aggr_from, recv_buf, out, False, True)):
        rows, cols = m.sparse_sizes()
        plan, plan_t = m.get_plan(), m.get_plan_for_transpose()
        for accumulate in (True, False):
            _, ms = time_plan(plan, m.csr()[2], src_x, dst, steps, 2, accumulate=accumulate)
            ops.append(op_report(name + ("" if accumulate else " (overwriting)"), m.nnz(), rows, cols, feat, ms,
                                 plan.info()["empty_rows"], accumulate,
                                 measured_traffic(args, "c4", key + ("" if accumulate else "_overwrite"), feat)))
            ops[-1]["as_run_by_aggregator"] = accumulate != fwd_overwrites
            if accumulate and not args.no_cpu_baseline:
                rowptr, col, val = [t.cpu().numpy() for t in m.csr()]
                sec, kind, threads = cpu_time_product(rowptr, col, val, src_x.cpu().numpy(), rows)
                ops[-1]["cpu_ms"] = round(sec * 1e3, 1)
                ops[-1]["cpu"] = f"{kind} operator, {threads} threads"
        back = torch.zeros(cols, feat, device=dev)
        for accumulate in (True, False):
            _, ms = time_plan(plan_t, m.storage.value_T(), dst, back, steps, 2, accumulate=accumulate)
            ops.append(op_report(name.split(" ")[0] + " transposed (gradient direction)"
                                 + ("" if accumulate else " (overwriting)"), m.nnz(), cols, rows, feat, ms,
                                 plan_t.info()["empty_rows"], accumulate,
                                 measured_traffic(args, "c4", key + "_T" + ("" if accumulate else "_overwrite"), feat)))
            ops[-1]["as_run_by_aggregator"] = accumulate != bwd_overwrites
        del back
    ms = time_planless(graph.local_adj_t, x, out, steps)
    ops.append(op_report("local A_local@X through computation_ops.spmm (no plan: natural row order, int64 column "
                         "indices)", graph.local_adj_t.nnz(), n, n, feat, ms,
                         graph.local_adj_t.get_plan().info()["empty_rows"],
                         measured=measured_traffic(args, "c4", "local_planless", feat)))
    # the whole autograd.Function, forward and backward, synthetic halo rows generated on the device
    xr = x.clone().requires_grad_()
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 32, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 32, True, True)
    torch.cuda.synchronize()
    fwd_ms = (time.perf_counter() - t0) * 1e3 / steps
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 32, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    both_ms = (time.perf_counter() - t0) * 1e3 / steps
    if gate is not None and gate.enabled:
        with torch.no_grad():
            o = Aggregator.apply(graph, x, 0, 32, True, True)
        parity_rows_of_pipeline(gate, graph, x, o, graph.comm_buf.recv_buf, 4000, args.seed + 11)
    # the same with the local and the received elements of every output row in ONE launch each way
    # (graph.one_launch: [A_local | A_from] over (x ; recv_buf), [A_local^T | A_to^T] over (g ; send_buf))
    from gnn_benchmark_amd.sparse_tensor import side_by_side

    graph.one_launch = True
    for _ in range(2):
        o1 = Aggregator.apply(graph, xr, 0, 32, True, True)
        o1.backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o1 = Aggregator.apply(graph, xr, 0, 32, True, True)
    torch.cuda.synchronize()
    fwd1_ms = (time.perf_counter() - t0) * 1e3 / steps
    t0 = time.perf_counter()
    for _ in range(steps):
        o1 = Aggregator.apply(graph, xr, 0, 32, True, True)
        o1.backward(g)
    torch.cuda.synchronize()
    both1_ms = (time.perf_counter() - t0) * 1e3 / steps
    graph.one_launch = False
    # the one-launch result against the three-launch one (`o`), every row: the same chains, so the same bits
    one_launch_same_bits = bool(torch.equal(o1.detach(), o.detach()))
    if not one_launch_same_bits and gate is not None and gate.enabled:
        print("bench.py: the one-launch aggregation differs from the three-launch one; no number is reported",
              file=sys.stderr, flush=True)
        sys.exit(4)
    del o, o1
    for key, left, right, transposed, a1, a2, nm in (
            ("local+post", graph.local_adj_t, graph.adj_t_pre_post_aggr_from, False, x, graph.comm_buf.recv_buf,
             "local + post-aggregation in one launch [A_local | A_from]@(X ; recv_buf) -> out (overwriting)"),
            ("local_T+pre_T", graph.local_adj_t, graph.adj_t_pre_post_aggr_to, True, g, graph.comm_buf.send_buf,
             "local + pre-aggregation transposed in one launch [A_local^T | A_to^T]@(G ; send_buf) -> dX (overwriting)")):
        m = side_by_side(left, right, transposed)
        plan = m.get_plan()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(steps + 2):
            if i == 2:
                e0.record()
            plan.spmm_two_sources(m.csr()[2], a1, a2, out, accumulate=False)
        e1.record()
        e1.synchronize()
        ops.append(op_report(nm, m.nnz(), m.sparse_size(0), m.sparse_size(1), feat, e0.elapsed_time(e1) / steps,
                             plan.info()["empty_rows"], False, measured_traffic(args, "c4", key, feat)))
        ops[-1]["as_run_by_aggregator"] = "one_launch"
    graph.comm_buf.resize_buffer(graph.comm_splits, feat, 32)  # (the buffer's own tensors again, not delivered rows)
    codec = run_c4_codec(graph, feat, steps, gen, cpu=not args.no_cpu_baseline)
    # the same autograd.Function with the boundary rows travelling as int2 (seeded packed rows)
    from gnn_benchmark_amd import synthetic
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits

    world = len(graph.comm_splits.send_splits)
    fp32_splits = graph.comm_splits
    graph.comm_splits = CommSplits(fp32_splits.recv_splits, fp32_splits.send_splits, world, 2)
    graph.comm_buf_for_quantization = CommBufferForQuantization(graph.comm_splits, feat, 2, device=dev)
    graph.exchange_quantized = synthetic.PregeneratedQuantizedHaloExchange(args.seed + 6)
    # the reference's form: the outgoing rows quantised out of the fp32 buffer, the received ones dequantised into it
    graph.fuse_dequantize = graph.fuse_quantize = False
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 2, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 2, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    int2_both_ms = (time.perf_counter() - t0) * 1e3 / steps
    # ... and as it runs by default: the products in front of the exchange write the packed rows themselves, the
    # products behind it aggregate straight from the packed bytes (no quantise pass, no dequantise pass)
    graph.fuse_dequantize = graph.fuse_quantize = True
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 2, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 2, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    int2_fused_ms = (time.perf_counter() - t0) * 1e3 / steps
    # ... and with one launch for the local elements and the received ones, gathered straight from the packed bytes
    graph.one_launch = True
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 2, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 2, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    int2_one_launch_ms = (time.perf_counter() - t0) * 1e3 / steps
    graph.one_launch = False
    from gnn_benchmark_amd.spmm_kernel import SPMM_forward_quantized

    qb, m = graph.comm_buf_for_quantization, graph.adj_t_pre_post_aggr_from
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(steps + 2):
        if i == 2:
            e0.record()
        SPMM_forward_quantized(m, qb.quantized_recv_data_buf, qb.quantized_recv_params_buf_fp32, qb.recv_row_code, out, 2)
    e1.record()
    e1.synchronize()
    codec.append({"op": "post-aggregation A_from@recv straight from the int2 bytes -> out", "bits": 2,
                  "rows_visited": m.sparse_size(0) - m.get_plan().info()["empty_rows"], "nnz": m.nnz(), "feat": feat,
                  "ms": round(e0.elapsed_time(e1) / steps, 4)})
    from gnn_benchmark_amd import computation_ops

    m = graph.adj_t_pre_post_aggr_to
    rp, cidx, vals = m.csr()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(steps + 2):
        if i == 2:
            e0.record()
        computation_ops.spmm_quantize_for_all_procs(rp, cidx, vals, x, qb.quantized_send_data_buf,
                                                    qb.quantized_send_params_buf_fp32, qb.quantized_work_range_per_proc,
                                                    world, 2)
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_time(e1) / steps
    gathered = m.nnz() * (4.0 * feat + 12.0) + m.sparse_size(0) * (8.0 + 8.0 + feat / 4.0)
    codec.append({"op": "pre-aggregation A_to@X straight into the int2 bytes (natural row order, int64 column indices)",
                  "bits": 2, "rows": m.sparse_size(0), "nnz": m.nnz(), "feat": feat, "ms": round(ms, 4),
                  "bytes_model": gathered, "gbs_model": round(gathered / (ms * 1e-3) / 1e9, 1),
                  "frac_model": round(gathered / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    graph.comm_splits, graph.comm_buf_for_quantization, graph.exchange_quantized = fp32_splits, None, None
    # ... and as bf16 (num_bits=16): the two conversion passes per direction around a seeded stand-in
    from gnn_benchmark_amd.aggregator import _convert
    from gnn_benchmark_amd.data_manager import CommBuffer

    fp32_buf = graph.comm_buf
    graph.comm_buf = CommBuffer(fp32_splits, feat, 16, device=dev)
    synthetic.PregeneratedHaloExchange.attach(graph)
    graph.exchange_bf16 = synthetic.PregeneratedBf16HaloExchange(args.seed + 7)
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 16, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 16, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    bf16_both_ms = (time.perf_counter() - t0) * 1e3 / steps
    graph.one_launch = True   # one launch for the local elements and the received bf16 rows
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 16, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 16, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    bf16_one_launch_ms = (time.perf_counter() - t0) * 1e3 / steps
    graph.one_launch = False
    # ... and with the two tensor copies around the exchange as passes of their own (the reference's form)
    graph.fuse_bf16_staging = False
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 16, True, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 16, True, True)
        o.backward(g)
    torch.cuda.synchronize()
    bf16_unfused_ms = (time.perf_counter() - t0) * 1e3 / steps
    graph.fuse_bf16_staging = True
    graph.comm_buf.resize_buffer(fp32_splits, feat, 16)   # the buffer's own rows again, not the delivered ones
    # the two products of the fused form: pre-aggregation writing bf16 rows, post-aggregation gathering bf16 rows
    from gnn_benchmark_amd import SPMM_forward

    for name, m, src, dst, acc in (
            ("pre-aggregation A_to@X -> bf16 send rows (overwriting)", graph.adj_t_pre_post_aggr_to, x,
             graph.comm_buf.send_buf_fp16, False),
            ("post-aggregation A_from@(bf16 recv rows) -> out", graph.adj_t_pre_post_aggr_from,
             graph.comm_buf.recv_buf_fp16, out, True)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(steps + 2):
            if i == 2:
                e0.record()
            SPMM_forward(m, src, dst, accumulate=acc)
        e1.record()
        e1.synchronize()
        codec.append({"op": name, "bits": 16, "nnz": m.nnz(), "feat": feat, "ms": round(e0.elapsed_time(e1) / steps, 4)})
    for name, src, dst in (("send_buf -> bf16", graph.comm_buf.send_buf, graph.comm_buf.send_buf_fp16),
                           ("bf16 -> recv_buf", graph.comm_buf.recv_buf_fp16, graph.comm_buf.recv_buf)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(steps + 2):
            if i == 2:
                e0.record()
            _convert(src, dst)
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1) / steps
        codec.append({"op": name, "bits": 16, "rows": int(src.size(0)), "feat": feat, "ms": round(ms, 4),
                      "gbs": round(src.numel() * 6.0 / (ms * 1e-3) / 1e9, 1),
                      "frac_of_hbm_peak": round(src.numel() * 6.0 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    graph.comm_buf, graph.exchange_bf16 = fp32_buf, None
    return {"partition": f"rank 3 of 16, {n} local nodes", "feat": feat, "setup_s": round(setup_s["total"], 2),
            "setup_breakdown_s": setup_s, "codec": codec,
            "local_nnz": graph.local_adj_t.nnz(), "halo_rows": int(recv_buf.size(0)), "send_rows": int(send_buf.size(0)),
            "from_nnz": graph.adj_t_pre_post_aggr_from.nnz(), "to_nnz": graph.adj_t_pre_post_aggr_to.nnz(),
            "ops": ops, "aggregator_forward_ms": round(fwd_ms, 3),
            "aggregator_forward_backward_ms": round(both_ms, 3),
            "aggregator_forward_ms_one_launch": round(fwd1_ms, 3),
            "aggregator_forward_backward_ms_one_launch": round(both1_ms, 3),
            "one_launch_same_bits": one_launch_same_bits,
            "aggregator_forward_backward_ms_bf16_exchange": round(bf16_both_ms, 3),
            "aggregator_forward_backward_ms_bf16_exchange_separate_copies": round(bf16_unfused_ms, 3),
            "aggregator_forward_backward_ms_int2_exchange": round(int2_fused_ms, 3),
            "aggregator_forward_backward_ms_int2_exchange_one_launch": round(int2_one_launch_ms, 3),
            "aggregator_forward_backward_ms_bf16_exchange_one_launch": round(bf16_one_launch_ms, 3),
            "aggregator_forward_backward_ms_int2_exchange_separate_codec_passes": round(int2_both_ms, 3)}


def cpu_time_codec(x_host, bits, reps=2):
    """Median seconds of the reference's compiled row-packed quantise / dequantise kernels on the
    host cores (self_benchmark/a64fx/model/ops/src/quantization_x86.cpp:17-162; the parameters,
    which that variant takes as inputs, come from the oracle and are not timed), or None when
    oracle/_ref is not loadable."""
    import torch

    from oracle import quantization as oq
    from oracle import spmm as ospmm

    ref = ospmm.load_reference_op()
    if ref is None:
        return None
    threads = ospmm.max_threads()
    torch.set_num_threads(threads)
    rows, feat = x_host.shape
    params = oq.row_params(x_host, bits)
    x = torch.from_numpy(x_host)
    lo, scale = torch.from_numpy(params[:, 0].copy()), torch.from_numpy(params[:, 1].copy())
    packed = torch.zeros((-(-rows // (8 // bits)), feat), dtype=torch.uint8)
    back = torch.empty_like(x)
    out = {}
    for name, run in (("quantize", lambda: ref.quantize_tensor(x, packed, lo, scale, bits)),
                      ("dequantize", lambda: ref.dequantize_tensor(packed, back, lo, scale, bits))):
        run()
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
        times.sort()
        out[name] = times[len(times) // 2]
    out["threads"] = threads
    return out


def run_c4_codec(graph, feat, steps, gen, cpu=False):
    """int2 codec of the partition's boundary buffers (one segment per peer rank): quantise the
    send buffer, dequantise into the receive buffer.  Bytes: fp32 rows + packed rows + 8 B of
    parameters per row, each moved once."""
    import torch

    from gnn_benchmark_amd import computation_ops as ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits

    world = len(graph.comm_splits.send_splits)
    out = []
    for bits in (2, 8):
        splits = CommSplits(graph.comm_splits.recv_splits, graph.comm_splits.send_splits, world, bits)
        q = CommBufferForQuantization(splits, feat, bits, device=graph.comm_buf.send_buf.device)
        send_buf, recv_buf = graph.comm_buf.send_buf, graph.comm_buf.recv_buf
        send_buf.normal_(generator=gen)

        def quantize():
            ops.quantize_tensor_for_all_procs(send_buf, q.quantized_send_data_buf, q.quantized_send_params_buf_fp32,
                                              q.quantized_work_range_per_proc, world, bits)

        def dequantize():
            ops.dequantize_tensor_for_all_procs(q.quantized_recv_data_buf, recv_buf, q.quantized_recv_params_buf_fp32,
                                                q.dequantized_work_range_per_proc, world, bits)

        for name, fn, rows, packed_rows in (("quantize send_buf", quantize, send_buf.size(0), q.quantized_send_data_buf.size(0)),
                                            ("dequantize into recv_buf", dequantize, recv_buf.size(0),
                                             q.quantized_recv_data_buf.size(0))):
            for _ in range(2):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            e1.synchronize()
            ms = e0.elapsed_time(e1) / steps
            nbytes = rows * feat * 4.0 + packed_rows * feat + rows * 8.0
            out.append({"op": name, "bits": bits, "rows": int(rows), "packed_rows": int(packed_rows), "feat": feat,
                        "ms": round(ms, 4), "bytes": nbytes, "gbs": round(nbytes / ms / 1e6, 1),
                        "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)})
        if cpu and bits == 2:
            host = cpu_time_codec(send_buf.cpu().numpy(), bits)
            if host is not None:
                out[-2]["cpu_ms"] = round(host["quantize"] * 1e3, 1)
                out[-1]["cpu_ms"] = round(host["dequantize"] * 1e3, 1)
                out[-2]["cpu"] = out[-1]["cpu"] = (f"reference x86 kernel on the send buffer's {send_buf.size(0)} rows, "
                                                   f"{host['threads']} threads")
        del q
    return out


def run_c4_raw_halo(args, part):
    """The same partition with raw boundary rows (``is_pre_delay=False``): rows gathered into the
    send buffer instead of pre-aggregated, halo rows aggregated through ``remote_adj_t``, and the
    backward's ``index_add_`` as a product with the selection matrix."""
    import torch

    from gnn_benchmark_amd import Aggregator, synthetic
    from gnn_benchmark_amd.aggregator import _gather_rows

    dev = "cuda:0"
    feat = 128
    steps = max(5, args.steps // 2)
    t0 = time.perf_counter()
    graph = synthetic.build_partition_graph(part, 256, False, exchange=synthetic.PregeneratedHaloExchange(args.seed + 4),
                                            device=dev)
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    n = graph.local_adj_t.sparse_size(0)
    gen = torch.Generator(device=dev).manual_seed(args.seed + 5)
    x = torch.randn(n, feat, device=dev, generator=gen)
    g = torch.randn(n, feat, device=dev, generator=gen)
    graph.comm_buf.resize_buffer(graph.comm_splits, feat, 32)
    send_buf, recv_buf = graph.comm_buf.send_buf, graph.comm_buf.recv_buf
    recv_buf.normal_(generator=gen)
    out = torch.zeros(n, feat, device=dev)
    idx = graph.idx_nodes_send_to_others
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(steps + 2):
        if i == 2:
            e0.record()
        _gather_rows(x, idx, send_buf)
    e1.record()
    e1.synchronize()
    gather_ms = e0.elapsed_time(e1) / steps
    gather_bytes = idx.numel() * (8.0 + 2 * 4.0 * feat)
    ops = [{"op": "gather boundary rows X[idx] -> send_buf", "rows": int(idx.numel()), "feat": feat,
            "ms": round(gather_ms, 4), "gbs_model": round(gather_bytes / (gather_ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(gather_bytes / (gather_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}]
    for name, m, src_x, dst in (("halo aggregation A_remote@recv_buf -> out", graph.remote_adj_t, recv_buf, out),
                                ("scatter of received gradients (index_add_ as a product) -> dX",
                                 graph.send_scatter_adj_t(), send_buf, out)):
        rows, cols = m.sparse_sizes()
        _, ms = time_plan(m.get_plan(), m.csr()[2], src_x, dst, steps, 2, accumulate=True)
        ops.append(op_report(name, m.nnz(), rows, cols, feat, ms, m.get_plan().info()["empty_rows"]))
    m = graph.remote_adj_t
    back = torch.zeros(m.sparse_size(1), feat, device=dev)
    _, ms = time_plan(m.get_plan_for_transpose(), m.storage.value_T(), out, back, steps, 2, accumulate=True)
    ops.append(op_report("halo aggregation transposed (gradient direction)", m.nnz(), m.sparse_size(1), m.sparse_size(0),
                         feat, ms, m.get_plan_for_transpose().info()["empty_rows"]))
    del back
    xr = x.clone().requires_grad_()
    for _ in range(2):
        Aggregator.apply(graph, xr, 0, 32, False, True).backward(g)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 32, False, True)
    torch.cuda.synchronize()
    fwd_ms = (time.perf_counter() - t0) * 1e3 / steps
    t0 = time.perf_counter()
    for _ in range(steps):
        o = Aggregator.apply(graph, xr, 0, 32, False, True)
        o.backward(g)
    torch.cuda.synchronize()
    both_ms = (time.perf_counter() - t0) * 1e3 / steps
    # the same with bf16 rows on the wire (num_bits=16): the gather writes the bf16 staging rows itself, or the tensor
    # copy follows it as a pass of its own (the reference's form)
    from gnn_benchmark_amd.data_manager import CommBuffer

    fp32_buf = graph.comm_buf
    graph.comm_buf = CommBuffer(graph.comm_splits, feat, 16, device=dev)
    synthetic.PregeneratedHaloExchange.attach(graph)
    graph.exchange_bf16 = synthetic.PregeneratedBf16HaloExchange(args.seed + 7)
    for i in range(steps + 2):
        if i == 2:
            e0.record()
        _gather_rows(x, idx, graph.comm_buf.send_buf_fp16)
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_time(e1) / steps
    gather16_bytes = idx.numel() * (8.0 + 6.0 * feat)
    ops.append({"op": "gather boundary rows X[idx] -> bf16 send rows", "rows": int(idx.numel()), "feat": feat,
                "ms": round(ms, 4), "gbs_model": round(gather16_bytes / (ms * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(gather16_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    bf16_ms = {}
    for fused in (True, False):
        graph.fuse_bf16_staging = fused
        for _ in range(2):
            Aggregator.apply(graph, xr, 0, 16, False, True).backward(g)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            o = Aggregator.apply(graph, xr, 0, 16, False, True)
            o.backward(g)
        torch.cuda.synchronize()
        bf16_ms[fused] = (time.perf_counter() - t0) * 1e3 / steps
    graph.fuse_bf16_staging = True
    graph.comm_buf, graph.exchange_bf16 = fp32_buf, None
    # ... and as int2 (num_bits=2): the gather and the gradient product writing the packed rows themselves and the
    # products behind the exchange reading them (the default), or the reference's passes each on its own
    from gnn_benchmark_amd import computation_ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits

    world = len(graph.comm_splits.send_splits)
    fp32_splits = graph.comm_splits
    graph.comm_buf.resize_buffer(fp32_splits, feat, 32)
    graph.comm_splits = CommSplits(fp32_splits.recv_splits, fp32_splits.send_splits, world, 2)
    qb = graph.comm_buf_for_quantization = CommBufferForQuantization(graph.comm_splits, feat, 2, device=dev)
    graph.exchange_quantized = synthetic.PregeneratedQuantizedHaloExchange(args.seed + 6)
    for i in range(steps + 2):
        if i == 2:
            e0.record()
        computation_ops.gather_quantize_for_all_procs(x, idx, qb.quantized_send_data_buf, qb.quantized_send_params_buf_fp32,
                                                      qb.quantized_work_range_per_proc, world, 2)
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_time(e1) / steps
    gq_bytes = idx.numel() * (8.0 + 4.0 * feat + feat / 4.0 + 8.0)
    ops.append({"op": "gather boundary rows X[idx] -> int2 bytes + parameters", "rows": int(idx.numel()), "feat": feat,
                "ms": round(ms, 4), "gbs_model": round(gq_bytes / (ms * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(gq_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    int2_ms = {}
    for fused in (True, False):
        graph.fuse_quantize = graph.fuse_dequantize = fused
        for _ in range(2):
            Aggregator.apply(graph, xr, 0, 2, False, True).backward(g)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            o = Aggregator.apply(graph, xr, 0, 2, False, True)
            o.backward(g)
        torch.cuda.synchronize()
        int2_ms[fused] = (time.perf_counter() - t0) * 1e3 / steps
    graph.fuse_quantize = graph.fuse_dequantize = True
    graph.comm_splits, graph.comm_buf_for_quantization, graph.exchange_quantized = fp32_splits, None, None
    return {"workload": "the c4 partition with raw boundary rows (is_pre_delay=False)", "feat": feat,
            "aggregator_forward_backward_ms_int2_exchange": round(int2_ms[True], 3),
            "aggregator_forward_backward_ms_int2_exchange_separate_codec_passes": round(int2_ms[False], 3),
            "send_rows": int(idx.numel()), "halo_rows": int(graph.remote_adj_t.sparse_size(1)), "setup_s": round(setup_s, 2),
            "ops": ops, "aggregator_forward_ms": round(fwd_ms, 3), "aggregator_forward_backward_ms": round(both_ms, 3),
            "aggregator_forward_backward_ms_bf16_exchange": round(bf16_ms[True], 3),
            "aggregator_forward_backward_ms_bf16_exchange_separate_copies": round(bf16_ms[False], 3)}


def run_c5(args, graph):
    import torch

    from gnn_benchmark_amd import gcn

    dev = "cuda:0"
    n = graph.local_adj_t.sparse_size(0)
    dims = [128, 256, 256, 172]
    gen = torch.Generator(device=dev).manual_seed(args.seed + 6)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 10]
    masks = gcn.make_dropout_masks(n, dims, 0.5, args.seed + 7, dev)
    steps = max(3, args.steps // 4)
    out = {"dims": dims, "nodes": n, "labelled": int(train_idx.numel()), "dropout": 0.5, "optimizer": "Adam(lr=0.01)",
           "steps": steps}
    # the two GEMM variants with dense hidden activations, then the same with the hidden activations
    # kept packed (non-zero values + bitmap), which the next layer's aggregation gathers instead,
    # then with the narrowing last layer multiplying before it aggregates (A (x W) instead of (A x) W)
    folded = None
    # (layers with dense activations run as one libgnnagg kernel each way; "separate_kernels" is the
    # same model with the product -- the same kernel, bare -- and the elementwise passes apart).
    # `library_products_per_step`: dense products of one step that fell through to the BLAS library (0: none)
    for gemm, packed_activations, linear_first, fused in (
            ("fp32", False, False, True), ("fp32", False, False, False), ("bf16", False, False, True),
            ("fp32", True, False, True), ("bf16", True, False, True), ("fp32", False, True, True),
            ("bf16", False, True, True), ("fp32", True, True, True), ("bf16", True, True, True),
            ("fp32", True, True, "folded"), ("bf16", True, True, "folded"),
            ("bf16x3", False, False, True), ("bf16x3", True, False, True),
            ("fp32", False, False, "all_nodes"), ("bf16", False, False, "all_nodes"), ("fp32", True, False, "all_nodes"),
            ("bf16", True, False, "all_nodes")):
        g = graph
        # the train step evaluates the last layer for the labelled rows only (the loss reads no others: same loss and
        # gradients); "all_nodes" sends every node through the last layer, as the reference's epoch does
        restrict = fused != "all_nodes"
        if not restrict:
            fused = True
        if fused == "folded":  # the degree division carried by the matrix values instead of the layers' epilogues
            if folded is None:
                from gnn_benchmark_amd import sage
                folded = sage.fold_in_degrees(graph)
                for m in (folded.local_adj_t, folded.adj_t_pre_post_aggr_from):
                    m.get_plan()
                    m.get_plan_for_transpose()
            g, fused = folded, True
        folded_tag = "_folded_degrees" if g is not graph else ""
        torch.manual_seed(args.seed)
        model = gcn.GCN(dims, gemm=gemm, packed_activations=packed_activations,
                        linear_first_when_narrowing=linear_first, fused_layers=fused).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        losses = [float(gcn.train_step(model, opt, g, x, labels, train_idx, True, masks, restrict)) for _ in range(2)]
        torch.cuda.synchronize()
        fell_through = gcn.LIBRARY_PRODUCTS["count"]
        t0 = time.perf_counter()
        for _ in range(steps):
            loss = gcn.train_step(model, opt, g, x, labels, train_idx, True, masks, restrict)
        torch.cuda.synchronize()
        tag = (f"{gemm}_gemm" + ("_packed_activations" if packed_activations else "")
               + ("_linear_first_when_narrowing" if linear_first else "") + ("" if fused else "_separate_kernels")
               + folded_tag + ("" if restrict else "_all_nodes_through_last_layer"))
        out[f"train_step_ms_{tag}"] = round((time.perf_counter() - t0) * 1e3 / steps, 2)
        out["library_products_per_step"] = max(out.get("library_products_per_step", 0),
                                               (gcn.LIBRARY_PRODUCTS["count"] - fell_through) // steps)
        out[f"loss_{tag}"] = [round(v, 5) for v in losses + [float(loss)]]
        del model, opt
    del folded
    # the default step with the local and the received elements of every output row in one launch (graph.one_launch),
    # in each form of the dense products
    graph.one_launch = True
    for gemm in ("fp32", "bf16x3", "bf16"):
        torch.manual_seed(args.seed)
        model = gcn.GCN(dims, gemm=gemm).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        losses = [float(gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)) for _ in range(2)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            loss = gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)
        torch.cuda.synchronize()
        out[f"train_step_ms_{gemm}_gemm_one_launch_aggregation"] = round((time.perf_counter() - t0) * 1e3 / steps, 2)
        out[f"loss_{gemm}_gemm_one_launch_aggregation"] = [round(v, 5) for v in losses + [float(loss)]]
        del model, opt
    graph.one_launch = False
    from gnn_benchmark_amd import synthetic
    from gnn_benchmark_amd.data_manager import CommBuffer, CommBufferForQuantization, CommSplits

    # the default step with the boundary rows of every layer travelling as bf16 / as int2 (the reference's runs
    # exchange at `--num_bits=2`); the rows a peer would have sent stand ready on the device
    world = len(graph.comm_splits.send_splits)
    fp32_splits, fp32_buf = graph.comm_splits, graph.comm_buf
    for bits, one_launch in ((16, False), (2, False), (2, True)):
        graph.one_launch = one_launch
        if bits == 16:
            graph.comm_buf = CommBuffer(fp32_splits, max(dims), 16, device=dev)
            synthetic.PregeneratedHaloExchange.attach(graph)
            graph.exchange_bf16 = synthetic.PregeneratedBf16HaloExchange(args.seed + 7)
        else:
            graph.comm_splits = CommSplits(fp32_splits.recv_splits, fp32_splits.send_splits, world, 2)
            graph.comm_buf_for_quantization = CommBufferForQuantization(graph.comm_splits, max(dims), 2, device=dev)
            graph.exchange_quantized = synthetic.PregeneratedQuantizedHaloExchange(args.seed + 6)
        torch.manual_seed(args.seed)
        model = gcn.GCN(dims, num_bits=bits).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        losses = [float(gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)) for _ in range(2)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            loss = gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)
        torch.cuda.synchronize()
        tag = ("fp32_gemm_bf16_exchange" if bits == 16 else "fp32_gemm_int2_exchange") + (
            "_one_launch_aggregation" if one_launch else "")
        out[f"train_step_ms_{tag}"] = round((time.perf_counter() - t0) * 1e3 / steps, 2)
        out[f"loss_{tag}"] = [round(v, 5) for v in losses + [float(loss)]]
        del model, opt
        graph.one_launch = False
        graph.comm_splits, graph.comm_buf = fp32_splits, fp32_buf
        graph.exchange_bf16 = graph.exchange_quantized = graph.comm_buf_for_quantization = None
        torch.cuda.empty_cache()
    # the same default step with the stand-in exchange drawing its rows inside the step (random-number kernels in
    # the timed region, which a real exchange would not run): how much of a step that was

    kept = graph.exchange
    graph.exchange = synthetic.SeededHaloExchange(kept.seed, std=kept.std, backward_std=kept.backward_std)
    torch.manual_seed(args.seed)
    model = gcn.GCN(dims).to(dev)
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    for _ in range(2):
        gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks, True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks, True)
    torch.cuda.synchronize()
    out["train_step_ms_fp32_gemm_halo_rows_drawn_inside_the_step"] = round((time.perf_counter() - t0) * 1e3 / steps, 2)
    graph.exchange = kept
    del model, opt
    return out


def run_c5_sage(args, graph):
    """The reference's own model on the same partition (DistSAGE: lin_neigh + lin_self per layer,
    dropout -> LayerNorm -> ReLU between layers), three ways: this build's layer stack (one
    stacked dense product per layer on [aggregated | x] kept side by side, fused elementwise
    chain), the same with the degree normalisation folded into the matrix values, that with the
    narrowing last layer applying lin_neigh before it aggregates, and -- as the yardstick -- plain
    torch ops around the same Aggregator, the way the reference writes them."""
    import torch
    import torch.nn.functional as F

    from gnn_benchmark_amd import Aggregator, sage

    dev = "cuda:0"
    n = graph.local_adj_t.sparse_size(0)
    dims = [128, 256, 256, 172]
    gen = torch.Generator(device=dev).manual_seed(args.seed + 6)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 10]
    steps = max(3, args.steps // 4)
    hidden = dims[1]
    masks = sage.make_dropout_masks(n, hidden, len(dims) - 1, 0.5, args.seed + 8, dev)
    out = {"layers": "DistSAGE %d->%d->%d->%d, LayerNorm, dropout 0.5" % tuple(dims), "steps": steps}

    from gnn_benchmark_amd import gcn

    def timed(step):
        losses = [float(step()) for _ in range(2)]
        torch.cuda.synchronize()
        fell_through = gcn.LIBRARY_PRODUCTS["count"]
        t0 = time.perf_counter()
        for _ in range(steps):
            loss = step()
        torch.cuda.synchronize()
        ms = round((time.perf_counter() - t0) * 1e3 / steps, 2)
        # dense products of one step that fell through to the BLAS library (0: none), the most over the forms
        out["library_products_per_step"] = max(out.get("library_products_per_step", 0),
                                               (gcn.LIBRARY_PRODUCTS["count"] - fell_through) // steps)
        return ms, [round(v, 5) for v in losses + [float(loss)]]

    staged = sage.stage_input(x)
    folded = None
    for tag, fold, linear_first, restrict, gemm in (
            ("", False, False, True, "fp32"), ("_folded_degrees", True, False, True, "fp32"),
            ("_folded_degrees_linear_first_when_narrowing", True, True, True, "fp32"),
            ("_folded_degrees_bf16x3_gemm", True, False, True, "bf16x3"),
            ("_folded_degrees_all_nodes_through_last_layer", True, False, False, "fp32"),
            ("_folded_degrees_one_launch_aggregation", True, False, True, "fp32")):
        if fold and folded is None:
            folded = sage.fold_in_degrees(graph)
        g = folded if fold else graph
        g.one_launch = tag.endswith("one_launch_aggregation")
        torch.manual_seed(args.seed)
        model = sage.DistSAGE(dims[0], hidden, dims[-1], num_layers=len(dims) - 1, dropout=0.5, is_pre_delay=True,
                              linear_first_when_narrowing=linear_first, gemm=gemm).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        ms, losses = timed(lambda: sage.train_step(model, opt, g, staged, labels, train_idx, masks, restrict))
        out["train_step_ms" + tag], out["loss" + tag] = ms, losses
        g.one_launch = False
        del model, opt, g
        torch.cuda.empty_cache()
    # the same step (degrees folded) with the boundary rows travelling as bf16 / as int2 -- the widths the reference's
    # own runs exchange at (`--num_bits=2 --is_pre_delay=true`); the rows a peer would have sent stand ready on the device
    from gnn_benchmark_amd import synthetic
    from gnn_benchmark_amd.data_manager import CommBuffer, CommBufferForQuantization, CommSplits

    world = len(graph.comm_splits.send_splits)
    fp32_splits, fp32_buf = folded.comm_splits, folded.comm_buf
    for tag, bits in (("_folded_degrees_bf16_exchange", 16), ("_folded_degrees_int2_exchange", 2),
                      ("_folded_degrees_int2_exchange_one_launch_aggregation", 2)):
        folded.one_launch = tag.endswith("one_launch_aggregation")
        if bits == 16:
            folded.comm_buf = CommBuffer(fp32_splits, hidden, 16, device=dev)
            synthetic.PregeneratedHaloExchange.attach(folded)
            folded.exchange_bf16 = synthetic.PregeneratedBf16HaloExchange(args.seed + 7)
        else:
            folded.comm_splits = CommSplits(fp32_splits.recv_splits, fp32_splits.send_splits, world, 2)
            folded.comm_buf_for_quantization = CommBufferForQuantization(folded.comm_splits, hidden, 2, device=dev)
            folded.exchange_quantized = synthetic.PregeneratedQuantizedHaloExchange(args.seed + 6)
        torch.manual_seed(args.seed)
        model = sage.DistSAGE(dims[0], hidden, dims[-1], num_layers=len(dims) - 1, dropout=0.5, num_bits=bits,
                              is_pre_delay=True).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        ms, losses = timed(lambda: sage.train_step(model, opt, folded, staged, labels, train_idx, masks, True))
        out["train_step_ms" + tag], out["loss" + tag] = ms, losses
        del model, opt
        folded.one_launch = False
        folded.comm_splits, folded.comm_buf = fp32_splits, fp32_buf
        folded.exchange_bf16 = folded.exchange_quantized = folded.comm_buf_for_quantization = None
        torch.cuda.empty_cache()
    del folded
    torch.cuda.empty_cache()

    class TorchOpsSage(torch.nn.Module):
        def __init__(self):
            super().__init__()
            widths = list(zip(dims[:-1], dims[1:]))
            self.lin_neigh = torch.nn.ModuleList([torch.nn.Linear(a, b, bias=False) for a, b in widths])
            self.lin_self = torch.nn.ModuleList([torch.nn.Linear(a, b, bias=False) for a, b in widths])
            self.bias = torch.nn.ParameterList([torch.nn.Parameter(torch.zeros(b)) for _, b in widths])
            self.norms = torch.nn.ModuleList([torch.nn.LayerNorm(b) for _, b in widths[:-1]])

        def forward(self, h):
            last = len(self.lin_neigh) - 1
            for i in range(last + 1):
                agg = Aggregator.apply(graph, h, i, 32, True, True)
                agg = agg / graph.in_degrees
                z = self.lin_neigh[i](agg) + self.lin_self[i](h) + self.bias[i]
                if i == last:
                    return F.log_softmax(z, dim=1)
                h = F.relu(self.norms[i](z * masks[i] * 2.0))

    torch.manual_seed(args.seed)
    model = TorchOpsSage().to(dev)
    opt = torch.optim.Adam(model.parameters(), lr=0.01)

    def torch_step():
        opt.zero_grad(set_to_none=True)
        loss = F.nll_loss(model(x)[train_idx], labels[train_idx])
        loss.backward()
        opt.step()
        return loss.detach()

    out["train_step_ms_torch_ops_around_aggregator"], out["loss_torch_ops_around_aggregator"] = timed(torch_step)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--feat", type=int, default=100)
    ap.add_argument("--nodes", type=int, default=2_450_000)
    ap.add_argument("--mean-out-degree", type=float, default=25.0)
    ap.add_argument("--c4-nodes", type=int, default=7_000_000)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--only", default="", help="'headline' = headline workload only; or a comma list of the extra "
                                                "workloads to add: c1 (single-rank 2-layer GCN), c2 (F=128/256 and "
                                                "the plan-less operator), c3, c4, c5 (GCN and SAGE train steps; "
                                                "c5sage: the SAGE one alone; "
                                                "ceilings: plain-kernel probes of the memory system).  Default: "
                                                "c1,c2,c3,c4,c5")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity-gate", action="store_true",
                    help="skip the comparison of the GPU results with the CPU operator in front of the number "
                         "(the line then says parity.checked = false)")
    ap.add_argument("--extra-out", default=os.path.join(ROOT, "bench_out", "bench_extra.json"),
                    help="side file for the full reports of the workloads besides the headline (also written to "
                         "stderr, one JSON line per workload as it finishes)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy 3 times (a kernel of known traffic for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    args.extras = [s for s in (args.only.split(",") if args.only else ["c1", "c2", "c3", "c4", "c5"])
                   if s and s != "headline"]
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the partitioned graph; --gpus must be 1 "
              "(no multi-GPU path exists in this build)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path)", file=sys.stderr)
        sys.exit(3)
    if args.copy_calibration:
        a = torch.ones(1 << 28, dtype=torch.float32, device="cuda:0")  # 1 GiB
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    gate = ParityGate(not args.no_parity_gate)
    sink = ExtraSink(args.extra_out)
    line = run_c2(args, gate, sink)
    torch.cuda.empty_cache()
    targets = {}
    if "c1" in args.extras:
        sink.put("c1", run_c1(args))
        torch.cuda.empty_cache()
    if "ceilings" in args.extras:
        sink.put("memory_ceilings", run_ceilings(args))
        torch.cuda.empty_cache()
    if "c3" in args.extras:
        sink.put("c3", run_c3(args))
        torch.cuda.empty_cache()
    if any(k in args.extras for k in ("c4", "c5", "c5sage")):
        _part, graph, setup_s = build_c4(args)
        if "c4" in args.extras:
            c4 = sink.put("c4", run_c4(args, graph, setup_s, gate))
            targets["c4"] = c4_targets(c4)
            torch.cuda.empty_cache()
            sink.put("c4_raw_halo", run_c4_raw_halo(args, _part))
            torch.cuda.empty_cache()
        if "c5" in args.extras:
            c5 = sink.put("c5", run_c5(args, graph))
            targets["c5_gcn_train_step_ms"] = {k[len("train_step_ms_"):]: c5[k] for k in (
                "train_step_ms_fp32_gemm", "train_step_ms_bf16_gemm", "train_step_ms_bf16x3_gemm",
                "train_step_ms_fp32_gemm_one_launch_aggregation", "train_step_ms_bf16x3_gemm_one_launch_aggregation",
                "train_step_ms_fp32_gemm_all_nodes_through_last_layer", "train_step_ms_fp32_gemm_int2_exchange",
                "train_step_ms_fp32_gemm_int2_exchange_one_launch_aggregation")
                if k in c5}
            targets["c5_gcn_train_step_ms"]["library_products"] = c5.get("library_products_per_step")
            torch.cuda.empty_cache()
        if "c5" in args.extras or "c5sage" in args.extras:
            c5s = sink.put("c5_sage", run_c5_sage(args, graph))
            targets["c5_sage_train_step_ms"] = {
                (k[len("train_step_ms_"):] if len(k) > len("train_step_ms") else "default"): c5s[k] for k in (
                    "train_step_ms", "train_step_ms_folded_degrees", "train_step_ms_folded_degrees_one_launch_aggregation",
                    "train_step_ms_folded_degrees_int2_exchange",
                    "train_step_ms_folded_degrees_int2_exchange_one_launch_aggregation",
                    "train_step_ms_torch_ops_around_aggregator") if k in c5s}
    line["parity"] = gate.report()
    line["targets"] = targets
    line["extra_file"] = sink.where()
    line["extra_keys"] = sorted(sink.keys)
    text = json.dumps(line, allow_nan=False, separators=(",", ":"))
    assert len(text) < MAX_LINE_BYTES, len(text)
    print(text, flush=True)


if __name__ == "__main__":
    main()
