#!/usr/bin/env python3
"""Benchmark of the aggregation hot path on ONE MI355X.

Default workload ("c2"): standalone CSR SpMM forward A @ X plus the transposed backward
A^T @ G on a seeded power-law graph of 2.45 M nodes / ~124 M stored elements with
GCN-normalised fp32 values and a 2.45 M x 100 fp32 dense operand.  One "step" is one
forward plus one backward, with every input already resident in HBM.

Prints ONE JSON line.  ``value`` is the FLOP rate of the whole step (2 * nnz * F per
product).  ``roofline`` prices the dominant kernel (the forward's row kernel) against
the 8 TB/s HBM peak with the no-reuse gather byte model:
    bytes = nnz*(8+4) + (rows+1)*8 + nnz*F*4 + 2*rows*F*4
over the rows / stored elements that kernel launch covers, divided by its duration
measured with HIP events on the launch stream inside the timed region.
``cpu_baseline`` is the reference's own compiled operator (or the C port of it when
that is not available on the host) timed on this machine's cores on the same matrices.
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


def b_alg(nnz: int, rows: int, feat: int) -> float:
    """Algorithmic bytes of one out += A @ X call (no-reuse gather model)."""
    return nnz * 12.0 + (rows + 1) * 8.0 + nnz * feat * 4.0 + 2.0 * rows * feat * 4.0


def b_min(nnz: int, rows: int, cols: int, feat: int) -> float:
    """Compulsory floor: the dense operand read once."""
    return nnz * 12.0 + (rows + 1) * 8.0 + cols * feat * 4.0 + 2.0 * rows * feat * 4.0


def rows_kernel_cover(src, plan_info):
    """(rows, nnz) covered by the dominant kernel launch with accumulate=1: every row
    that has a stored element (empty rows are not visited)."""
    rowptr = src.csr()[0]
    return plan_info["rows"] - plan_info["empty_rows"], int(rowptr[-1])


def time_spmm(plan, value, x, out, steps, warmup):
    """Median/mean of the dominant-kernel and whole-call durations over `steps` calls."""
    import torch

    plan.profile(True)
    k_ms, c_ms = [], []
    for i in range(warmup + steps):
        plan.spmm(value, x, out, accumulate=True)
        k, c = plan.profile_read()
        if i >= warmup:
            k_ms.append(k)
            c_ms.append(c)
    plan.profile(False)
    return sum(k_ms) / len(k_ms), sum(c_ms) / len(c_ms), min(c_ms)


def cpu_baseline_spmm(src, x_host, g_host, reps=3):
    """Forward + transposed backward on the host cores with the reference's compiled
    operator when oracle/_ref holds it (kind "reference"), else the C port (kind "port")."""
    import numpy as np
    import torch

    from oracle import spmm as ospmm

    threads = ospmm.max_threads()
    rowptr, col, val = [t.cpu().numpy() for t in src.csr()]
    colptr = src.storage.colptr().cpu().numpy()
    row_t = src.storage.row_T().cpu().numpy()
    val_t = src.storage.value_T().cpu().numpy()
    rows, cols = src.sparse_sizes()
    feat = x_host.shape[1]
    # the reference balances its threads on per-row work (model/ops/spmm_kernel.py:7-28); unit weights = nnz
    rs_f = ospmm.distribute_work_for_row(rowptr, np.ones(col.shape[0], np.float32), threads)
    rs_b = ospmm.distribute_work_for_row(colptr, np.ones(col.shape[0], np.float32), threads)
    ref = ospmm.load_reference_op()
    out_f = np.zeros((rows, feat), dtype=np.float32)
    out_b = np.zeros((cols, feat), dtype=np.float32)
    if ref is not None:
        kind = "reference"
        torch.set_num_threads(threads)
        t = lambda a: torch.from_numpy(a)  # noqa: E731
        cs = torch.tensor([0, feat], dtype=torch.int32)
        args_f = (t(rowptr), t(col), t(val), t(x_host), t(out_f), rows, t(rs_f), cs)
        args_b = (t(colptr), t(row_t), t(val_t), t(g_host), t(out_b), cols, t(rs_b), cs)

        def run():
            ref.spmm(*args_f)
            ref.spmm(*args_b)
    else:
        kind = "port"

        def run():
            ospmm.spmm(rowptr, col, val, x_host, out_f, rs_f, threads)
            ospmm.spmm(colptr, row_t, val_t, g_host, out_b, rs_b, threads)

    run()  # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    sec = times[len(times) // 2]
    flops = 2 * 2.0 * col.shape[0] * feat
    return {"value": round(flops / sec / 1e9, 3), "unit": "GFLOP/s", "cores": int(threads), "kind": kind,
            "sample": f"full workload: 1 forward + 1 transposed backward, F={feat}, median of {reps} after 1 warm-up",
            "ms_per_step": round(sec * 1e3, 2)}


def run_c2(args):
    import torch

    from gnn_benchmark_amd import synthetic

    dev = "cuda:0"
    feat = args.feat
    t0 = time.perf_counter()
    g = synthetic.power_law_graph(num_nodes=args.nodes, mean_out_degree=args.mean_out_degree, zipf_s=1.8,
                                  max_degree=15000, seed=args.seed, device=dev)
    src = g.adj
    n, nnz = g.num_nodes, g.nnz
    plan_f = src.get_plan()
    plan_b = src.get_plan_for_transpose()
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    info = plan_f.info()
    _, _, val = src.csr()
    val_t = src.storage.value_T()

    results = {}
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    feats = [feat] + [f for f in args.extra_feats if f != feat]
    main = None
    for f in feats:
        x = torch.randn(n, f, device=dev, generator=gen)
        gr = torch.randn(n, f, device=dev, generator=gen)
        out = torch.zeros(n, f, device=dev)
        dx = torch.zeros(n, f, device=dev)
        steps, warmup = (args.steps, args.warmup) if f == feat else (max(3, args.steps // 4), 2)
        # whole-step timing: exactly `steps` steps between two synchronisations
        for _ in range(warmup):
            plan_f.spmm(val, x, out, True)
            plan_b.spmm(val_t, gr, dx, True)
        plan_f.profile(True)
        k_ms = []
        torch.cuda.synchronize()
        t_begin = time.perf_counter()
        for _ in range(steps):
            plan_f.spmm(val, x, out, True)
            plan_b.spmm(val_t, gr, dx, True)
            k_ms.append(plan_f.profile_read()[0])
        torch.cuda.synchronize()
        ms_step = (time.perf_counter() - t_begin) * 1e3 / steps
        plan_f.profile(False)
        kern_ms = sum(k_ms) / len(k_ms)
        rows_cov, nnz_cov = rows_kernel_cover(src, info)
        bytes_launch = b_alg(nnz_cov, rows_cov, f)
        # separate forward / backward whole-call timings
        _, fwd_ms, _ = time_spmm(plan_f, val, x, out, max(3, steps // 2), 1)
        _, bwd_ms, _ = time_spmm(plan_b, val_t, gr, dx, max(3, steps // 2), 1)
        r = {
            "feat": f, "ms_per_step": round(ms_step, 4), "fwd_ms": round(fwd_ms, 4), "bwd_ms": round(bwd_ms, 4),
            "gflops": round(2 * 2.0 * nnz * f / (ms_step * 1e-3) / 1e9, 2),
            "fwd_gbs_model": round(b_alg(nnz, n, f) / (fwd_ms * 1e-3) / 1e9, 1),
            "fwd_frac_of_hbm_peak": round(b_alg(nnz, n, f) / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "bwd_gbs_model": round(b_alg(nnz, n, f) / (bwd_ms * 1e-3) / 1e9, 1),
            "fwd_gbs_floor": round(b_min(nnz, n, n, f) / (fwd_ms * 1e-3) / 1e9, 1),
            "kernel_ms": round(kern_ms, 4), "kernel_bytes": bytes_launch, "steps": steps,
        }
        results[f] = r
        if f == feat:
            main = (r, x, gr)
        else:
            del x, gr
        del out, dx
    r, x, gr = main
    line = {
        "metric": "spmm_fwd_bwd_gflops", "value": r["gflops"], "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"c2: CSR SpMM forward A@X + transposed backward A^T@G, power-law graph "
                               f"{n} nodes / {nnz} nnz (Zipf s=1.8, max row {g.max_degree}), GCN-normalised fp32, "
                               f"dense operand {n}x{feat} fp32",
                   "nodes": n, "nnz": nnz, "feat": feat, "seed": args.seed, "long_rows": info["long_rows"],
                   "max_row_len": info["max_row_len"], "setup_s": round(setup_s, 2)},
        "roofline": {"bound": "hbm", "achieved": round(r["kernel_bytes"] / (r["kernel_ms"] * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(r["kernel_bytes"] / (r["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "kernel": "spmm_tasks_kernel (forward A@X, all rows)",
                     "kernel_ms": r["kernel_ms"], "bytes_per_launch": r["kernel_bytes"]},
        "extra": {"c2": [results[f] for f in feats]},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_spmm(src, x.cpu().numpy(), gr.cpu().numpy())
    else:
        line["cpu_baseline"] = None
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=["c2"])
    ap.add_argument("--feat", type=int, default=100)
    ap.add_argument("--extra-feats", type=int, nargs="*", default=[128, 256])
    ap.add_argument("--nodes", type=int, default=2_450_000)
    ap.add_argument("--mean-out-degree", type=float, default=25.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy 3 times (a kernel of known traffic for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
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
    line = run_c2(args)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
