"""bench.py's output contract: exactly one compact, strict-JSON line on stdout with the agreed keys (the full
reports of the other workloads go to stderr and a side file); more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and not r.stdout.strip()


def _strict(text):
    def refuse(name):
        raise ValueError(f"{name} is not strict JSON")

    return json.loads(text, parse_constant=refuse)


def test_the_compact_line_of_the_default_argument_set_stays_small(tmp_path):
    """The assembly of the stdout line -- the code path of the default argument set, fed with reports of the shape
    the workloads produce -- stays a few KB of strict JSON however much the workloads report (no GPU needed)."""
    sys.path.insert(0, ROOT)
    import bench

    sink = bench.ExtraSink(str(tmp_path / "extra.json"))
    op = lambda name, run: {"op": name, "ms": 2.5, "frac_model": 0.7, "frac_measured": 0.72,  # noqa: E731
                            "as_run_by_aggregator": run, "filler": "x" * 500}
    names = ["pre-aggregation A_to@X -> send_buf", "local A_local@X -> out", "post-aggregation A_from@recv_buf -> out",
             "pre-aggregation transposed (gradient direction)", "local transposed (gradient direction)",
             "post-aggregation transposed (gradient direction)"]
    c4 = sink.put("c4", {"feat": 128, "ops": [op(n + s, s == "") for n in names for s in ("", " (overwriting)")],
                         "aggregator_forward_ms": 13.2, "aggregator_forward_backward_ms": 27.0, "bad": float("nan")})
    assert c4["bad"] == "nan"   # non-finite values are named, the files stay strict JSON
    targets = bench.c4_targets(c4)
    assert sorted(targets["products_ms_fracmodel_fracmeasured"]) == ["local", "local_T", "post", "post_T", "pre", "pre_T"]
    assert targets["min_frac_model"] == 0.7
    sink.put("c5", {f"train_step_ms_variant_{i}": 100.0 + i for i in range(60)})
    gate = bench.ParityGate(True)
    gate.kind = "reference, 16 threads"
    import numpy as np

    a = np.ones((5, 4), np.float32)
    gate.record("c2_forward", a, a.copy(), "A@X")
    line = {"metric": "spmm_fwd_bwd_gflops", "value": 1.0, "config": {"workload": "w" * 300}, "roofline": {"k": "r" * 300},
            "cpu_baseline": {"protocol": "p" * 200}, "parity": gate.report(), "targets": {"c4": targets},
            "extra_file": sink.where(), "extra_keys": sorted(sink.keys)}
    text = json.dumps(line, allow_nan=False, separators=(",", ":"))
    assert len(text) < bench.MAX_LINE_BYTES < 8192
    assert _strict(text)["parity"] == {"checked": True, "tolerance": "abs 1e-06 + rel 1e-05",
                                       "against": "CPU operator (reference, 16 threads)", "max_excess": -1e-06,
                                       "bit_identical": True, "cases": {"c2_forward": [-1e-06, True]}}
    assert sorted(_strict(open(tmp_path / "extra.json").read())) == ["c4", "c5"]


def test_a_result_outside_the_tolerance_stops_the_bench_without_a_number(capsys):
    sys.path.insert(0, ROOT)
    import numpy as np

    import bench

    gate = bench.ParityGate(True)
    want = np.ones((3, 4), np.float32)
    got = want.copy()
    got[1, 2] += 1e-3
    with pytest.raises(SystemExit) as e:
        gate.record("c2_forward", got, want, "A@X")
    assert e.value.code == 4
    captured = capsys.readouterr()
    assert "parity gate FAILED" in captured.err and not captured.out


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline(tmp_path):
    side = str(tmp_path / "extra.json")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--nodes", "60000", "--mean-out-degree", "10",
                        "--steps", "3", "--warmup", "1", "--only", "headline", "--extra-out", side],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and len(lines[0]) < 8192
    d = _strict(lines[0])
    assert "extra" not in d and d["extra_keys"] == ["c2_headline"]
    assert d["parity"]["checked"] is True and d["parity"]["bit_identical"] is True and d["parity"]["max_excess"] <= 0
    assert sorted(d["parity"]["cases"]) == ["c2_backward", "c2_forward"]
    assert d["metric"] == "spmm_fwd_bwd_gflops" and d["unit"] == "GFLOP/s" and d["value"] > 0
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["ms_per_step"] > 0
    assert d["higher_is_better"] is True and d["vs_baseline"] is None and d["dtype"] == "f32" and d["data"] == "synthetic"
    assert isinstance(d["config"]["workload"], str) and "model" not in d["config"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert roof["traffic"] is None  # measured traffic exists for the default workload only
    cpu = d["cpu_baseline"]
    assert cpu["kind"] in ("reference", "port") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["unit"] == "GFLOP/s"
    assert isinstance(cpu["sample"], str)
    assert isinstance(cpu["cpu_model"], str) and cpu["host_physical_cores"] >= 1 and "2 warm-ups" in cpu["protocol"]
    fwd = _strict(open(side).read())["c2_headline"]["forward"]
    assert "frac_model" in fwd and "frac_of_hbm_peak" not in fwd and "frac_measured" not in fwd  # (no profile for this size)


@pytest.mark.gpu
def test_smoke_entry_point_runs_and_checks_itself():
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry

    entry.smoke()  # raises on any mismatch with the oracle
