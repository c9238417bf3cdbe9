"""bench.py's output contract: exactly one JSON line with the agreed keys; more than one GPU is refused."""
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


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--nodes", "60000", "--mean-out-degree", "10",
                        "--steps", "3", "--warmup", "1", "--only", "headline"], capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
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
    fwd = d["extra"]["c2"][0]["forward"]
    assert "frac_model" in fwd and "frac_of_hbm_peak" not in fwd and "frac_measured" not in fwd  # (no profile for this size)


@pytest.mark.gpu
def test_smoke_entry_point_runs_and_checks_itself():
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry

    entry.smoke()  # raises on any mismatch with the oracle
