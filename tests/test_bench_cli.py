"""The benchmark's command line: what the driver relies on."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
def test_quick_run_prints_one_json_line_with_the_contract_keys(built_library):
    r = subprocess.run([sys.executable, BENCH, "--quick", "--steps", "20", "--warmup", "5"], capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 5 and d["vs_baseline"] is None
    assert d["unit"] == "TFLOP/s" and d["higher_is_better"] is True and "workload" in d["config"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9
    assert abs(d["value"] - 2.0 * 128 * 2048 * 512 * 0.1 * 256 / d["ms_per_step"] / 1e9) / d["value"] < 0.02


@pytest.mark.gpu
def test_default_path_ends_in_a_short_parsable_line(built_library, tmp_path):
    """The run the driver records (no --quick): the LAST line of stdout is valid JSON, shorter than 4 KiB, and carries
    the roofline and the CPU baseline; the full dictionary of figures goes to the extras file."""
    extras = str(tmp_path / "bench_extra.json")
    r = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--extras-file", extras],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-3000:]
    last = [l for l in r.stdout.splitlines() if l.strip()][-1]
    assert len(last.encode()) < 4096, len(last)
    d = json.loads(last)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity_max_rel_err", "extra"):
        assert key in d, key
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "alg_bytes_per_launch"):
        assert key in roof, key
    assert roof["bound"] == "hbm" and 0.0 < roof["frac"] < 1.0
    assert roof["traffic"] is not None and roof["traffic"] > 0.9 * roof["alg_bytes_per_launch"]
    cpu = d["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] == 1 and cpu["value"] > 0 and cpu["unit"] == "TFLOP/s"
    assert d["parity_max_rel_err"] <= 1e-2
    assert len(d["extra"]) <= 12 and all(not isinstance(v, (dict, list)) for v in d["extra"].values())
    with open(extras) as f:
        full = json.load(f)
    assert full["value"] == d["value"] and len(full["extra"]) > len(d["extra"])


def test_traffic_table_is_read_from_the_profile_summaries():
    sys.path.insert(0, ROOT)
    import bench
    t = bench.measured_traffic()
    assert "headline_batch128" in t
    row = t["headline_batch128"]
    assert row["source"].startswith("profiles/") and os.path.exists(os.path.join(ROOT, row["source"]))
    assert 0.9 < row["bytes"] / row["alg_bytes"] < 1.5


def test_parity_gate_finds_failures_anywhere_in_the_tree():
    sys.path.insert(0, ROOT)
    import bench
    tree = {"a": {"max_rel_err_vs_host_loop": 1e-6}, "b": {"c": {"spmm_max_rel_err_vs_host_loop": 0.5}},
            "d": {"svc_bit_exact_vs_python": False}, "e": {"bit_exact_vs_python": True}}
    assert sorted(bench.parity_failures(tree)) == ["b/c/spmm_max_rel_err_vs_host_loop", "d/svc_bit_exact_vs_python"]
    nan = {"x": {"max_rel_err_vs_host_loop": float("nan")}}
    assert list(bench.parity_failures(nan)) == ["x/max_rel_err_vs_host_loop"]
