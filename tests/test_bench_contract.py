"""The command-line contract of bench.py that can be checked without a GPU, and the shape of its
one JSON line where a GPU is there."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_algorithmic_byte_counts():
    # the figures the roofline is computed from: 2 x size for a copy; 2 x (q + k) + the table once
    sys.path.insert(0, ROOT)
    import bench
    assert bench.HBM_PEAK_GBPS == 8000.0
    q, k, table = 8 * 4096 * 32 * 128 * 2, 8 * 4096 * 8 * 128 * 2, 4096 * 128 * 4
    assert 2 * (q + k) + table == 673185792
    # measured traffic constants stay within 1 % of those algorithmic bytes
    assert abs(bench.COPY_256MIB_TRAFFIC_BYTES / (2 * 256 * 2 ** 20) - 1) < 0.01
    assert abs(bench.ROPE_STEP_TRAFFIC_BYTES / 673185792 - 1) < 0.01
    sizes = bench.churn_sizes()
    assert len(sizes) == 10000 and min(sizes) >= 4096 and max(sizes) <= 512 * 2 ** 20 and all(s % 16 == 0 for s in sizes)
    assert sizes == bench.churn_sizes()                          # seeded


@pytest.mark.gpu
def test_quick_run_prints_one_json_line_with_roofline_and_cpu_baseline():
    print("bench.py --quick", flush=True)
    proc = subprocess.run([sys.executable, BENCH, "--quick", "--steps", "10", "--warmup", "2"],
                          capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    r = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in r, key
    assert r["n_gpus"] == 1 and r["steps"] == 10 and r["warmup"] == 2 and r["vs_baseline"] is None
    assert r["unit"] == "GB/s" and r["dtype"] == "u8" and r["config"]["bit_exact"] is True
    roof = r["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9 and 0.3 < roof["frac"] < 1.0
    assert abs(r["value"] - 2 * 256 * 2 ** 20 / (r["ms_per_step"] * 1e-3) / 1e9) < 1.0
    rope = r["roofline_rope_bf16"]
    assert rope["bound"] == "hbm" and rope["peak"] == 8000.0 and 0.3 < rope["frac"] < 1.0
    assert abs(rope["frac"] - rope["achieved"] / rope["peak"]) < 1e-9
    assert abs(rope["achieved"] - 673185792 / (rope["ms_per_step"] * 1e-3) / 1e9) < 1.0
    assert "cycle over 8 distinct" in r["config"]["workload"]
    cpu = r["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] == 1 and cpu["value"] > 0
    assert r["library_error"] is None
