"""The bench line's contract on a GPU box, on a workload small enough for the test suite: `bench.py --workload` in a
child process, one JSON line on stdout with the fields the driver and the docs rely on, parity checked inside."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-3000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1, p.stdout[-2000:]
    return json.loads(lines[0])


def _check_contract(d, steps, warmup):
    assert d["unit"] == "keys/s" and d["n_gpus"] == 1 and d["steps"] == steps and d["warmup"] == warmup
    assert d["higher_is_better"] is True and d["scaling"] == "weak" and d["vs_baseline"] is None
    assert d["dtype"] == "u8" and d["data"] == "synthetic" and "workload" in d["config"]
    assert d["value"] > 0 and d["ms_per_step"] > 0
    n = d["config"]["keys_per_batch"]
    assert abs(d["value"] - n / (d["ms_per_step"] * 1e-3)) < 1e-6 * d["value"]
    r = d["roofline"]
    assert r["bound"] in ("hbm", "mfma") and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9 and 0 < r["frac"] < 1
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["value"] > 0 and c["cores"] >= 1 and c["sample"]
    assert "bit-exact" in d["parity"]


def test_mixed_workload_line_with_the_serving_loop():
    d = _bench("--workload", "small_mixed_4Mx128xfp32_262144_i64_zipf0.9_cache25pct", "--steps", "12", "--warmup", "3",
               "--cpu-seconds", "0.2", "--serving")
    _check_contract(d, 12, 3)
    link = d["host_link"]
    assert 0 < link["frac"] <= 1.05 and link["achieved"] > 0
    # the CPU leg both ways: the whole step (lookup + per-row source + copy) and a plain gather by row number
    c = d["cpu_baseline"]
    assert c["gather_by_row_number"]["value"] > 0 and c["gather_by_row_number"]["cores"] == c["cores"]
    assert 0 < c["rows_from_cache_copy_first_batch"] < 262_144
    assert abs(d["gpu_over_cpu"] - d["value"] / c["value"]) < 1e-6 * d["gpu_over_cpu"]
    b = d["cache_build"]
    assert b["seconds"] > 0 and b["rows_filled"] == d["config"]["cached_rows"] and b["bytes_filled"] == b["rows_filled"] * 512
    s = d["serving_loop"]
    assert s["steps"] == 12 and s["ms_per_step"] > 0 and s["refreshes_completed"] >= 1
    assert sum(s["steps_of_each"]) == 12 and s["hotness_recorded_on"] == "host"


def test_all_hit_workload_line():
    d = _bench("--workload", "c2_all_hit_10Mx128xfp32_262144_u32_uniform", "--steps", "20", "--warmup", "5",
               "--cpu-seconds", "0.2")
    _check_contract(d, 20, 5)
    assert d["roofline"]["frac"] > 0.5  # the gather kernel alone, 262,144 rows of 512 bytes
    assert d["stream_ordered"]["keys_per_s"] > d["value"] * 0.9
