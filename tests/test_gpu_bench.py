"""bench.py end to end on the GPU, at a handful of steps: one JSON line with the fields the
measurement contract names, the launch checked bit for bit against the oracle inside the run."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_headline_line_has_its_fields_and_parity():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "8", "--warmup", "3", "--no-extras",
                        "--cpu-seconds", "1"], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    d = json.loads(lines[0])
    assert d["n_gpus"] == 1 and d["steps"] == 8 and d["warmup"] == 3 and d["unit"] == "GB/s" and d["higher_is_better"] is True
    assert d["dtype"] == "bf16" and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert d["config"]["parity_vs_oracle_bit_exact"] is True and d["config"]["algorithmic_bytes_per_step"] == 78_643_200
    assert d["config"]["workload"].startswith("C2")
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(roof["achieved"] - 78.6432 / roof["kernel_us"] * 1e3) < 0.01 * roof["achieved"]
    assert 0.5 < roof["frac"] < 1.0, "a fold launch of 78.6 MB neither crawls nor beats the memory's peak"
    assert 0.99 < roof["traffic"] / 78_643_200 < 1.02
    assert d["value"] <= roof["achieved"] * 1.02, "the wall clock cannot beat the device's own time"
    assert abs(d["ms_per_step"] * 1e3 - 78.6432 / d["value"] * 1e3) < 0.02 * d["ms_per_step"] * 1e3
    cpu = d["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "GB/s" and cpu["cores"] >= 1 and 0 < cpu["value"] < 1000
    gate = d["extra"]["hold_gate"]
    assert gate["latency_ticks"] == 40 and 40_000 < gate["bytes_per_tick"] < 110_000
