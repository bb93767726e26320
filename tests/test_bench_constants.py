"""bench.py reports the HBM traffic of the C2 launch as a constant (counters cannot be
read from inside the process); the constant must be the total the tracked rocprofv3
summary arrives at, so that it cannot go stale without a test noticing."""
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_constant_equals_the_profile_total():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    text = open(os.path.join(ROOT, "profiles", "c2_fold_hbm_traffic_pmc.txt")).read()
    m = re.search(r"total\s+(\d+) B of HBM traffic vs 78,643,200 algorithmic bytes", text)
    assert m, "the profile summary no longer states the total"
    assert int(m.group(1)) == bench.C2_MEASURED_TRAFFIC_BYTES
    read = re.search(r"read\s+[\d.]+ KiB = (\d+) B", text)
    write = re.search(r"write\s+[\d.]+ KiB = (\d+) B", text)
    assert abs(int(read.group(1)) + int(write.group(1)) - int(m.group(1))) <= 2   # rounding of the two parts
    assert 0.99 < int(m.group(1)) / 78_643_200 < 1.02, "traffic well above the algorithmic bytes means wasted re-reads"
