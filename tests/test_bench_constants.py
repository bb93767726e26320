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


def test_the_headline_range_in_the_readme_covers_the_committed_measurements():
    """README.md quotes the headline launch as a range of microseconds; the figures it stands for are
    the unprofiled runs quoted in the kernel-trace profile (the driver's command line and the
    default step count) and the headline row of the design document's measured table."""
    readme = open(os.path.join(ROOT, "README.md")).read()
    m = re.search(r"runs in (\d+\.\d+)–(\d+\.\d+) µs per launch", readme)
    assert m, "README.md no longer states the headline as a range"
    lo, hi = float(m.group(1)), float(m.group(2))
    assert 0 < lo <= hi < 1.05 * lo, "a range wider than 5 % says nothing"
    prof = open(os.path.join(ROOT, "profiles", "c2_fold_kernel_trace.txt")).read()
    runs = [float(x) for x in re.findall(r"Unprofiled run of the same command[^\n]*?kernel_us (\d+\.\d+)", prof)]
    assert len(runs) == 2, "the profile quotes one unprofiled run per command line"
    design = open(os.path.join(ROOT, "DESIGN.md")).read()
    row = re.search(r"\*\*C2 fused fold, cold \(headline\)\*\* \| \*\*(\d+\.\d+) µs[^|]*\| \*\*(\d+\.\d+) µs", design)
    assert row, "the design document's measured table has no headline row"
    for us in runs + [float(row.group(1)), float(row.group(2))]:
        assert lo <= us <= hi, (us, lo, hi)
    # and the fraction of the peak that goes with it
    pct = re.search(r"\((\d+)–(\d+) %\s+of the 8 TB/s HBM peak", readme)
    assert pct and abs(78.6432 / hi / 8 * 100 - int(pct.group(1))) <= 1 and abs(78.6432 / lo / 8 * 100 - int(pct.group(2))) <= 1


def test_more_than_one_gpu_is_refused_with_a_message():
    """This build measures one GPU's share of the path: `bench.py --gpus N` with N above 1 says so and exits."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "single GPU" in r.stderr and r.stdout.strip() == ""
