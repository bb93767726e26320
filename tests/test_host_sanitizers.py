"""The host components of the c10d surface (in-process mesh with its polling meeting point,
FIFO engine, byte transport) under ThreadSanitizer and AddressSanitizer + UBSan on the CPU:
groups of 2-4 rank threads created, used and torn down a few hundred times
(tests/native/mesh_stress.cpp).  No GPU and no torch involved."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
OUT = os.path.join(HERE, "native", "_build")
SOURCES = [os.path.join(HERE, "native", "mesh_stress.cpp"),
           os.path.join(ROOT, "mccl_amd", "csrc", "backend", "LocalMesh.cpp"),
           os.path.join(ROOT, "mccl_amd", "csrc", "backend", "Progress.cpp")]


def build(name, flags):
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, name)
    cmd = ["g++", "-std=c++17", "-O1", "-g", *flags, "-I" + os.path.join(ROOT, "mccl_amd", "csrc"),
           "-I" + os.path.join(ROOT, "include"), *SOURCES, "-o", exe, "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0 and ("cannot find" in r.stderr or "No such file" in r.stderr):
        pytest.skip("this toolchain lacks the sanitizer runtime: " + r.stderr.strip().splitlines()[-1])
    assert r.returncode == 0, r.stderr
    return exe


@pytest.mark.skipif(shutil.which("g++") is None, reason="no g++")
@pytest.mark.parametrize("name,flags,spin", [
    ("mesh_stress_tsan", ["-fsanitize=thread", "-DWAIT_MS=0"], "200"),
    ("mesh_stress_tsan", ["-fsanitize=thread", "-DWAIT_MS=0"], "0"),
    ("mesh_stress_asan", ["-fsanitize=address,undefined", "-DWAIT_MS=20000"], "200"),
])
def test_groups_of_rank_threads_come_and_go_under_a_sanitizer(name, flags, spin):
    exe = build(name, flags)
    env = dict(os.environ, MCCL_MEET_SPIN_US=spin)
    r = subprocess.run([exe, "150"], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "ok: 150 groups" in r.stdout
    assert "ThreadSanitizer" not in r.stderr and "AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-4000:]
