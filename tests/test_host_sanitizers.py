"""The host components of the c10d surface (in-process mesh with its polling meeting point,
FIFO engine, byte transport) under ThreadSanitizer and AddressSanitizer + UBSan on the CPU:
groups of 2-4 rank threads created, used and torn down a few hundred times
(tests/native/mesh_stress.cpp; no GPU and no torch involved), and the whole c10d backend --
ProcessGroupMCCL, Work, Future completion, completer, registries, chunk scheduler -- compiled
with -DMCCL_NULL_DEVICE over a host stand-in of the kernel layer (tests/native/pg_stress.cpp,
null_mcclx.cpp; libtorch's CPU libraries only), where the last reference to a group is dropped
on its own engine thread and on the completer thread."""
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


# ---- the whole backend over a host stand-in of the kernel layer ---------------------------------

PG_SOURCES = [os.path.join(HERE, "native", "pg_stress.cpp"), os.path.join(HERE, "native", "null_mcclx.cpp"),
              os.path.join(ROOT, "mccl_amd", "csrc", "mcclx_sched.cpp")] + \
             [os.path.join(ROOT, "mccl_amd", "csrc", "backend", f)
              for f in ("ProcessGroupMCCL.cpp", "WorkMCCL.cpp", "Progress.cpp", "LocalMesh.cpp", "HostWire.cpp")]


def build_pg(name, flags):
    import torch
    from torch.utils import cpp_extension as ce
    out = os.path.join(OUT, name + "_obj")
    os.makedirs(out, exist_ok=True)
    exe = os.path.join(OUT, name)
    newest = max(os.path.getmtime(p) for p in PG_SOURCES + [os.path.join(ROOT, "include", "mcclx.h")] +
                 [os.path.join(ROOT, "mccl_amd", "csrc", "backend", f)
                  for f in os.listdir(os.path.join(ROOT, "mccl_amd", "csrc", "backend")) if f.endswith(".hpp")])
    if os.path.exists(exe) and os.path.getmtime(exe) >= newest:
        return exe
    inc = ["-I" + p for p in ce.include_paths()] + ["-I" + os.path.join(ROOT, "mccl_amd", "csrc"),
                                                     "-I" + os.path.join(ROOT, "include")]
    common = ["g++", "-std=c++17", "-O1", "-g", "-DMCCL_NULL_DEVICE=1", "-Wno-unknown-pragmas",
              "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), *flags, *inc]
    procs, objs = [], []
    for src in PG_SOURCES:
        obj = os.path.join(out, os.path.basename(src) + ".o")
        objs.append(obj)
        procs.append(subprocess.Popen(common + ["-c", src, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    for p in procs:
        text, _ = p.communicate()
        if p.returncode != 0 and ("cannot find" in text or "No such file" in text and "sanitizer" in text):
            pytest.skip("this toolchain lacks the sanitizer runtime")
        assert p.returncode == 0, text[-4000:]
    lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    r = subprocess.run(["g++", *flags, *objs, "-o", exe, "-L" + lib, "-ltorch_cpu", "-lc10", "-Wl,-rpath," + lib, "-lpthread"],
                       capture_output=True, text=True)
    if r.returncode != 0 and "cannot find" in r.stderr and "san" in r.stderr:
        pytest.skip("this toolchain lacks the sanitizer runtime: " + r.stderr.strip().splitlines()[-1])
    assert r.returncode == 0, r.stderr[-4000:]
    return exe


@pytest.mark.skipif(shutil.which("g++") is None, reason="no g++")
@pytest.mark.parametrize("name,flags,groups", [
    ("pg_stress_asan", ["-fsanitize=address,undefined", "-DWAIT_MS=20000"], "90"),
    ("pg_stress_tsan", ["-fsanitize=thread", "-DWAIT_MS=0"], "60"),
])
def test_process_groups_come_and_go_and_die_on_their_own_threads_under_a_sanitizer(name, flags, groups):
    exe = build_pg(name, flags)
    env = dict(os.environ, MCCL_MEET_SPIN_US="50", ASAN_OPTIONS="detect_leaks=0",
               TSAN_OPTIONS="report_signal_unsafe=0 history_size=4")
    env.pop("MCCL_ABORT_BACKTRACE", None)
    r = subprocess.run([exe, groups], capture_output=True, text=True, timeout=900, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert f"ok: {groups} groups" in r.stdout
    assert "ThreadSanitizer" not in r.stderr and "AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-6000:]
