"""Compiles libmcclx.so (HIP kernels + C ABI + chunk scheduler) for gfx950.

hipcc cross-compiles without a GPU.  The shared library is written next to this
file so that it travels with the source tree; objects go to build/.

    python -m mccl_amd.build            # build if sources are newer than the library
    python -m mccl_amd.build --force
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(ROOT, "build", "mcclx")
LIB_PATH = os.path.join(HERE, "libmcclx.so")

SOURCES = ["fold_kernels.hip", "copy_kernel.hip", "static_table.hip", "mcclx_api.cpp", "mcclx_sched.cpp"]
FOLD_PARTS = 7  # fold_kernels.hip is compiled once per part (-DMCCLX_PART=n), in parallel
HEADERS = ["fold_launch.h", "mcclx_internal.h", os.path.join(ROOT, "include", "mcclx.h")]

# -ffp-contract=off / -fno-fast-math: IEEE fp32 add and mul, no FMA fusion, so
# the kernels match the CPU oracle bit for bit.  Denormals are kept (hipcc's
# default for gfx9).  Packed-FP32 instructions are disabled.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fvisibility=hidden", "-Wall", "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libmcclx.so cannot be built")
    return exe


def _newest_source_mtime() -> float:
    paths = [os.path.join(CSRC, s) for s in SOURCES]
    paths += [h if os.path.isabs(h) else os.path.join(CSRC, h) for h in HEADERS]
    return max(os.path.getmtime(p) for p in paths)


def needs_build() -> bool:
    return not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < _newest_source_mtime()


def _compile_and_link(out_path: str, obj_dir: str, extra_flags, verbose: bool) -> str:
    os.makedirs(obj_dir, exist_ok=True)
    cc = hipcc()
    procs = []
    objs = []
    units = []
    for src in SOURCES:
        if src == "fold_kernels.hip":
            units += [(src, f"fold_kernels_part{n}.o", [f"-DMCCLX_PART={n}"]) for n in range(FOLD_PARTS)]
        else:
            units.append((src, os.path.splitext(src)[0] + ".o", []))
    for src, objname, extra in units:
        obj = os.path.join(obj_dir, objname)
        objs.append(obj)
        cmd = [cc] + HIPCC_FLAGS + list(extra_flags) + extra + (["-x", "hip"] if src.endswith(".cpp") else []) + \
              ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((objname, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out, flush=True)
    tmp = out_path + ".tmp"
    link = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    r = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    os.replace(tmp, out_path)
    return out_path


def build(force: bool = True, verbose: bool = False) -> str:
    """Compile every source and link mccl_amd/libmcclx.so.  Returns its path."""
    if not force and not needs_build():
        return LIB_PATH
    return _compile_and_link(LIB_PATH, OBJ_DIR, [], verbose)


BACKEND_DIR = os.path.join(CSRC, "backend")
BACKEND_SOURCES = ["Progress.cpp", "LocalMesh.cpp", "WorkMCCL.cpp", "HostWire.cpp", "ProcessGroupMCCL.cpp", "bindings.cpp"]


def backend_path() -> str:
    import sysconfig
    return os.path.join(HERE, "_C" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_backend(verbose: bool = False) -> str:
    """Compile the c10d backend (host C++ against the installed torch) into
    mccl_amd/_C*.so, linked against libmcclx.so next to it."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce

    if not os.path.exists(LIB_PATH):
        build(force=True, verbose=verbose)
    os.makedirs(OBJ_DIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = ["-I" + p for p in ce.include_paths()] + ["-I" + sysconfig.get_paths()["include"],
                                                     "-I/opt/rocm/include", "-I" + CSRC,
                                                     "-I" + os.path.join(ROOT, "include")]
    flags = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-parameter",
             "-Wno-sign-compare", "-Wno-unknown-pragmas", "-pthread",
             "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
             "-DTORCH_API_INCLUDE_EXTENSION_H",
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    procs, objs = [], []
    for src in BACKEND_SOURCES:
        obj = os.path.join(OBJ_DIR, "backend_" + os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        cmd = ["g++"] + flags + inc + ["-c", os.path.join(BACKEND_DIR, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f"g++ failed on {src}:\n{out[-6000:]}")
        if verbose and out.strip():
            print(out[-3000:], flush=True)
    out_path = backend_path()
    tmp = out_path + ".tmp"
    # libmcclx last: its HIP runtime dependency (soname libamdhip64.so.N) must be
    # resolved after torch's own copy of that library is loaded, so that the
    # process ends up with ONE runtime (see mccl_amd/_lib.py).
    link = ["g++", "-shared", "-o", tmp] + objs + [
        "-L" + torch_lib, "-ltorch_python", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
        "-L" + HERE, "-lmcclx", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib, "-pthread"]
    r = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    os.replace(tmp, out_path)
    return out_path


BENCH_LIB_PATH = os.path.join(HERE, "libmcclx_bench.so")


def build_bench(verbose: bool = False) -> str:
    """The measurement build (include/mcclx_bench.h), on request only
    (`python -m mccl_amd.build --bench`): the same sources with
    -DMCCLX_TUNE_TIMELINE=1 -- every block of a by-value fold launch can record its
    start, data and end times, and the read-only / write-only probe launch is
    exported.  bench.py takes its one-directional ceilings from it and
    `bench.py --timeline` runs on it; without it those figures are left out.
    Written to mccl_amd/libmcclx_bench.so; the shipped library is not touched."""
    return _compile_and_link(BENCH_LIB_PATH, os.path.join(ROOT, "build", "mcclx_bench"), ["-DMCCLX_TUNE_TIMELINE=1"], verbose)


def ensure_built() -> None:
    """Load what is built; build only if nothing is (used by bench.py and the smoke check)."""
    if not os.path.exists(LIB_PATH):
        build(force=True)


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or needs_build(), verbose=True))
    if "--backend" in sys.argv:
        print(build_backend(verbose=True))
    if "--bench" in sys.argv:
        print(build_bench(verbose=True))
