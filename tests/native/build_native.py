"""Compiles the plain-C clients of the C ABI (cabi_host.c, cabi_gpu.c) with gcc in strict
C99 against include/mcclx.h and links them to the built libmcclx.so."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_build")


def build(name: str, force: bool = False) -> str:
    src = os.path.join(HERE, name + ".c")
    exe = os.path.join(OUT, name)
    lib = os.path.join(ROOT, "mccl_amd", "libmcclx.so")
    hdr = os.path.join(ROOT, "include", "mcclx.h")
    if not os.path.exists(lib):
        raise RuntimeError("libmcclx.so is not built (run __graft_entry__.build())")
    fresh = os.path.exists(exe) and all(os.path.getmtime(exe) >= os.path.getmtime(p) for p in (src, hdr))
    if fresh and not force:
        return exe
    os.makedirs(OUT, exist_ok=True)
    cmd = ["gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-Werror", "-pedantic", "-ffp-contract=off",
           "-I" + os.path.join(ROOT, "include"), src, "-o", exe,
           "-L" + os.path.join(ROOT, "mccl_amd"), "-lmcclx", "-Wl,-rpath,$ORIGIN/../../../mccl_amd"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return exe
