"""CPU-side checks of the C-ABI library: it loads, exports every symbol
include/mcclx.h declares, and its host logic (chunkize, algorithm selection,
workspace sizing, argument checking) matches the oracle.  No compute calls."""
import ctypes as C
import os
import re
import sys

import numpy as np
import pytest

from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    from mccl_amd import _lib
    _lib.lib()
    return _lib


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mcclx.h")).read()
    return sorted(set(re.findall(r"MCCLX_API\s+[\w\s\*]+?\b(mcclx_\w+)\s*\(", text)))


def test_header_symbols_are_all_exported_and_bound(L):
    names = declared_symbols()
    assert len(names) >= 30
    raw = C.CDLL(L.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in mcclx.h but not exported"
        assert n in L.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(L.SIGNATURES) == names
    assert L.lib().mcclx_abi_version() == 4


def test_measurement_aids_are_not_in_the_shipped_library(L):
    """The probe launch, the event timer and the per-block timeline belong to the measurement
    build (include/mcclx_bench.h); libmcclx.so exports nothing that the header does not declare."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", L.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if " T " in line and "mcclx_" in line.split()[-1])
    assert exported == sorted(declared_symbols()), sorted(set(exported) ^ set(declared_symbols()))
    for gone in ("mcclx_probe_stream", "mcclx_timer_begin", "mcclx_timer_end", "mcclx_tune_timeline", "mcclx_bench_probe"):
        assert gone not in exported


def test_struct_layouts_match_header(L):
    assert C.sizeof(L.Seg) == 8 + 8 + 8 * 8 + 8
    assert C.sizeof(L.Plan) == 8 * 4 + 8
    assert C.sizeof(L.Chunk) == 32
    assert C.sizeof(L.Replay) == 8 * 4 + 8 + 8 + 8 + 8


def test_chunkize_matches_oracle_and_reference(L):
    from mccl_amd import harness as H
    rng = np.random.default_rng(0)
    cases = [(w, n) for w in (1, 2, 3, 4, 7, 8, 16, 30) for n in (0, 1, 3, 100, 1024, 1025, 1 << 20, 1234567,
                                                                    6553600, 110000002)]
    cases += [(int(w), int(n)) for w, n in zip(rng.integers(1, 64, 100), rng.integers(0, 1 << 34, 100))]
    for world, numel in cases:
        for es in (2, 4):
            assert H.chunkize(numel, es, world) == orc.chunkize(numel, es, world)
    from mccl_amd import MCCLError
    with pytest.raises(MCCLError):
        H.chunkize(10, 4, 0)


def test_select_algo_matches_oracle(L):
    from mccl_amd import harness as H
    for env in (None, "auto", "ring", "tree", "butterfly", "bogus", ""):
        for below in (None, 0, 1000, 262144, 1 << 30):
            for nbytes, numel in ((4, 1), (8, 2), (999, 499), (1000, 500), (1001, 500), (262144, 65536),
                                  (262145, 65537), (1 << 26, 1 << 24)):
                for world in (1, 2, 3, 8):
                    assert H.select_algo(env, below, nbytes, numel, world) == \
                        orc.select_algo(env, below, nbytes, numel, world), (env, below, nbytes, world)


def test_replay_workspace_sizes(L):
    def need(world, algo, numel, dtype, wire, mode):
        r = L.Replay()
        r.world, r.algo, r.op, r.dtype, r.wire_bf16, r.mode, r.numel = world, algo, 0, dtype, wire, mode, numel
        return L.lib().mcclx_replay_workspace_bytes(C.byref(r))

    up = lambda x: (x + 255) // 256 * 256
    per = lambda n, w: (n + w - 1) // w
    n = 1000003
    # STEPWISE: recv scratch per rank as ProcessGroupMCCL.cpp:152-162 (+ one bf16 copy per rank with the wire codec)
    assert need(4, L.ALGO_RING, n, L.F32, 0, 0) == 4 * up(per(n, 4) * 4)
    assert need(4, L.ALGO_BUTTERFLY, n, L.F32, 0, 0) == 4 * up(3 * per(n, 4) * 4)
    assert need(4, L.ALGO_TREE, n, L.BF16, 0, 0) == 4 * up(n * 2)
    assert need(3, L.ALGO_BUTTERFLY, n, L.F32, 1, 0) == 3 * up(n * 2) + 3 * up(2 * per(n, 3) * 2)
    # FUSED: peers are read in place; only the wire copies remain
    assert need(4, L.ALGO_RING, n, L.F32, 0, 1) == 0
    assert need(3, L.ALGO_BUTTERFLY, n, L.F32, 1, 1) == 3 * up(n * 2)
    assert need(3, L.ALGO_BUTTERFLY, n, L.BF16, 1, 1) == 0     # the codec only acts on fp32 tensors


def test_calls_fail_cleanly_without_a_context(L):
    lib = L.lib()
    assert lib.mcclx_queue_drain(None) == L.ERR_STATE
    assert "mcclx_init not called" in L.last_error()
    assert lib.mcclx_reduce(None, None, None, 0, 0, 0) == L.ERR_STATE
    assert lib.mcclx_batch_begin(None, b"x") == L.ERR_STATE
    assert lib.mcclx_destroy(None) == L.OK
    with pytest.raises(L.MCCLError, match=r"^\[MCCL\] "):
        L.check(lib.mcclx_queue_drain(None))


def test_init_without_gpu_reports_an_error(L):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    rc = L.lib().mcclx_init(0, C.byref(h))
    assert rc in (L.ERR_HIP, L.ERR_INVALID) and not h.value
    assert L.last_error().startswith("[MCCL] ")
    from mccl_amd import kernels
    with pytest.raises(L.MCCLError):
        kernels.ReduceQueue(0)                     # no silent fallback: the product path needs the GPU
    with pytest.raises(L.MCCLError, match="not called"):
        kernels.hip_reduce_op(torch.ones(2), torch.ones(2), 0)


def test_missing_library_is_loud(L, monkeypatch, tmp_path):
    from mccl_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmcclx.so"))
    with pytest.raises(_lib.MCCLError, match="is missing"):
        _lib.lib()


def test_only_one_hip_runtime_is_loaded_whatever_the_import_order():
    """PyTorch-ROCm wheels bundle a libamdhip64 next to the system's; loading
    libmcclx before torch used to pull in both (heap corruption at exit)."""
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r)\n"
            "import mccl_amd\n"
            "from mccl_amd import _lib; _lib.lib()\n"
            "import torch\n"
            "libs = sorted(set(l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l))\n"
            "print('\\n'.join(libs))\n") % ROOT
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    libs = [l for l in out.stdout.strip().splitlines() if l]
    assert len(libs) == 1, libs


def test_header_is_strict_c99_and_a_plain_c_client_links_and_runs():
    """include/mcclx.h compiles as C99 with -pedantic -Werror; a C program linked against
    libmcclx.so uses the host-only entry points (tests/native/cabi_host.c).  The GPU client
    is compiled here too, so that it travels with the tree."""
    import subprocess
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "native"))
    import build_native
    try:
        exe = build_native.build("cabi_host", force=True)
        build_native.build("cabi_gpu", force=True)
    except subprocess.CalledProcessError as e:
        raise AssertionError(e.stderr)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr
