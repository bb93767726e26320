"""ctypes binding of libmcclx.so -- the C ABI declared in include/mcclx.h.

The library is loaded from this directory.  There is no fallback: if it is
missing the import of any compute entry point raises, so a GPU run can never
silently use something else.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# The in-tree library.  MCCLX_LIBRARY, read when the library is first loaded, names a
# differently built libmcclx.so (tuning builds).
LIB_PATH = os.path.join(HERE, "libmcclx.so")

MAX_INPUTS = 8
NOALLOC_MAX_SEGS = 1024

OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP, ERR_STATE, ERR_NOMEM = 0, -1, -2, -3, -4, -5
F32, F16, BF16 = 0, 1, 2
SUM, AVG, PRODUCT, MIN, MAX = 0, 1, 2, 3, 4
SCALE_NONE, SCALE_VIEW, SCALE_TENSOR = 0, 1, 2
IO_PURE, IO_OUT_F32, IO_OWN_FIRST_F32, IO_OWN_LAST_F32, IO_ALL_F32 = 0, 1, 2, 3, 4
TOPO_FOLD, TOPO_BINOMIAL = 0, 1
ACC_STEP, ACC_F32 = 0, 1
ALGO_RING, ALGO_TREE, ALGO_BUTTERFLY = 0, 1, 2
REPLAY_STEPWISE, REPLAY_FUSED, REPLAY_DIRECT = 0, 1, 2
PLAN_ACC_IS_SRC = 1


def PLAN_FANOUT(n: int) -> int:
    """plan.flags bits: the result also goes to n further destinations, in[k .. k+n-1]."""
    return n << 8



class Seg(C.Structure):
    _fields_ = [("out", C.c_void_p), ("wire_out", C.c_void_p),
                ("inp", C.c_void_p * MAX_INPUTS), ("count", C.c_uint64)]


class CopyDesc(C.Structure):
    _fields_ = [("dst", C.c_void_p), ("src", C.c_void_p), ("nbytes", C.c_uint64)]


class Plan(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("io", C.c_int32), ("k", C.c_int32), ("topo", C.c_int32),
                ("op", C.c_int32), ("acc", C.c_int32), ("scale_mode", C.c_int32),
                ("flags", C.c_int32), ("scale", C.c_double)]


class Chunk(C.Structure):
    _fields_ = [("elem_start", C.c_int64), ("elem_count", C.c_int64),
                ("byte_off", C.c_uint64), ("byte_len", C.c_uint64)]


class Replay(C.Structure):
    _fields_ = [("world", C.c_int32), ("algo", C.c_int32), ("op", C.c_int32), ("dtype", C.c_int32),
                ("wire_bf16", C.c_int32), ("mode", C.c_int32), ("acc", C.c_int32),
                ("reserved", C.c_int32), ("numel", C.c_uint64), ("tensors", C.POINTER(C.c_void_p)),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64)]


# name -> (restype, argtypes); every symbol include/mcclx.h declares
_vp, _i, _u64, _i64, _d = C.c_void_p, C.c_int, C.c_uint64, C.c_int64, C.c_double
_pp = C.POINTER(C.c_void_p)
SIGNATURES = {
    "mcclx_last_error": (C.c_char_p, []),
    "mcclx_abi_version": (_i, []),
    "mcclx_init": (_i, [_i, _pp]),
    "mcclx_init_on_stream": (_i, [_i, _vp, _pp]),
    "mcclx_destroy": (_i, [_vp]),
    "mcclx_queue_stream": (_vp, [_vp]),
    "mcclx_device_cus": (_i, [_vp]),
    "mcclx_launch_count": (_u64, [_vp]),
    "mcclx_hold_launch_count": (_u64, [_vp]),
    "mcclx_set_hold": (_i, [_vp, _i]),
    "mcclx_hold_model": (_i, [_vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "mcclx_reduce": (_i, [_vp, _vp, _vp, _i, _u64, _i]),
    "mcclx_scale": (_i, [_vp, _vp, _i, _u64, _d, _i]),
    "mcclx_accumulate_scale": (_i, [_vp, _vp, _vp, _i, _u64, _d]),
    "mcclx_batch_begin": (_i, [_vp, C.c_char_p]),
    "mcclx_batch_end": (_i, [_vp]),
    "mcclx_encode_bf16": (_i, [_vp, _vp, _vp, _u64]),
    "mcclx_decode_bf16": (_i, [_vp, _vp, _vp, _u64]),
    "mcclx_fold": (_i, [_vp, C.POINTER(Plan), C.POINTER(Seg)]),
    "mcclx_fold_batched": (_i, [_vp, C.POINTER(Plan), C.POINTER(Seg), C.c_uint32]),
    "mcclx_fold_batched_noalloc": (_i, [_vp, C.POINTER(Plan), C.POINTER(Seg), C.c_uint32]),
    "mcclx_copy": (_i, [_vp, _vp, _vp, _u64]),
    "mcclx_copy_batched": (_i, [_vp, C.POINTER(CopyDesc), C.c_uint32]),
    "mcclx_queue_drain": (_i, [_vp]),
    "mcclx_queue_wait_stream": (_i, [_vp, _vp]),
    "mcclx_stream_wait_queue": (_i, [_vp, _vp]),
    "mcclx_event_record": (_i, [_vp, C.POINTER(C.c_uint64)]),
    "mcclx_event_query": (_i, [_vp, _u64, C.POINTER(C.c_int)]),
    "mcclx_event_wait": (_i, [_vp, _u64]),
    "mcclx_graph_begin": (_i, [_vp]),
    "mcclx_graph_end": (_i, [_vp, _pp]),
    "mcclx_graph_launch": (_i, [_vp, _vp]),
    "mcclx_graph_destroy": (_i, [_vp, _vp]),
    "mcclx_host_alloc": (_i, [_vp, _u64, _pp, _pp]),
    "mcclx_host_free": (_i, [_vp, _vp]),
    "mcclx_stage_for_send": (_i, [_vp, _vp, _u64, _pp]),
    "mcclx_unstage_from_recv": (_i, [_vp, _vp, _vp, _u64]),
    "mcclx_chunkize": (_i, [_i64, _u64, _i, C.POINTER(Chunk)]),
    "mcclx_select_algo": (_i, [C.c_char_p, _i64, _u64, _i64, _i]),
    "mcclx_replay_workspace_bytes": (_u64, [C.POINTER(Replay)]),
    "mcclx_allreduce_replay": (_i, [_vp, C.POINTER(Replay)]),
    "mcclx_allreduce_replay_many": (_i, [_vp, C.POINTER(Replay), C.c_uint32]),
    "mcclx_reduce_scatter_replay": (_i, [_vp, _i, _pp, _pp, _i, _u64, _i, _i, _i]),
    "mcclx_reduce_scatter_shares": (_i, [_vp, _i, _pp, _pp, _i, _u64, _i, _i, _i]),
    "mcclx_allgather_replay": (_i, [_vp, _i, _pp, _pp, _u64]),
}


class MCCLError(RuntimeError):
    """Mirrors mccl::MCCLError (csrc/common/Errors.hpp:9-13): message starts with "[MCCL] "."""

    def __init__(self, msg: str, code: int = ERR_INVALID):
        super().__init__(msg)
        self.code = code


_lib = None


def lib() -> C.CDLL:
    """Load libmcclx.so (once) and type every entry point.  Raises if absent."""
    global _lib
    if _lib is None:
        # One HIP runtime per process.  PyTorch-ROCm wheels bundle their own
        # libamdhip64 (file "libamdhip64.so", soname "libamdhip64.so.N") next to the
        # system's /opt/rocm copy of the same soname.  The dynamic loader reuses an
        # already loaded library with a matching soname, so torch must be loaded
        # first: then libmcclx binds to the runtime that owns torch's tensors.  The
        # other order loads both runtimes and corrupts the heap at exit.
        import torch  # noqa: F401
        path = os.environ.get("MCCLX_LIBRARY") or LIB_PATH
        if not os.path.exists(path):
            raise MCCLError(
                f"[MCCL] native library {path} is missing: build it with "
                "`python -m mccl_amd.build` (there is no fallback path)")
        L = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


BENCH_LIB_PATH = os.path.join(HERE, "libmcclx_bench.so")
_bench = None


def bench_lib():
    """The measurement build (include/mcclx_bench.h), or None when it has not been built
    (`python -m mccl_amd.build --bench`).  Loaded next to the shipped library; only its
    probe launch, which takes a raw stream, is used from here."""
    global _bench
    if _bench is None:
        import torch  # noqa: F401  (one HIP runtime per process, see lib())
        if not os.path.exists(BENCH_LIB_PATH):
            return None
        B = C.CDLL(BENCH_LIB_PATH)
        B.mcclx_bench_probe.restype = _i
        B.mcclx_bench_probe.argtypes = [_vp, _vp, _u64, _i]
        B.mcclx_last_error.restype = C.c_char_p
        _bench = B
    return _bench


def last_error() -> str:
    return lib().mcclx_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Turn a C-ABI return code back into the exception the reference throws."""
    if rc != OK:
        raise MCCLError(last_error() or f"[MCCL] error code {rc}", rc)
