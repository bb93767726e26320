"""ctypes front end of the CPU oracle (oracle/mccl_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py.  The shipped package never imports this module.

Buffers are numpy arrays: float32 for fp32, uint16 bit patterns for bf16/f16.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmccl_oracle.so")
REF_LIB_PATH = os.path.join(HERE, "_ref", "libmccl_ref.so")

F32, F16, BF16 = 0, 1, 2
SUM, AVG, PRODUCT, MIN, MAX = 0, 1, 2, 3, 4
RING, TREE, BUTTERFLY = 0, 1, 2
SCALE_VIEW, SCALE_TENSOR = 0, 1

NP_DTYPE = {F32: np.float32, F16: np.uint16, BF16: np.uint16}


class Chunk(C.Structure):
    _fields_ = [("elem_start", C.c_int64), ("elem_count", C.c_int64),
                ("byte_off", C.c_uint64), ("byte_len", C.c_uint64)]


def build() -> None:
    """Compile the oracle (and oracle/_ref when the reference checkout exists)."""
    subprocess.run(["make", "-C", HERE, "all"], check=True, capture_output=True)


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, i32, i64, u64, sz, dbl = C.c_void_p, C.c_int, C.c_int64, C.c_uint64, C.c_size_t, C.c_double
        L.orc_chunkize.argtypes = [i64, sz, i32, C.POINTER(Chunk)]
        L.orc_chunkize.restype = None
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_f64_to_f16.argtypes = [dbl]
        L.orc_f64_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_encode_bf16.argtypes = [vp, vp, sz, i32]
        L.orc_encode_bf16.restype = None
        L.orc_decode_bf16.argtypes = [vp, vp, sz, i32]
        L.orc_decode_bf16.restype = None
        L.orc_reduce.argtypes = [vp, vp, i32, sz, i32, i32]
        L.orc_reduce.restype = i32
        L.orc_scale.argtypes = [vp, i32, sz, dbl, i32, i32]
        L.orc_scale.restype = i32
        L.orc_accumulate_scale.argtypes = [vp, vp, i32, sz, dbl, i32]
        L.orc_accumulate_scale.restype = i32
        L.orc_scale_constant_bits.argtypes = [i32, dbl, i32]
        L.orc_scale_constant_bits.restype = C.c_uint32
        L.orc_select_algo.argtypes = [C.c_char_p, i64, u64, i64, i32]
        L.orc_select_algo.restype = i32
        L.orc_allreduce.argtypes = [i32, i32, C.POINTER(vp), i32, i64, i32, i32]
        L.orc_allreduce.restype = i32
        L.orc_pg_allreduce.argtypes = [i32, C.POINTER(vp), i32, i64, i32, i32, C.c_char_p, i64,
                                       C.POINTER(i32), i32]
        L.orc_pg_allreduce.restype = i32
        L.orc_reduce_scatter.argtypes = [i32, C.POINTER(vp), C.POINTER(vp), i32, i64, i32, i32]
        L.orc_reduce_scatter.restype = i32
        L.orc_reduce_scatter_f32acc.argtypes = [i32, C.POINTER(vp), C.POINTER(vp), i64, i32, i32]
        L.orc_reduce_scatter_f32acc.restype = i32
        L.orc_allgather.argtypes = [i32, C.POINTER(vp), C.POINTER(vp), sz]
        L.orc_allgather.restype = None
        L.orc_wire_fold_chunk.argtypes = [vp, vp, C.POINTER(vp), i32, sz, i32, i32, dbl, vp, vp, i32]
        L.orc_wire_fold_chunk.restype = None
        L.orc_max_threads.argtypes = []
        L.orc_max_threads.restype = i32
        _lib = L
    return _lib


_ref = None


def ref_lib():
    """The reference's own torch-free sources (oracle/_ref), or None if absent."""
    global _ref
    if _ref is None and os.path.exists(REF_LIB_PATH):
        R = C.CDLL(REF_LIB_PATH)
        R.ref_chunkize.argtypes = [C.c_int64, C.c_int, C.c_uint64, C.POINTER(C.c_int64)]
        R.ref_chunkize.restype = None
        R.ref_ring_chunks_selftest.restype = C.c_int
        R.ref_progress_order.argtypes = [C.c_int, C.c_uint64, C.POINTER(C.c_int)]
        R.ref_progress_order.restype = C.c_int
        _ref = R
    return _ref


def _p(a: np.ndarray) -> C.c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return C.c_void_p(a.ctypes.data)


def _pa(arrs):
    return (C.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])


def elem_size(dtype: int) -> int:
    return 4 if dtype == F32 else 2


def chunkize(numel: int, esize: int, world: int):
    out = (Chunk * world)()
    lib().orc_chunkize(numel, esize, world, out)
    return [(c.elem_start, c.elem_count, c.byte_off, c.byte_len) for c in out]


def encode_bf16(src: np.ndarray, threads: int = 1) -> np.ndarray:
    src = np.ascontiguousarray(src, dtype=np.float32)
    dst = np.empty(src.shape, dtype=np.uint16)
    lib().orc_encode_bf16(_p(dst), _p(src), src.size, threads)
    return dst


def decode_bf16(src: np.ndarray, threads: int = 1) -> np.ndarray:
    src = np.ascontiguousarray(src, dtype=np.uint16)
    dst = np.empty(src.shape, dtype=np.float32)
    lib().orc_decode_bf16(_p(dst), _p(src), src.size, threads)
    return dst


def reduce(dst: np.ndarray, src: np.ndarray, dtype: int, op: int, threads: int = 1) -> int:
    """In place: dst = dst (op) src."""
    assert dst.dtype == NP_DTYPE[dtype] and src.dtype == NP_DTYPE[dtype] and dst.size == src.size
    return lib().orc_reduce(_p(dst), _p(src), dtype, dst.size, op, threads)


def scale(buf: np.ndarray, dtype: int, s: float, mode: int = SCALE_VIEW, threads: int = 1) -> int:
    assert buf.dtype == NP_DTYPE[dtype]
    return lib().orc_scale(_p(buf), dtype, buf.size, s, mode, threads)


def accumulate_scale(dst, src, dtype: int, s: float, threads: int = 1) -> int:
    assert dst.dtype == NP_DTYPE[dtype] and src.dtype == NP_DTYPE[dtype]
    return lib().orc_accumulate_scale(_p(dst), _p(src), dtype, dst.size, s, threads)


def scale_constant_bits(dtype: int, s: float, mode: int) -> int:
    return lib().orc_scale_constant_bits(dtype, s, mode)


def select_algo(env_algo, tree_below, wire_nbytes, numel, world) -> int:
    e = env_algo.encode() if env_algo is not None else None
    return lib().orc_select_algo(e, -1 if tree_below is None else tree_below, wire_nbytes, numel,
                                 world)


def allreduce(algo: int, bufs, dtype: int, op: int, threads: int = 1) -> int:
    """In place on the list of per-rank arrays."""
    n = bufs[0].size
    assert all(b.size == n and b.dtype == NP_DTYPE[dtype] for b in bufs)
    return lib().orc_allreduce(algo, len(bufs), _pa(bufs), dtype, n, op, threads)


def pg_allreduce(bufs, dtype: int, op: int, wire_bf16: bool = False, env_algo=None,
                 tree_below=None, threads: int = 1):
    """Returns (rc, algo_used); results are written in place."""
    n = bufs[0].size
    algo = C.c_int(-1)
    e = env_algo.encode() if env_algo is not None else None
    rc = lib().orc_pg_allreduce(len(bufs), _pa(bufs), dtype, n, op, int(wire_bf16), e,
                                -1 if tree_below is None else tree_below, C.byref(algo), threads)
    return rc, algo.value


def reduce_scatter(outs, ins, dtype: int, op: int, threads: int = 1) -> int:
    return lib().orc_reduce_scatter(len(ins), _pa(outs), _pa(ins), dtype, outs[0].size, op, threads)


def reduce_scatter_f32acc(outs, ins, op: int, threads: int = 1) -> int:
    return lib().orc_reduce_scatter_f32acc(len(ins), _pa(outs), _pa(ins), outs[0].size, op, threads)


def allgather(outs, ins) -> None:
    lib().orc_allgather(len(ins), _pa(outs), _pa(ins), ins[0].nbytes)


def wire_fold_chunk(own: np.ndarray, peers, own_last: bool = False, scale_by=None,
                    want_wire: bool = False, threads: int = 1):
    """Reference-shaped passes for one owner's chunk; returns fp32 (and bf16 bits)."""
    n = own.size
    out = np.empty(n, dtype=np.float32)
    tmp = np.empty(n + 1, dtype=np.uint16)
    wire = np.empty(n, dtype=np.uint16) if want_wire else None
    lib().orc_wire_fold_chunk(_p(out), _p(own), _pa(peers), len(peers), n, int(own_last),
                              int(scale_by is not None), float(scale_by or 0.0), _p(tmp),
                              _p(wire) if want_wire else None, threads)
    return (out, wire) if want_wire else out


def max_threads() -> int:
    return lib().orc_max_threads()
