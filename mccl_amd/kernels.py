"""Host launch API over torch tensors -- the counterpart of the reference's
csrc/metal/MetalKernels.hpp, calling libmcclx.so through its C ABI.

Function names, argument meaning and error behaviour follow the reference
(`metal_*` became `hip_*`): SUM and AVG both accumulate, unsupported ops raise
MCCLError("... Unsupported ReduceOp: n"), shape/dtype mismatches raise, a
second begin_batch raises "batch already active".

torch is used for device memory and streams only; every arithmetic launch is a
hand-written HIP kernel inside libmcclx.so.
"""
from __future__ import annotations

import ctypes as C
import sys as _sys
from typing import Optional, Sequence

import torch

from . import _lib as L
from ._lib import MCCLError

_DTYPE = {torch.float32: L.F32, torch.float16: L.F16, torch.bfloat16: L.BF16}

# torch.distributed.ReduceOp values, without importing torch.distributed here
REDUCE_OPS = {"sum": L.SUM, "avg": L.AVG, "product": L.PRODUCT, "min": L.MIN, "max": L.MAX}


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        # select_op_pipeline returns nil -> "No Metal pipeline for dtype" (MetalKernels.mm:634-635)
        raise MCCLError(f"[MCCL] No HIP kernel for dtype {t.dtype}", L.ERR_UNSUPPORTED)


def op_code(op) -> int:
    if isinstance(op, str):
        return REDUCE_OPS[op.lower()]
    return int(op)


def _check_tensor(t: torch.Tensor, what: str) -> None:
    # check_mps_ (ProcessGroupMCCL.cpp:72-79) + check_single_tensor (TensorChecks.hpp:10-35)
    if not t.is_cuda:
        raise MCCLError(f"[MCCL] {what}: tensor must live on the GPU; got {t.device.type} tensor")
    if not t.is_contiguous():
        raise MCCLError(f"[MCCL] {what}: tensor must be contiguous")


def _check_same(a: torch.Tensor, b: torch.Tensor) -> None:
    # check_same_shape_dtype, TensorChecks.hpp:45-54
    if a.shape != b.shape:
        raise MCCLError("[MCCL] Tensor: Tensor check failed: Shape mismatch in collective")
    if a.dtype != b.dtype:
        raise MCCLError("[MCCL] Tensor: Tensor check failed: Dtype mismatch in collective")


class ReduceQueue:
    """One context of libmcclx: kernel dispatch + a HIP stream with event
    completion (the reference's KernelCache + dedicated MTLCommandQueue,
    MetalKernels.mm:29-52, MPSInterop.mm:32-36)."""

    def __init__(self, device: int = 0, on_torch_stream: bool = False):
        self._h = C.c_void_p()
        self.device = device
        if on_torch_stream:
            s = torch.cuda.current_stream(device).cuda_stream
            L.check(L.lib().mcclx_init_on_stream(device, C.c_void_p(s), C.byref(self._h)))
        else:
            L.check(L.lib().mcclx_init(device, C.byref(self._h)))
        self._host = {}

    # -- lifetime --------------------------------------------------------
    def close(self) -> None:
        if self._h:
            L.lib().mcclx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        # At interpreter shutdown the HIP runtime and torch may already be tearing
        # down; the process is about to release everything anyway.
        if _sys is None or _sys.is_finalizing():
            return
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self) -> C.c_void_p:
        if not self._h:
            raise MCCLError("[MCCL] hip_kernels_init() not called", L.ERR_STATE)
        return self._h

    @property
    def stream(self) -> int:
        return L.lib().mcclx_queue_stream(self.handle) or 0

    @property
    def compute_units(self) -> int:
        return L.lib().mcclx_device_cus(self.handle)

    # -- ordering ----------------------------------------------------------
    def drain(self) -> None:
        """mccl_queue_drain (MPSInterop.mm:312-318)."""
        L.check(L.lib().mcclx_queue_drain(self.handle))

    def wait_torch_stream(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        """Device-side replacement of mps_stream_sync (MPSInterop.mm:308-310)."""
        s = stream or torch.cuda.current_stream(self.device)
        L.check(L.lib().mcclx_queue_wait_stream(self.handle, C.c_void_p(s.cuda_stream)))

    def torch_stream_wait(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        s = stream or torch.cuda.current_stream(self.device)
        L.check(L.lib().mcclx_stream_wait_queue(self.handle, C.c_void_p(s.cuda_stream)))

    def record(self) -> int:
        t = C.c_uint64()
        L.check(L.lib().mcclx_event_record(self.handle, C.byref(t)))
        return t.value

    def query(self, ticket: int) -> bool:
        d = C.c_int()
        L.check(L.lib().mcclx_event_query(self.handle, ticket, C.byref(d)))
        return bool(d.value)

    def wait(self, ticket: int) -> None:
        L.check(L.lib().mcclx_event_wait(self.handle, ticket))

    # Device time on the queue, for measurement: torch events recorded on the queue's own
    # stream (torch.cuda.Event sees the stream it is recorded on, not the current one).
    def _torch_stream(self) -> "torch.cuda.Stream":
        if getattr(self, "_ext_stream", None) is None:
            self._ext_stream = torch.cuda.ExternalStream(self.stream, device=self.device)
        return self._ext_stream

    def timer_begin(self) -> None:
        self._t0 = torch.cuda.Event(enable_timing=True)
        self._t1 = torch.cuda.Event(enable_timing=True)
        self._t0.record(self._torch_stream())

    def timer_end(self) -> float:
        """Milliseconds between timer_begin and now, both on the queue; waits for the queue."""
        self._t1.record(self._torch_stream())
        self._t1.synchronize()
        return self._t0.elapsed_time(self._t1)

    # -- launch graphs --------------------------------------------------------
    def graph_begin(self) -> None:
        L.check(L.lib().mcclx_graph_begin(self.handle))

    def graph_end(self) -> int:
        g = C.c_void_p()
        L.check(L.lib().mcclx_graph_end(self.handle, C.byref(g)))
        return g.value

    def graph_launch(self, graph: int) -> None:
        L.check(L.lib().mcclx_graph_launch(self.handle, C.c_void_p(graph)))

    def graph_destroy(self, graph: int) -> None:
        L.check(L.lib().mcclx_graph_destroy(self.handle, C.c_void_p(graph)))

    # -- pinned, device-mapped host memory ----------------------------------
    def host_alloc(self, nbytes: int):
        """Returns (host_address, device_address)."""
        h, d = C.c_void_p(), C.c_void_p()
        L.check(L.lib().mcclx_host_alloc(self.handle, nbytes, C.byref(h), C.byref(d)))
        return h.value, d.value

    def host_free(self, host_address: int) -> None:
        L.check(L.lib().mcclx_host_free(self.handle, C.c_void_p(host_address)))

    # -- staging for memory the host cannot address -----------------------------
    def stage_for_send(self, device_ptr: int, nbytes: int) -> int:
        """Device bytes -> pinned staging; returns the host address (valid until the
        next call).  stage_for_send, MPSInterop.mm:365-406."""
        h = C.c_void_p()
        L.check(L.lib().mcclx_stage_for_send(self.handle, C.c_void_p(device_ptr), nbytes, C.byref(h)))
        return h.value

    def unstage_from_recv(self, device_ptr: int, host_ptr: int, nbytes: int) -> None:
        """Host bytes -> device, asynchronously on the queue.  unstage_from_recv, MPSInterop.mm:408-435."""
        L.check(L.lib().mcclx_unstage_from_recv(self.handle, C.c_void_p(device_ptr), C.c_void_p(host_ptr), nbytes))

    # -- raw launches ----------------------------------------------------
    def fold(self, plan: L.Plan, segs: Sequence[L.Seg]) -> None:
        arr = (L.Seg * len(segs))(*segs)
        L.check(L.lib().mcclx_fold_batched(self.handle, C.byref(plan), arr, len(segs)))

    def launch_count(self) -> int:
        """Kernel launches issued on this queue so far (diagnostic)."""
        return int(L.lib().mcclx_launch_count(self.handle))

    def hold_launch_count(self) -> int:
        """Launches of this queue that took the hold form: reads first, results kept in registers,
        writes once the reads are through (diagnostic)."""
        return int(L.lib().mcclx_hold_launch_count(self.handle))

    def set_hold(self, enabled: bool) -> None:
        """Switch the hold form of fold launches off (a queue whose launches overlap with other
        work on the GPU) or on again."""
        L.check(L.lib().mcclx_set_hold(self.handle, int(enabled)))

    def copy(self, dst_ptr: int, src_ptr: int, nbytes: int) -> None:
        L.check(L.lib().mcclx_copy(self.handle, C.c_void_p(dst_ptr), C.c_void_p(src_ptr), nbytes))

    def hold_model(self):
        """(latency_ticks, bytes_per_tick, measured): the gate of the hold form on this device."""
        lat, bpt = C.c_uint32(), C.c_uint32()
        measured = L.lib().mcclx_hold_model(self.handle, C.byref(lat), C.byref(bpt))
        return lat.value, bpt.value, bool(measured)

    def probe_stream(self, ptr: int, nbytes: int, write: bool) -> None:
        """One read-only or write-only pass over a buffer on this queue: a launch of the
        measurement build (python -m mccl_amd.build --bench), which must be there."""
        B = L.bench_lib()
        if B is None:
            raise MCCLError("[MCCL] the measurement build is missing: python -m mccl_amd.build --bench", L.ERR_STATE)
        rc = B.mcclx_bench_probe(C.c_void_p(self.stream), C.c_void_p(ptr), nbytes, int(write))
        if rc != L.OK:
            raise MCCLError(B.mcclx_last_error().decode("utf-8", "replace"), rc)

    def copy_batched(self, triples) -> None:
        """Many (dst, src, nbytes) copies in one launch (a few large ones go out one by one)."""
        arr = (L.CopyDesc * len(triples))(*[L.CopyDesc(d, s, n) for d, s, n in triples])
        L.check(L.lib().mcclx_copy_batched(self.handle, arr, len(triples)))


_default: Optional[ReduceQueue] = None
_batch_depth_owner = None


def hip_kernels_init(device: int = 0) -> ReduceQueue:
    """metal_kernels_init (MetalKernels.mm:189): idempotent, process-wide."""
    global _default
    if _default is None:
        _default = ReduceQueue(device)
    return _default


def _q(queue: Optional[ReduceQueue]) -> ReduceQueue:
    if queue is not None:
        return queue
    if _default is None:
        raise MCCLError("[MCCL] Check failed: c.initialized — hip_kernels_init() not called", L.ERR_STATE)
    return _default


def make_seg(out=0, wire_out=0, inputs=(), count=0) -> L.Seg:
    s = L.Seg()
    s.out = out or None
    s.wire_out = wire_out or None
    for i, p in enumerate(inputs):
        s.inp[i] = p
    s.count = count
    return s


def make_plan(dtype, k, io=L.IO_PURE, topo=L.TOPO_FOLD, op=L.SUM, acc=L.ACC_STEP,
              scale_mode=L.SCALE_NONE, scale=0.0, flags=0, fanout=0) -> L.Plan:
    """`fanout` = n: the result is also stored to n further destinations, which the segment
    names in inputs[k .. k+n-1]."""
    return L.Plan(dtype, io, k, topo, op, acc, scale_mode, flags | L.PLAN_FANOUT(fanout), scale)


# ---- tensor variants (MetalKernels.hpp:14-43) ------------------------------
#
# Tensors are produced and consumed on torch's current stream, the kernels run
# on the reduce queue: each tensor variant makes the queue wait for torch's
# stream before the launch and torch's stream wait for the queue after it
# (two device-side event waits, the host is never blocked).  The reference
# reaches the same ordering with a blocking mps_stream_sync() before and
# mccl_queue_drain() after (ProcessGroupMCCL.cpp:172,178).  The *_view variants
# take raw addresses and leave the ordering to the caller, as the reference's do.

class _ordered:
    def __init__(self, q: "ReduceQueue"):
        self.q = q

    def __enter__(self):
        self.q.wait_torch_stream()
        return self.q

    def __exit__(self, *exc):
        self.q.torch_stream_wait()
        return False


def hip_reduce_op(dst: torch.Tensor, src: torch.Tensor, op, queue=None) -> torch.Tensor:
    """dst (op)= src.  metal_reduce_op, MetalKernels.mm:530-550."""
    q = _q(queue)
    _check_tensor(dst, "reduce_op")
    _check_tensor(src, "reduce_op")
    _check_same(dst, src)
    code = dtype_code(dst)
    with _ordered(q):
        L.check(L.lib().mcclx_reduce(q.handle, dst.data_ptr(), src.data_ptr(), code, dst.numel(),
                                     op_code(op)))
    return dst


def hip_accumulate_chunk(dst, src, queue=None):
    return hip_reduce_op(dst, src, L.SUM, queue)


def hip_elementwise_min(dst, src, queue=None):
    return hip_reduce_op(dst, src, L.MIN, queue)


def hip_elementwise_max(dst, src, queue=None):
    return hip_reduce_op(dst, src, L.MAX, queue)


def hip_elementwise_product(dst, src, queue=None):
    return hip_reduce_op(dst, src, L.PRODUCT, queue)


def hip_scale_inplace(buf: torch.Tensor, scale: float, queue=None) -> torch.Tensor:
    """buf *= scale, tensor-variant constant.  metal_scale_inplace, MetalKernels.mm:365-405."""
    q = _q(queue)
    _check_tensor(buf, "scale_inplace")
    code = dtype_code(buf)
    with _ordered(q):
        L.check(L.lib().mcclx_scale(q.handle, buf.data_ptr(), code, buf.numel(), float(scale),
                                    L.SCALE_TENSOR))
    return buf


def hip_accumulate_and_scale(dst, src, scale: float, queue=None) -> torch.Tensor:
    """dst = (dst + src) * scale.  metal_accumulate_and_scale, MetalKernels.mm:408-458."""
    q = _q(queue)
    _check_tensor(dst, "accumulate_and_scale")
    _check_tensor(src, "accumulate_and_scale")
    _check_same(dst, src)
    code = dtype_code(dst)
    with _ordered(q):
        L.check(L.lib().mcclx_accumulate_scale(q.handle, dst.data_ptr(), src.data_ptr(), code,
                                               dst.numel(), float(scale)))
    return dst


# ---- view variants (MetalKernels.hpp:45-54): raw address + count, then drain --

def hip_reduce_op_view(dst_ptr: int, src_ptr: int, dtype: int, count: int, op, queue=None,
                       drain: bool = True) -> None:
    """metal_reduce_op_view, MetalKernels.mm:628-640 (launch, then block)."""
    q = _q(queue)
    L.check(L.lib().mcclx_reduce(q.handle, C.c_void_p(dst_ptr), C.c_void_p(src_ptr), dtype, count,
                                 op_code(op)))
    if drain:
        q.drain()


def hip_scale_inplace_view(ptr: int, dtype: int, count: int, scale: float, queue=None,
                           drain: bool = True) -> None:
    """metal_scale_inplace_view, MetalKernels.mm:642-674 (truncated bf16 constant)."""
    q = _q(queue)
    L.check(L.lib().mcclx_scale(q.handle, C.c_void_p(ptr), dtype, count, float(scale), L.SCALE_VIEW))
    if drain:
        q.drain()


def hip_begin_batch(label: str = "mccl_batch", queue=None) -> None:
    L.check(L.lib().mcclx_batch_begin(_q(queue).handle, label.encode()))


def hip_end_batch(queue=None) -> None:
    L.check(L.lib().mcclx_batch_end(_q(queue).handle))


def hip_sync(queue=None) -> None:
    """metal_sync, MetalKernels.mm:552-557: end an open batch, then drain."""
    q = _q(queue)
    L.check(L.lib().mcclx_batch_end(q.handle))
    torch.cuda.current_stream(q.device).synchronize()
    q.drain()


# ---- wire codec -----------------------------------------------------------------

def encode_bf16(src: torch.Tensor, out: Optional[torch.Tensor] = None, queue=None) -> torch.Tensor:
    """fp32 -> bf16, round to nearest even, NaN -> 0x7FC0 (ProcessGroupMCCL.cpp:131-132)."""
    q = _q(queue)
    _check_tensor(src, "encode_bf16")
    if src.dtype != torch.float32:
        raise MCCLError("[MCCL] encode_bf16 expects a float32 tensor")
    if out is None:
        out = torch.empty(src.shape, dtype=torch.bfloat16, device=src.device)
    with _ordered(q):
        L.check(L.lib().mcclx_encode_bf16(q.handle, out.data_ptr(), src.data_ptr(), src.numel()))
    return out


def decode_bf16(src: torch.Tensor, out: Optional[torch.Tensor] = None, queue=None) -> torch.Tensor:
    """bf16 -> fp32, exact (ProcessGroupMCCL.cpp:179-183)."""
    q = _q(queue)
    _check_tensor(src, "decode_bf16")
    if src.dtype != torch.bfloat16:
        raise MCCLError("[MCCL] decode_bf16 expects a bfloat16 tensor")
    if out is None:
        out = torch.empty(src.shape, dtype=torch.float32, device=src.device)
    with _ordered(q):
        L.check(L.lib().mcclx_decode_bf16(q.handle, out.data_ptr(), src.data_ptr(), src.numel()))
    return out
