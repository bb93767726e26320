"""Single-process replay of the reference's collectives for N virtual ranks
whose tensors all live on one GPU (there is no cross-GPU traffic here).

`allreduce` follows ProcessGroupMCCL::allreduce (ProcessGroupMCCL.cpp:105-186):
it reads MCCL_WIRE_DTYPE / MCCL_ALLREDUCE_ALGO / MCCL_TREE_BELOW on every call,
resolves the algorithm exactly as the reference does, then hands the schedule
to the C++ chunk scheduler in libmcclx.so.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Sequence

import torch

from . import _lib as L
from ._lib import MCCLError
from .kernels import ReduceQueue, _q, _check_tensor, dtype_code, op_code

ALGO_NAMES = {"ring": L.ALGO_RING, "tree": L.ALGO_TREE, "butterfly": L.ALGO_BUTTERFLY}


def chunkize(numel: int, elem_size: int, world: int):
    """[(elem_start, elem_count, byte_off, byte_len)] -- AllreduceAlgos.cpp:22-34."""
    out = (L.Chunk * world)()
    L.check(L.lib().mcclx_chunkize(numel, elem_size, world, out))
    return [(c.elem_start, c.elem_count, c.byte_off, c.byte_len) for c in out]


def select_algo(env_algo: Optional[str], tree_below: Optional[int], wire_nbytes: int, numel: int,
                world: int) -> int:
    """ProcessGroupMCCL.cpp:134-145."""
    return L.lib().mcclx_select_algo(env_algo.encode() if env_algo is not None else None,
                                     -1 if tree_below is None else tree_below, wire_nbytes, numel,
                                     world)


def _env_config():
    wire = os.environ.get("MCCL_WIRE_DTYPE") == "bf16"          # PG.cpp:117-120
    algo = os.environ.get("MCCL_ALLREDUCE_ALGO")                 # :134
    below = os.environ.get("MCCL_TREE_BELOW")                    # :138-139 (strtoull)
    tree_below = None
    if below is not None:
        digits = ""
        for ch in below.strip():
            if not ch.isdigit():
                break
            digits += ch
        tree_below = int(digits) if digits else 0
    return wire, algo, tree_below


def _ptr_array(ptrs: Sequence[int]):
    return (C.c_void_p * len(ptrs))(*ptrs)


class Workspace:
    """Scratch for a replay: HBM (a torch byte tensor) or pinned host memory
    mapped into the device (the zero-copy path: the wire delivers into host RAM
    and the kernels read it across PCIe)."""

    def __init__(self, queue: ReduceQueue, nbytes: int, pinned_host: bool = False):
        self.queue, self.nbytes, self.pinned = queue, nbytes, pinned_host
        self._tensor = None
        self._host = None
        if nbytes == 0:
            self.ptr = 0
        elif pinned_host:
            self._host, self.ptr = queue.host_alloc(nbytes)
        else:
            self._tensor = torch.empty(nbytes + 256, dtype=torch.uint8, device=f"cuda:{queue.device}")
            self.ptr = (self._tensor.data_ptr() + 255) // 256 * 256

    def free(self):
        if self._host is not None:
            self.queue.host_free(self._host)
            self._host = None
        self._tensor = None


def allreduce_replay(tensors: List[torch.Tensor], op, algo: int, wire_bf16: bool = False,
                     mode: int = L.REPLAY_FUSED, acc: int = L.ACC_STEP, queue=None,
                     workspace: Optional[Workspace] = None, sync: bool = True) -> None:
    """In-place allreduce over the virtual ranks' tensors with a fixed algorithm."""
    q = _q(queue)
    if not tensors:
        raise MCCLError("[MCCL] Check failed: !tensors.empty() — allreduce: empty tensor list")
    for t in tensors:
        _check_tensor(t, "allreduce")
        if t.dtype != tensors[0].dtype or t.numel() != tensors[0].numel():
            raise MCCLError("[MCCL] allreduce: virtual ranks must hold same-shaped tensors")
    r = L.Replay()
    r.world = len(tensors)
    r.algo, r.op, r.dtype = algo, op_code(op), dtype_code(tensors[0])
    r.wire_bf16, r.mode, r.acc, r.reserved = int(wire_bf16), mode, acc, 0
    r.numel = tensors[0].numel()
    ptrs = _ptr_array([t.data_ptr() for t in tensors])
    r.tensors = ptrs
    # the scheduler runs the stepwise schedule itself when a fused request cannot be
    # folded (binary-only ops, fp16, more than MAX_INPUTS ranks): size for both
    need = L.lib().mcclx_replay_workspace_bytes(C.byref(r))
    if mode == L.REPLAY_FUSED:
        r.mode = L.REPLAY_STEPWISE
        need = max(need, L.lib().mcclx_replay_workspace_bytes(C.byref(r)))
        r.mode = mode
    own_ws = None
    if workspace is None:
        own_ws = workspace = Workspace(q, need)
    elif workspace.nbytes < need:
        raise MCCLError(f"[MCCL] workspace too small: {workspace.nbytes} < {need}")
    r.workspace = workspace.ptr or None
    r.workspace_bytes = workspace.nbytes
    q.wait_torch_stream()                      # PG.cpp:172 mps_stream_sync, without blocking the host
    L.check(L.lib().mcclx_allreduce_replay(q.handle, C.byref(r)))
    if sync or own_ws is not None:
        q.drain()                              # PG.cpp:178 mccl_queue_drain
    else:
        q.torch_stream_wait()
    if own_ws is not None:
        own_ws.free()


def allreduce_replay_many(groups: List[List[torch.Tensor]], op, algo: int, wire_bf16: bool = False,
                          mode: int = L.REPLAY_FUSED, acc: int = L.ACC_STEP, queue=None) -> None:
    """A list of allreduces (groups[i] = the virtual ranks' tensors of message i), as a
    c10d allreduce over a list of tensors: entries that share a plan go out together,
    one launch per phase for all of them."""
    q = _q(queue)
    reps = (L.Replay * len(groups))()
    keep = []
    needs = []
    for i, tensors in enumerate(groups):
        for t in tensors:
            _check_tensor(t, "allreduce")
        r = reps[i]
        r.world = len(tensors)
        r.algo, r.op, r.dtype = algo, op_code(op), dtype_code(tensors[0])
        r.wire_bf16, r.mode, r.acc, r.reserved = int(wire_bf16), L.REPLAY_STEPWISE, acc, 0
        r.numel = tensors[0].numel()
        ptrs = _ptr_array([t.data_ptr() for t in tensors])
        keep.append(ptrs)
        r.tensors = ptrs
        need = L.lib().mcclx_replay_workspace_bytes(C.byref(r))     # stepwise needs the most
        r.mode = mode
        needs.append((max(need, L.lib().mcclx_replay_workspace_bytes(C.byref(r))) + 255) // 256 * 256)
    ws = Workspace(q, sum(needs))
    off = 0
    for i, need in enumerate(needs):
        reps[i].workspace = (ws.ptr + off) or None
        reps[i].workspace_bytes = need
        off += need
    q.wait_torch_stream()
    try:
        L.check(L.lib().mcclx_allreduce_replay_many(q.handle, reps, len(groups)))
    finally:
        q.drain()
        ws.free()


def allreduce(tensors: List[torch.Tensor], op="sum", queue=None, mode: int = L.REPLAY_FUSED) -> int:
    """ProcessGroupMCCL::allreduce for N virtual ranks; returns the algorithm used."""
    wire, env_algo, tree_below = _env_config()
    t0 = tensors[0]
    use_wire = wire and t0.dtype == torch.float32
    wire_nbytes = t0.numel() * (2 if use_wire else t0.element_size())
    algo = select_algo(env_algo, tree_below, wire_nbytes, t0.numel(), len(tensors))
    allreduce_replay(tensors, op, algo, wire_bf16=wire, mode=mode, queue=queue)
    return algo


def reduce_scatter_replay(outs: List[torch.Tensor], ins: List[torch.Tensor], op="sum",
                          mode: int = L.REPLAY_FUSED, acc: int = L.ACC_STEP, queue=None) -> None:
    """_reduce_scatter_base (ProcessGroupMCCL.cpp:331-390) for every virtual rank."""
    q = _q(queue)
    world = len(ins)
    for o, i in zip(outs, ins):
        _check_tensor(o, "_reduce_scatter_base")
        _check_tensor(i, "_reduce_scatter_base")
        if i.numel() * i.element_size() != o.numel() * o.element_size() * world:
            raise MCCLError("[MCCL] Check failed: send_sb.nbytes == chunk * world — "
                            "_reduce_scatter_base: input size != output * world")
    q.wait_torch_stream()
    L.check(L.lib().mcclx_reduce_scatter_replay(
        q.handle, world, _ptr_array([o.data_ptr() for o in outs]),
        _ptr_array([i.data_ptr() for i in ins]), dtype_code(outs[0]), outs[0].numel(), op_code(op),
        mode, acc))
    q.drain()


def allgather_replay(outs: List[torch.Tensor], ins: List[torch.Tensor], queue=None) -> None:
    """_allgather_base (ProcessGroupMCCL.cpp:232-273) for every virtual rank."""
    q = _q(queue)
    world = len(ins)
    chunk = ins[0].numel() * ins[0].element_size()
    for o in outs:
        _check_tensor(o, "_allgather_base")
        if o.numel() * o.element_size() != chunk * world:
            raise MCCLError("[MCCL] Check failed: total == chunk * world — "
                            "_allgather_base: output size != input * world")
    q.wait_torch_stream()
    L.check(L.lib().mcclx_allgather_replay(
        q.handle, world, _ptr_array([o.data_ptr() for o in outs]),
        _ptr_array([i.data_ptr() for i in ins]), chunk))
    q.drain()
