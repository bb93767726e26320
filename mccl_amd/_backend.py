"""Registers the "mccl" c10d backend with torch.distributed for ROCm tensors.

Counterpart of the reference's mccl/_backend.py:30-75: `register()` is
idempotent, coerces the timeout to a timedelta, and hands torch a creator
function `(prefix_store, rank, world_size, timeout) -> Backend` that calls the
native factory `_C._create_process_group_mccl`.

Device list: ROCm tensors have device type "cuda", whose c10d ops torch
registers itself, so the reference's MPS-to-CPU redispatch shim
(csrc/backend/MPSFallback.cpp) has no counterpart here.
"""
from __future__ import annotations

import datetime as _dt
import warnings as _warnings

_REGISTERED = False

BACKEND_NAME = "mccl"
DEVICES = ["cuda"]


def register() -> bool:
    """Register the 'mccl' backend.  Returns True once it is registered."""
    global _REGISTERED
    if _REGISTERED:
        return True
    try:
        import torch.distributed as dist
    except ImportError:
        _warnings.warn("torch.distributed not available; skipping mccl registration",
                       RuntimeWarning, stacklevel=2)
        return False
    try:
        from mccl_amd._C import _create_process_group_mccl
    except ImportError as e:
        _warnings.warn(f"mccl_amd._C native extension missing _create_process_group_mccl: {e}",
                       RuntimeWarning, stacklevel=2)
        return False

    def _create(prefix_store, rank, world_size, timeout):
        td = timeout if isinstance(timeout, _dt.timedelta) else _dt.timedelta(seconds=1800)
        return _create_process_group_mccl(prefix_store, rank, world_size, td)

    try:
        dist.Backend.register_backend(BACKEND_NAME, _create, devices=DEVICES)
    except TypeError:  # older torch without the devices argument
        dist.Backend.register_backend(BACKEND_NAME, _create)
    _REGISTERED = True
    return True
