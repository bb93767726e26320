"""Makes "mccl" a torch.distributed backend for ROCm tensors.

What the reference's mccl/_backend.py:30-75 does for MPS: `register()` can be
called any number of times, hands torch a creator
`(prefix_store, rank, world_size, timeout) -> Backend` around the native
factory `_C._create_process_group_mccl`, and makes sure the factory always
receives a timedelta.

ROCm tensors have device type "cuda", whose c10d ops torch registers itself, so
the reference's MPS-to-CPU redispatch shim (csrc/backend/MPSFallback.cpp) has no
counterpart here.
"""
from __future__ import annotations

import datetime
import threading
import warnings

BACKEND_NAME = "mccl"
DEVICES = ["cuda"]
DEFAULT_TIMEOUT = datetime.timedelta(minutes=30)

_lock = threading.Lock()
_done = False


def _as_timedelta(timeout) -> datetime.timedelta:
    if isinstance(timeout, datetime.timedelta):
        return timeout
    if isinstance(timeout, (int, float)) and timeout > 0:
        return datetime.timedelta(seconds=timeout)
    return DEFAULT_TIMEOUT


def _skip(reason: str) -> bool:
    warnings.warn(f"backend '{BACKEND_NAME}' not registered: {reason}", RuntimeWarning, stacklevel=3)
    return False


def register() -> bool:
    """True once torch.distributed knows the backend; False (with a warning) if it cannot."""
    global _done
    with _lock:
        if _done:
            return True
        try:
            import torch.distributed as dist
        except ImportError:
            return _skip("torch.distributed is not available")
        try:
            from mccl_amd import _C
            factory = _C._create_process_group_mccl
        except (ImportError, AttributeError) as e:
            return _skip(f"the native extension mccl_amd._C is missing or incomplete ({e})")

        def create(prefix_store, rank, world_size, timeout):
            return factory(prefix_store, rank, world_size, _as_timedelta(timeout))

        try:
            dist.Backend.register_backend(BACKEND_NAME, create, devices=DEVICES)
        except TypeError:  # a torch that predates the `devices` argument
            dist.Backend.register_backend(BACKEND_NAME, create)
        _done = True
        return True
