"""mccl_amd -- the per-rank reduce + bf16 wire-codec path of dormlab/mccl as
hand-written CDNA4 HIP kernels behind a C ABI (libmcclx.so), with the
reference's c10d backend surface on top.

Layout:
  csrc/          HIP kernels, the C ABI, the C++ chunk scheduler, the c10d backend
  _lib.py        ctypes binding of the C ABI (no fallback if the library is missing)
  kernels.py     counterpart of the reference's MetalKernels.hpp over torch tensors
  harness.py     N-virtual-rank replay of ring / tree / butterfly / reduce_scatter / allgather
  _backend.py    registers backend "mccl" with torch.distributed (reference: mccl/_backend.py)

Importing the package registers the backend when the native extension is
built, as the reference's mccl/__init__.py:38-45 does; if it is not, a warning
says so and `init_process_group("mccl")` stays unavailable -- nothing falls
back to another implementation.
"""
import warnings as _warnings

import torch as _torch  # noqa: F401  first: its HIP runtime must be the one libmcclx binds to (see _lib.py)

from ._lib import MCCLError, LIB_PATH  # noqa: F401
from ._backend import register

__version__ = "0.1.0"

try:
    from . import _C  # noqa: F401
    register()
except ImportError as _e:  # pragma: no cover - depends on the build state
    _warnings.warn(f"mccl_amd native backend not loaded: {_e}", RuntimeWarning, stacklevel=2)

__all__ = ["__version__", "MCCLError", "register"]
