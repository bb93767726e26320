"""mccl_amd -- the per-rank reduce + bf16 wire-codec path of dormlab/mccl as
hand-written CDNA4 HIP kernels behind a C ABI (libmcclx.so).

Layout:
  csrc/          HIP kernels, the C ABI, the C++ chunk scheduler
  _lib.py        ctypes binding of the C ABI (no fallback if the library is missing)
  kernels.py     counterpart of the reference's MetalKernels.hpp over torch tensors
  harness.py     N-virtual-rank replay of ring / tree / butterfly / reduce_scatter / allgather
"""
from ._lib import MCCLError, LIB_PATH  # noqa: F401

__version__ = "0.1.0"
