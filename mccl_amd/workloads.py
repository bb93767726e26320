"""Synthetic inputs of the five measured configurations (deterministic per
(config, rank)), used by bench.py, the smoke check and the full-size tests.

  C1  ring,      2 ranks, 1,048,576 fp32 ~N(0,1), SUM, no wire codec
  C2  butterfly, 3 ranks, 6,553,600 fp32 (one 25 MiB DDP bucket) ~N(0,1e-3) with
      0.1 % outliers at +-1e2, bf16 wire, AVG (x 1/3)            <- headline
  C3  ring,      4 ranks, 110,000,002 fp32 ~N(0,1e-4), bf16 wire, ragged tail
  C4  tree,      3 ranks, 4096 messages x 16,384 fp32 ~U[-1,1], SUM
  C5  reduce_scatter + allgather, 8 ranks x 268,435,456 bf16 ~N(0,1e-2) plus
      NaN / +-Inf / denormals at fixed indices
"""
from __future__ import annotations

import numpy as np

SEED_BASE = 0x6D63636C00000000  # "mccl" << 32

C1 = dict(name="C1", algo="ring", world=2, numel=1_048_576, op="sum", wire=False)
C2 = dict(name="C2", algo="butterfly", world=3, numel=6_553_600, op="avg", wire=True)
C3 = dict(name="C3", algo="ring", world=4, numel=110_000_002, op="sum", wire=True)
C4 = dict(name="C4", algo="tree", world=3, messages=4096, numel=16_384, op="sum", wire=False)
C5 = dict(name="C5", world=8, numel=268_435_456, op="sum")


def rng_for(config: int, rank: int, extra: int = 0) -> np.random.Generator:
    return np.random.default_rng(SEED_BASE | (config << 8) | rank | (extra << 16))


def c1_input(rank: int, numel: int = C1["numel"]) -> np.ndarray:
    return rng_for(1, rank).standard_normal(numel, dtype=np.float32)


def c2_input(rank: int, numel: int = C2["numel"], variant: int = 0) -> np.ndarray:
    """N(0, 1e-3) gradients with 0.1 % of indices at +-1e2."""
    g = rng_for(2, rank, variant)
    x = g.standard_normal(numel, dtype=np.float32) * np.float32(1e-3)
    n_out = max(1, numel // 1000)
    idx = g.choice(numel, size=n_out, replace=False)
    x[idx] = np.where(g.integers(0, 2, n_out) == 0, np.float32(1e2), np.float32(-1e2))
    return x


def c3_input(rank: int, numel: int = C3["numel"]) -> np.ndarray:
    return rng_for(3, rank).standard_normal(numel, dtype=np.float32) * np.float32(1e-4)


def c4_input(rank: int, messages: int = C4["messages"], numel: int = C4["numel"]) -> np.ndarray:
    return rng_for(4, rank).uniform(-1.0, 1.0, messages * numel).astype(np.float32)


C5_SPECIALS_F32 = np.array([0x7FC00000, 0x7F800001, 0x7F800000, 0xFF800000, 0x00000000, 0x80000000,
                            0x00010000, 0x007F0000, 0x7F7F0000, 0xFF7F0000], dtype=np.uint32)


def c5_input_bf16_bits(rank: int, numel: int = C5["numel"]) -> np.ndarray:
    """bf16 bit patterns: N(0,1e-2), with qNaN, sNaN, +-Inf, +-0, min/max
    denormal and +-max finite cycling through indices i = 0 mod 1,000,003."""
    g = rng_for(5, rank)
    x = g.standard_normal(numel, dtype=np.float32) * np.float32(1e-2)
    u = x.view(np.uint32)
    # round to nearest even on the bit pattern (finite values only here)
    bits = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    idx = np.arange(0, numel, 1_000_003)
    sp = (C5_SPECIALS_F32 >> 16).astype(np.uint16)
    bits[idx] = sp[(np.arange(idx.size) + rank) % sp.size]
    return bits
