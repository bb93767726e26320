"""Helpers shared by the GPU parity tests: numpy <-> device tensors by bit pattern."""
import numpy as np
import torch

from oracle import oracle as orc

TORCH_DT = {orc.F32: torch.float32, orc.F16: torch.float16, orc.BF16: torch.bfloat16}


def to_dev(a: np.ndarray, dtype: int) -> torch.Tensor:
    """fp32 arrays as float32; uint16 bit patterns reinterpreted as f16 / bf16."""
    if dtype == orc.F32:
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint16).view(np.int16)).cuda()
    return t.view(TORCH_DT[dtype])


def bits(t: torch.Tensor) -> np.ndarray:
    """Device tensor -> numpy bit patterns (uint32 for fp32, uint16 otherwise)."""
    if t.dtype == torch.float32:
        return t.detach().cpu().numpy().view(np.uint32)
    return t.detach().view(torch.int16).cpu().numpy().view(np.uint16)


def np_bits(a: np.ndarray) -> np.ndarray:
    return a.view(np.uint32) if a.dtype == np.float32 else a


def assert_same_bits(got: torch.Tensor, want: np.ndarray, dtype: int, what=""):
    """Bit-exact, except that fp32 NaNs only need to be NaN on both sides (the
    payload of a NaN produced by an fp32 add differs between x86 and the GPU);
    16-bit results are canonicalised by the encode, so they compare exactly."""
    g = bits(got)
    w = np_bits(np.ascontiguousarray(want))
    assert g.shape == w.shape, (what, g.shape, w.shape)
    if dtype == orc.F32:
        gn = np.isnan(g.view(np.float32))
        wn = np.isnan(w.view(np.float32))
        assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
        same = (g == w) | gn
    else:
        same = g == w
    if not same.all():
        i = int(np.flatnonzero(~same)[0])
        raise AssertionError(f"{what}: {int((~same).sum())} of {same.size} differ; first at {i}: "
                             f"got {int(g[i]):#x} want {int(w[i]):#x}")


def rand_values(rng, n, dtype, scale=1.0, specials=False):
    """Random payload in the buffer's own representation."""
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    if specials and n >= 16:
        sp = np.array([np.nan, -np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, -1e-40, 9.2e-41, 3.3e38,
                       -3.3e38, 3.4e38, 1.0, -1.0, 65504.0, 1e-8], dtype=np.float32)
        idx = rng.choice(n, size=min(n, 4 * sp.size), replace=False)
        x[idx] = np.resize(sp, idx.size)
    if dtype == orc.F32:
        return x
    if dtype == orc.BF16:
        return orc.encode_bf16(x)
    with np.errstate(over="ignore"):
        return x.astype(np.float16).view(np.uint16)
