"""Pins the oracle's scalar codecs.

bf16 encode/decode are checked against torch's CPU cast -- the very call the
reference makes (ProcessGroupMCCL.cpp:131-132, :181) -- and against the special
values IEEE-754 and the torch header fix.  fp16 is checked against numpy.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as orc


def torch_encode(x_f32: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x_f32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def is_bf16_nan(h):
    return (h & 0x7FFF) > 0x7F80


SPECIALS = {
    0x7F800000: 0x7F80,  # +Inf
    0xFF800000: 0xFF80,  # -Inf
    0x7F7FFFFF: 0x7F80,  # max finite rounds up to Inf
    0xFF7FFFFF: 0xFF80,
    0x7F7F0000: 0x7F7F,  # max bf16 stays
    0x7F7F7FFF: 0x7F7F,  # just below the tie: down
    0x7F7F8000: 0x7F80,  # tie, odd kept bit: up to Inf
    0x3F808000: 0x3F80,  # tie, even kept bit: down
    0x3F818000: 0x3F82,  # tie, odd kept bit: up
    0x3F808001: 0x3F81,  # above tie: up
    0x3F807FFF: 0x3F80,  # below tie: down
    0x00008000: 0x0000,  # denormal tie to even (zero)
    0x00018000: 0x0002,  # denormal tie to even (up)
    0x00008001: 0x0001,  # denormal above tie
    0x00010000: 0x0001,  # min bf16 denormal exact
    0x007F8000: 0x0080,  # largest denormal tie rounds into the normals
    0x80000000: 0x8000,  # -0
    0x00000000: 0x0000,
    0x7FC00000: 0x7FC0,  # qNaN
    0x7F800001: 0x7FC0,  # sNaN -> canonical
    0xFFC00000: 0x7FC0,  # negative NaN loses its sign
    0xFFFFFFFF: 0x7FC0,
    0x7F80FFFF: 0x7FC0,  # NaN whose rounding would carry into Inf without the NaN test
}


def test_encode_specials():
    L = orc.lib()
    for bits, want in SPECIALS.items():
        x = np.array([bits], dtype=np.uint32).view(np.float32)
        got = orc.encode_bf16(x)[0]
        assert L.orc_f32_to_bf16(float(x[0])) == want or np.isnan(x[0])
        assert got == want, f"{bits:#010x}: got {got:#06x} want {want:#06x}"


def test_encode_matches_torch_strided_sweep():
    # every 4099th pattern of the 2^32 (about one million), plus all patterns
    # whose dropped half sits on or beside the tie point.
    bits = np.arange(0, 2**32, 4099, dtype=np.uint64).astype(np.uint32)
    hi = (np.arange(65536, dtype=np.uint32) << 16)
    ties = np.concatenate([hi | lo for lo in (0x7FFF, 0x8000, 0x8001, 0x0000, 0xFFFF, 0x0001)])
    allb = np.concatenate([bits, ties])
    x = allb.view(np.float32)
    got = orc.encode_bf16(x)
    want = torch_encode(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN: torch's AVX path emits 0xFFFF and its scalar path 0x7FC0 (both NaN);
    # the oracle follows the header's scalar algorithm.
    assert np.all(is_bf16_nan(want[nan]))
    assert np.all(got[nan] == 0x7FC0)


def test_encode_is_nearest_even_by_brute_force():
    # independent statement: the result is the bf16 neighbour closest in value,
    # ties to the even pattern, checked in float64.
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    fin = np.isfinite(x) & (np.abs(x) < 3.3e38)
    x = x[fin]
    bits = bits[fin]
    got = orc.encode_bf16(x)
    lo = (bits >> 16).astype(np.uint32)           # truncation neighbour
    hi = lo + 1                                    # next pattern away from zero
    vlo = (lo << 16).view(np.float32).astype(np.float64)
    vhi = (hi << 16).astype(np.uint32).view(np.float32).astype(np.float64)
    xv = x.astype(np.float64)
    dlo, dhi = np.abs(xv - vlo), np.abs(vhi - xv)
    want = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo & 1, hi, lo)))
    assert np.array_equal(got.astype(np.uint32), want.astype(np.uint32))


def test_decode_all_65536():
    h = np.arange(65536, dtype=np.uint16)
    got = orc.decode_bf16(h).view(np.uint32)
    assert np.array_equal(got, h.astype(np.uint32) << 16)
    want = torch.from_numpy(h.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got, want.view(np.uint32))


def test_decode_encode_round_trip():
    h = np.arange(65536, dtype=np.uint16)
    back = orc.encode_bf16(orc.decode_bf16(h))
    nan = is_bf16_nan(h)
    assert np.array_equal(back[~nan], h[~nan])
    assert np.all(back[nan] == 0x7FC0)


def test_f16_decode_all_65536_matches_numpy():
    L = orc.lib()
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([np.float32(L.orc_f16_to_f32(int(v))) for v in h], dtype=np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got.view(np.float32)[nan]))


def test_f16_encode_matches_numpy():
    L = orc.lib()
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2**32, size=30000, dtype=np.uint64).astype(np.uint32)
    # add every half value, its midpoints to both neighbours and the overflow edge
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    x = np.concatenate([bits.view(np.float32), mids, -mids,
                        np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e-8, 2.98e-8, 2.9802322e-8, 3e-8],
                                 dtype=np.float32)])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_f64_to_f16_single_rounding():
    L = orc.lib()
    for n in (2, 3, 4, 5, 6, 7, 8, 16, 30):
        want = np.float64(1.0 / n).astype(np.float16).view(np.uint16)
        assert L.orc_f64_to_f16(1.0 / n) == want
    # a value where double -> float -> half would round twice and differ:
    # 1 + 2^-11 + 2^-30 is above the half tie, but (float) drops the 2^-30.
    v = 1.0 + 2.0**-11 + 2.0**-30
    assert L.orc_f64_to_f16(v) == 0x3C01
    assert np.float32(v).astype(np.float16).view(np.uint16) == 0x3C00
