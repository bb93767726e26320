"""Pins the oracle's element kernels: the reference's known-answer vectors
(tests/test_local_kernels.py), torch CPU bf16 arithmetic, numpy fp16 arithmetic,
and the closed forms of the scale constants."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG, PRODUCT, MIN, MAX

TAIL_SIZES = (1, 3, 7, 13, 97, 997)  # reference tests/test_local_kernels.py:82-90


def f32(*v):
    return np.array(v, dtype=np.float32)


def bf(x):
    return orc.encode_bf16(np.asarray(x, dtype=np.float32))


def hf(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def tbf(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def tbits(t):
    return t.view(torch.int16).numpy().view(np.uint16)


# ---- reference known-answer vectors ------------------------------------

def test_kat_accumulate_f32():  # test_local_kernels.py:67-73
    a, b = f32(1, 2, 3), f32(4, 5, 6)
    assert orc.reduce(a, b, F32, SUM) == 0
    assert np.array_equal(a, f32(5, 7, 9))


@pytest.mark.parametrize("n", TAIL_SIZES)
@pytest.mark.parametrize("dtype,enc", [(F32, lambda x: x), (F16, hf), (BF16, bf)])
def test_kat_tail_sizes(n, dtype, enc):  # :82-90, :115-123
    a = enc(np.full(n, 2.0, dtype=np.float32))
    b = enc(np.full(n, 3.0, dtype=np.float32))
    orc.reduce(a, b, dtype, SUM)
    assert np.array_equal(a, enc(np.full(n, 5.0, dtype=np.float32)))


def test_kat_min_max_product():  # :125-214
    a, b = f32(1, 5, 3), f32(4, 2, 6)
    x = a.copy(); orc.reduce(x, b, F32, MIN); assert np.array_equal(x, f32(1, 2, 3))
    x = a.copy(); orc.reduce(x, b, F32, MAX); assert np.array_equal(x, f32(4, 5, 6))
    x = f32(2, 3, 4); orc.reduce(x, f32(5, 6, 7), F32, PRODUCT); assert np.array_equal(x, f32(10, 18, 28))
    for enc in (hf, bf):
        x = enc([1, 5, 3]); orc.reduce(x, enc([4, 2, 6]), F16 if enc is hf else BF16, MIN)
        assert np.array_equal(x, enc([1, 2, 3]))
        x = enc([2, 3, 4]); orc.reduce(x, enc([5, 6, 7]), F16 if enc is hf else BF16, PRODUCT)
        assert np.array_equal(x, enc([10, 18, 28]))


def test_kat_scale():  # :218-241
    x = f32(2, 4, 6); orc.scale(x, F32, 0.5); assert np.array_equal(x, f32(1, 2, 3))
    for world in (2, 3, 4, 8):
        x = np.full(256, float(world), dtype=np.float32)
        orc.scale(x, F32, 1.0 / world)
        assert np.allclose(x, 1.0, rtol=1e-5, atol=1e-5)
    x = hf([2, 4, 6]); orc.scale(x, F16, 0.5); assert np.array_equal(x, hf([1, 2, 3]))


def test_kat_accumulate_scale():  # :264-271
    a = f32(1, 3, 5); orc.accumulate_scale(a, f32(3, 5, 7), F32, 0.5)
    assert np.array_equal(a, f32(2, 4, 6))
    a = hf([1, 3, 5]); orc.accumulate_scale(a, hf([3, 5, 7]), F16, 0.5)
    assert np.array_equal(a, hf([2, 4, 6]))


def test_unsupported_op_is_rejected():  # MetalKernels.mm:546-548
    a = f32(1, 2)
    for bad in (5, 6, 7, 8, 99):
        assert orc.reduce(a, a.copy(), F32, bad) == -1


# ---- what IEEE-754 / third-party arithmetic fixes -----------------------

def test_f32_ops_match_numpy_bit_for_bit():
    rng = np.random.default_rng(11)
    a = rng.standard_normal(100003).astype(np.float32)
    b = rng.standard_normal(100003).astype(np.float32)
    # include denormals and huge values
    a[:100] = np.float32(1e-41); b[:100] = np.float32(3e-42)
    a[100:200] = np.float32(3e38); b[100:200] = np.float32(3e38)
    for op, fn in ((SUM, np.add), (PRODUCT, np.multiply), (MIN, np.minimum), (MAX, np.maximum)):
        x = a.copy()
        orc.reduce(x, b, F32, op)
        with np.errstate(over="ignore", under="ignore"):
            assert np.array_equal(x.view(np.uint32), fn(a, b).view(np.uint32)), op
    x = a.copy(); orc.scale(x, F32, 1.0 / 3)
    with np.errstate(under="ignore"):
        assert np.array_equal(x.view(np.uint32), (a * np.float32(1.0 / 3)).view(np.uint32))
    x = a.copy(); orc.accumulate_scale(x, b, F32, 1.0 / 3)
    with np.errstate(over="ignore", under="ignore"):
        assert np.array_equal(x.view(np.uint32), ((a + b) * np.float32(1.0 / 3)).view(np.uint32))


def _bf16_operands():
    rng = np.random.default_rng(5)
    h = rng.integers(0, 65536, size=400000, dtype=np.uint32).astype(np.uint16)
    g = rng.integers(0, 65536, size=400000, dtype=np.uint32).astype(np.uint16)
    # near-cancellation, equal exponents, specials x specials
    g[:50000] = h[:50000] ^ np.uint16(0x8000) ^ rng.integers(0, 4, 50000).astype(np.uint16)
    sp = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80,
                   0x7FC0, 0xFFC0, 0x7F81, 0x3F80, 0xBF80, 0x3EAA, 0x3EAB], dtype=np.uint16)
    A, B = np.meshgrid(sp, sp)
    return np.concatenate([h, A.ravel()]), np.concatenate([g, B.ravel()])


@pytest.mark.parametrize("op,fn", [(SUM, torch.add), (PRODUCT, torch.mul)])
def test_bf16_step_matches_torch(op, fn):
    a, b = _bf16_operands()
    x = a.copy()
    orc.reduce(x, b, BF16, op)
    want = tbits(fn(tbf(a), tbf(b)))
    nan = (want & 0x7FFF) > 0x7F80
    assert np.array_equal(x[~nan], want[~nan])
    assert np.all(x[nan] == 0x7FC0)  # canonical NaN, as the scalar torch conversion


def test_bf16_min_max_match_torch_on_non_nan():
    a, b = _bf16_operands()
    ok = ((a & 0x7FFF) <= 0x7F80) & ((b & 0x7FFF) <= 0x7F80)
    # +0/-0 ties: the "y if y < x else x" definition keeps dst; torch may pick either zero
    ok &= ~(((a & 0x7FFF) == 0) & ((b & 0x7FFF) == 0))
    a, b = a[ok], b[ok]
    for op, fn in ((MIN, torch.minimum), (MAX, torch.maximum)):
        x = a.copy(); orc.reduce(x, b, BF16, op)
        assert np.array_equal(x, tbits(fn(tbf(a), tbf(b))))


def test_min_max_keep_dst_on_nan_and_signed_zero():
    nan = np.float32(np.nan)
    for op in (MIN, MAX):
        x = f32(1.0, nan, 0.0, -0.0)
        orc.reduce(x, f32(nan, 1.0, -0.0, 0.0), F32, op)
        assert x[0] == 1.0 and np.isnan(x[1])
        assert x.view(np.uint32)[2] == 0x00000000 and x.view(np.uint32)[3] == 0x80000000


def test_f16_ops_match_numpy():
    rng = np.random.default_rng(9)
    a = rng.integers(0, 65536, 300000, dtype=np.uint32).astype(np.uint16)
    b = rng.integers(0, 65536, 300000, dtype=np.uint32).astype(np.uint16)
    fa, fb = a.view(np.float16), b.view(np.float16)
    ok = ~(np.isnan(fa) | np.isnan(fb))
    a, b, fa, fb = a[ok], b[ok], fa[ok], fb[ok]
    for op, fn in ((SUM, np.add), (PRODUCT, np.multiply)):
        x = a.copy(); orc.reduce(x, b, F16, op)
        with np.errstate(all="ignore"):
            want = fn(fa, fb)
        good = ~np.isnan(want)
        assert np.array_equal(x[good], want.view(np.uint16)[good])
        assert np.all(np.isnan(x.view(np.float16)[~good]))


def test_bf16_scale_matches_torch():
    h = np.arange(65536, dtype=np.uint16)
    for world in (2, 3, 4, 5, 7, 8):
        for mode in (orc.SCALE_VIEW, orc.SCALE_TENSOR):
            sbits = np.array([orc.scale_constant_bits(BF16, 1.0 / world, mode)], dtype=np.uint16)
            x = h.copy(); orc.scale(x, BF16, 1.0 / world, mode)
            want = tbits(tbf(h) * tbf(sbits))
            nan = (want & 0x7FFF) > 0x7F80
            assert np.array_equal(x[~nan], want[~nan])
            assert np.all(x[nan] == 0x7FC0)


# ---- scale constants: closed forms ---------------------------------------

def test_scale_constants():
    C = orc.scale_constant_bits
    assert C(F32, 1 / 3, 0) == 0x3EAAAAAB
    assert C(BF16, 1 / 3, orc.SCALE_VIEW) == 0x3EAA      # MetalKernels.mm:659-662 truncates
    assert C(BF16, 1 / 3, orc.SCALE_TENSOR) == 0x3EAB    # MetalKernels.mm:390-392 rounds
    assert C(F16, 1 / 3, 0) == 0x3555
    for n, f, b, h in ((2, 0x3F000000, 0x3F00, 0x3800), (4, 0x3E800000, 0x3E80, 0x3400),
                       (8, 0x3E000000, 0x3E00, 0x3000)):
        assert C(F32, 1 / n, 0) == f
        assert C(BF16, 1 / n, 0) == b and C(BF16, 1 / n, 1) == b
        assert C(F16, 1 / n, 0) == h
    assert C(BF16, 1 / 7, orc.SCALE_VIEW) == 0x3E12 and C(BF16, 1 / 7, orc.SCALE_TENSOR) == 0x3E12
    assert C(BF16, 1 / 5, orc.SCALE_VIEW) == 0x3E4C and C(BF16, 1 / 5, orc.SCALE_TENSOR) == 0x3E4D


def test_power_of_two_scale_is_exact_and_bf16_accumulate_scale_rounds_twice():
    rng = np.random.default_rng(2)
    a = bf(rng.standard_normal(5000)); b = bf(rng.standard_normal(5000))
    x = a.copy(); orc.accumulate_scale(x, b, BF16, 0.5)
    y = a.copy(); orc.reduce(y, b, BF16, SUM); orc.scale(y, BF16, 0.5, orc.SCALE_TENSOR)
    assert np.array_equal(x, y)
    # halving a bf16 normal only lowers the exponent
    v = orc.decode_bf16(y) * 2
    s = a.copy(); orc.reduce(s, b, BF16, SUM)
    assert np.array_equal(orc.decode_bf16(s), v)
