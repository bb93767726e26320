"""GPU parity of the element kernels through the C ABI (libmcclx.so) against
the CPU oracle: the reference's known-answer vectors, bit-exact random sweeps
over dtypes / ops / tail sizes / misaligned offsets, and the bf16 codec."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG, PRODUCT, MIN, MAX

pytestmark = pytest.mark.gpu

TAIL_SIZES = (1, 3, 7, 13, 97, 997)  # reference tests/test_local_kernels.py:82-90


@pytest.fixture(scope="module")
def K():
    from mccl_amd import kernels
    kernels.hip_kernels_init(0)
    return kernels


@pytest.fixture(scope="module")
def U():
    import gpu_util
    return gpu_util


def dev(v, dtype=torch.float32):
    return torch.tensor(v, dtype=dtype, device="cuda")


# ---- the reference's own kernel tests, restated ----------------------------

class TestAccumulateChunk:  # tests/test_local_kernels.py:66-123
    def test_f32_basic(self, K):
        r = K.hip_accumulate_chunk(dev([1.0, 2.0, 3.0]), dev([4.0, 5.0, 6.0])); K.hip_sync()
        assert torch.equal(r, dev([5.0, 7.0, 9.0]))

    def test_f32_zeros(self, K):
        b = torch.ones(256, device="cuda") * 3.0
        r = K.hip_accumulate_chunk(torch.zeros(256, device="cuda"), b); K.hip_sync()
        assert torch.equal(r, b)

    @pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
    def test_non_aligned_size(self, K, dtype):
        for size in TAIL_SIZES:
            a = torch.ones(size, device="cuda", dtype=dtype) * 2.0
            b = torch.ones(size, device="cuda", dtype=dtype) * 3.0
            r = K.hip_accumulate_chunk(a, b); K.hip_sync()
            assert torch.equal(r, torch.ones(size, device="cuda", dtype=dtype) * 5.0), size

    def test_f32_large(self, K):
        torch.manual_seed(0)
        a = torch.randn(1_000_000, device="cuda"); b = torch.randn(1_000_000, device="cuda")
        want = a.cpu() + b.cpu()
        r = K.hip_accumulate_chunk(a, b); K.hip_sync()
        assert torch.equal(r.cpu(), want)  # the reference asserts rtol 1e-5; IEEE add is exact

    def test_f16_basic(self, K):
        h = torch.float16
        r = K.hip_accumulate_chunk(dev([1, 2, 3], h), dev([4, 5, 6], h)); K.hip_sync()
        assert torch.equal(r, dev([5, 7, 9], h))


class TestMinMaxProduct:  # :125-214
    def test_basic(self, K):
        for dt in (torch.float32, torch.float16, torch.bfloat16):
            r = K.hip_elementwise_min(dev([1, 5, 3], dt), dev([4, 2, 6], dt)); K.hip_sync()
            assert torch.equal(r, dev([1, 2, 3], dt))
            r = K.hip_elementwise_max(dev([1, 5, 3], dt), dev([4, 2, 6], dt)); K.hip_sync()
            assert torch.equal(r, dev([4, 5, 6], dt))
            r = K.hip_elementwise_product(dev([2, 3, 4], dt), dev([5, 6, 7], dt)); K.hip_sync()
            assert torch.equal(r, dev([10, 18, 28], dt))

    def test_non_aligned(self, K):
        torch.manual_seed(1)
        for size in (1, 3, 7, 13, 97):
            a = torch.randn(size, device="cuda"); b = torch.randn(size, device="cuda")
            r = K.hip_elementwise_min(a.clone(), b); K.hip_sync(); assert torch.equal(r, torch.minimum(a, b))
            r = K.hip_elementwise_max(a.clone(), b); K.hip_sync(); assert torch.equal(r, torch.maximum(a, b))
            r = K.hip_elementwise_product(a.clone(), b); K.hip_sync(); assert torch.equal(r, a * b)


class TestScale:  # :218-260
    def test_f32_half_identity_world(self, K):
        r = K.hip_scale_inplace(dev([2.0, 4.0, 6.0]), 0.5); K.hip_sync()
        assert torch.equal(r, dev([1.0, 2.0, 3.0]))
        a = torch.randn(1000, device="cuda")
        r = K.hip_scale_inplace(a.clone(), 1.0); K.hip_sync(); assert torch.equal(r, a)
        for world in (2, 3, 4, 8):
            r = K.hip_scale_inplace(torch.ones(256, device="cuda") * world, 1.0 / world); K.hip_sync()
            assert torch.allclose(r, torch.ones(256, device="cuda"), rtol=1e-5, atol=1e-5)

    def test_f16(self, K):
        h = torch.float16
        r = K.hip_scale_inplace(dev([2, 4, 6], h), 0.5); K.hip_sync()
        assert torch.equal(r, dev([1, 2, 3], h))


class TestAccumulateAndScale:  # :264-292
    def test_avg_two_ranks(self, K):
        for dt in (torch.float32, torch.float16, torch.bfloat16):
            r = K.hip_accumulate_and_scale(dev([1, 3, 5], dt), dev([3, 5, 7], dt), 0.5); K.hip_sync()
            assert torch.equal(r, dev([2, 4, 6], dt))


# ---- error behaviour ---------------------------------------------------------

def test_errors(K):
    from mccl_amd import MCCLError
    a = torch.ones(8, device="cuda")
    with pytest.raises(MCCLError, match="Unsupported ReduceOp: 7"):   # MetalKernels.mm:546-548
        K.hip_reduce_op(a, a.clone(), 7)
    with pytest.raises(MCCLError, match="Shape mismatch"):
        K.hip_reduce_op(a, torch.ones(9, device="cuda"), SUM)
    with pytest.raises(MCCLError, match="Dtype mismatch"):
        K.hip_reduce_op(a, torch.ones(8, device="cuda", dtype=torch.float16), SUM)
    with pytest.raises(MCCLError, match="must live on the GPU"):
        K.hip_reduce_op(torch.ones(8), torch.ones(8), SUM)
    with pytest.raises(MCCLError, match="contiguous"):
        K.hip_reduce_op(torch.ones(8, 2, device="cuda").t(), torch.ones(2, 8, device="cuda"), SUM)
    with pytest.raises(MCCLError, match="No HIP kernel for dtype"):
        K.hip_reduce_op(torch.ones(8, device="cuda", dtype=torch.float64),
                        torch.ones(8, device="cuda", dtype=torch.float64), SUM)
    K.hip_begin_batch("x")
    with pytest.raises(MCCLError, match="batch already active"):     # MetalKernels.mm:562
        K.hip_begin_batch("y")
    K.hip_end_batch(); K.hip_end_batch()                              # second end is a no-op (:571)
    # validation mode: a count that runs past the allocation is refused before launch
    with pytest.raises(MCCLError, match="runs past its allocation"):
        K.hip_reduce_op_view(a.data_ptr(), a.data_ptr(), F32, 1 << 24, SUM)


# ---- bit-exact parity with the oracle ------------------------------------------

SIZES = (1, 7, 8, 9, 1023, 4096, 8191, 8192, 8193, 65537, 300001)


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("op", [SUM, AVG, PRODUCT, MIN, MAX])
def test_reduce_bit_exact(K, U, dtype, op):
    rng = np.random.default_rng(1000 + 10 * dtype + op)
    for n in SIZES:
        a = U.rand_values(rng, n, dtype, specials=True)
        b = U.rand_values(rng, n, dtype, specials=True)
        if op in (MIN, MAX):  # NaN operands: parity unpinned in the reference; keep them out
            fa = a if dtype == F32 else (orc.decode_bf16(a) if dtype == BF16 else a.view(np.float16))
            fb = b if dtype == F32 else (orc.decode_bf16(b) if dtype == BF16 else b.view(np.float16))
            bad = np.isnan(fa) | np.isnan(fb)
            a[bad] = 0; b[bad] = 0
        want = a.copy(); orc.reduce(want, b, dtype, op)
        d, s = U.to_dev(a, dtype), U.to_dev(b, dtype)
        K.hip_reduce_op(d, s, op); K.hip_sync()
        if dtype == F16:  # half NaN payloads are hardware-defined: compare NaN-ness
            g = U.bits(d); nan = np.isnan(want.view(np.float16))
            assert np.array_equal(g[~nan], want[~nan]) and np.all(np.isnan(g.view(np.float16)[nan]))
        else:
            U.assert_same_bits(d, want, dtype, f"reduce dtype={dtype} op={op} n={n}")


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_misaligned_views_bit_exact(K, U, dtype):
    """Element-aligned but not 16-byte aligned dst/src (the reference's
    unaligned branch, shaders.metal:170-183; reduce_scatter's narrowed views)."""
    rng = np.random.default_rng(77)
    n = 20011
    es = 4 if dtype == F32 else 2
    for off_d in (0, 1, 3, 5):
        for off_s in (0, 1, 2, 7):
            a = U.rand_values(rng, n + 16, dtype); b = U.rand_values(rng, n + 16, dtype)
            want = a.copy(); w = want[off_d:off_d + n].copy(); orc.reduce(w, b[off_s:off_s + n].copy(), dtype, SUM)
            want[off_d:off_d + n] = w
            d, s = U.to_dev(a, dtype), U.to_dev(b, dtype)
            K.hip_reduce_op_view(d.data_ptr() + off_d * es, s.data_ptr() + off_s * es, dtype, n, SUM)
            U.assert_same_bits(d, want, dtype, f"offsets {off_d},{off_s}")  # neighbours untouched too


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("world", [2, 3, 4, 5, 7, 8])
def test_scale_both_constants_bit_exact(K, U, dtype, world):
    rng = np.random.default_rng(world)
    n = 70001
    a = U.rand_values(rng, n, dtype, specials=(dtype != F16))
    for mode_o, view in ((orc.SCALE_VIEW, True), (orc.SCALE_TENSOR, False)):
        want = a.copy(); orc.scale(want, dtype, 1.0 / world, mode_o)
        d = U.to_dev(a, dtype)
        if view:
            K.hip_scale_inplace_view(d.data_ptr(), dtype, n, 1.0 / world)
        else:
            K.hip_scale_inplace(d, 1.0 / world); K.hip_sync()
        U.assert_same_bits(d, want, dtype, f"scale 1/{world} mode {mode_o}")
    b = U.rand_values(rng, n, dtype)
    want = a.copy(); orc.accumulate_scale(want, b, dtype, 1.0 / world)
    d = U.to_dev(a, dtype)
    K.hip_accumulate_and_scale(d, U.to_dev(b, dtype), 1.0 / world); K.hip_sync()
    if dtype == F16:
        assert np.array_equal(U.bits(d), want)
    else:
        U.assert_same_bits(d, want, dtype, "accumulate_scale")


def test_bf16_view_and_tensor_constants_differ_for_thirds(K, U):
    a = orc.encode_bf16(np.full(64, 3.0, np.float32))
    d = U.to_dev(a, BF16); K.hip_scale_inplace_view(d.data_ptr(), BF16, 64, 1 / 3)
    e = U.to_dev(a, BF16); K.hip_scale_inplace(e, 1 / 3); K.hip_sync()
    assert U.bits(d)[0] == 0x3F7F and U.bits(e)[0] == 0x3F80  # 3*0.33203125 vs 3*0.333984375


# ---- codec -----------------------------------------------------------------------

def test_codec_specials_and_round_trip(K, U):
    import test_oracle_codec as T
    x = np.array(list(T.SPECIALS.keys()), dtype=np.uint32).view(np.float32)
    e = K.encode_bf16(U.to_dev(x, F32)); K.hip_sync()
    got = U.bits(e)
    assert [int(v) for v in got] == list(T.SPECIALS.values())
    h = np.arange(65536, dtype=np.uint16)
    f = K.decode_bf16(U.to_dev(h, BF16)); K.hip_sync()
    assert np.array_equal(U.bits(f), h.astype(np.uint32) << 16)           # all 65536 decodes
    back = K.encode_bf16(f); K.hip_sync()
    nan = (h & 0x7FFF) > 0x7F80
    assert np.array_equal(U.bits(back)[~nan], h[~nan]) and np.all(U.bits(back)[nan] == 0x7FC0)


def test_encode_exhaustive_2_32(K, U):
    """All 2^32 fp32 patterns: the HIP encode against torch's device cast (the
    library the reference itself calls) everywhere, and against the CPU oracle
    on every 64th block."""
    blk = 1 << 26
    base = torch.arange(blk, dtype=torch.int64, device="cuda")
    for i in range((1 << 32) // blk):
        u = (base + i * blk).to(torch.int32) if i * blk < (1 << 31) else (base + i * blk - (1 << 32)).to(torch.int32)
        x = u.view(torch.float32)
        got = K.encode_bf16(x); K.hip_sync()
        ref = x.to(torch.bfloat16)
        nan = torch.isnan(x)
        assert torch.equal(got.view(torch.int16)[~nan], ref.view(torch.int16)[~nan]), i
        assert bool((got.view(torch.int16)[nan] == 0x7FC0).all()), i
        if i % 8 == 0:
            sub = x[::64].contiguous()
            want = orc.encode_bf16(sub.cpu().numpy(), threads=8)
            g = K.encode_bf16(sub); K.hip_sync()
            assert np.array_equal(U.bits(g), want), i


def test_encode_decode_large_ragged(K, U):
    rng = np.random.default_rng(5)
    for n in (1, 9, 8191, 1_000_003):
        x = U.rand_values(rng, n, F32, scale=1e-3, specials=True)
        e = K.encode_bf16(U.to_dev(x, F32)); K.hip_sync()
        assert np.array_equal(U.bits(e), orc.encode_bf16(x))
        d = K.decode_bf16(e); K.hip_sync()
        assert np.array_equal(U.bits(d), orc.decode_bf16(orc.encode_bf16(x)).view(np.uint32))
