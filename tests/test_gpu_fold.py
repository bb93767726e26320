"""GPU parity of the fused multi-input fold (mcclx_fold / mcclx_fold_batched)
against chains of the oracle's binary kernels: every k, io mode, topology and
accumulator mode, by-value and table launches, ragged and misaligned segments."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from mccl_amd import kernels
    kernels.hip_kernels_init(0)
    return kernels


@pytest.fixture(scope="module")
def U():
    import gpu_util
    return gpu_util


def L():
    from mccl_amd import _lib
    return _lib


def oracle_fold(ins, dtype, binomial=False, scale=None, scale_mode=orc.SCALE_VIEW):
    """Left fold (or binomial tree) of same-dtype operands with the oracle's binary kernel."""
    v = [x.copy() for x in ins]
    k = len(v)
    if not binomial:
        for j in range(1, k):
            orc.reduce(v[0], v[j], dtype, SUM)
    else:
        mask = 1
        while mask < k:
            for r in range(0, k - mask, 2 * mask):
                orc.reduce(v[r], v[r + mask], dtype, SUM)
            mask <<= 1
    if scale is not None:
        orc.scale(v[0], dtype, scale, scale_mode)
    return v[0]


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("binomial", [False, True])
def test_fold_pure(K, U, k, dtype, binomial):
    rng = np.random.default_rng(10 * k + dtype)
    n = 50021
    ins = [U.rand_values(rng, n, dtype, scale=10.0 ** rng.integers(-2, 3), specials=True) for _ in range(k)]
    for scale, mode_o, mode_x in ((None, 0, L().SCALE_NONE), (1.0 / 3, orc.SCALE_VIEW, L().SCALE_VIEW),
                                  (1.0 / 3, orc.SCALE_TENSOR, L().SCALE_TENSOR)):
        want = oracle_fold(ins, dtype, binomial, scale, mode_o)
        d = [U.to_dev(x, dtype) for x in ins]
        out = torch.empty_like(d[0])
        plan = K.make_plan(dtype, k, topo=L().TOPO_BINOMIAL if binomial else L().TOPO_FOLD,
                           scale_mode=mode_x, scale=scale or 0.0)
        K._q(None).fold(plan, [K.make_seg(out.data_ptr(), 0, [t.data_ptr() for t in d], n)])
        K.hip_sync()
        U.assert_same_bits(out, want, dtype, f"k={k} dtype={dtype} binomial={binomial} scale={scale}")


@pytest.mark.parametrize("k", [2, 3, 5, 8])
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("binomial", [False, True])
def test_fold_other_ops_and_fp16(K, U, k, dtype, binomial):
    """MIN / MAX / PRODUCT (and fp16 SUM) as one k-input pass == k-1 binary kernels."""
    rng = np.random.default_rng(1000 + 10 * k + dtype)
    n = 30011
    ops = [orc.MIN, orc.MAX, orc.PRODUCT] + ([SUM] if dtype == F16 else [])
    for op in ops:
        ins = [U.rand_values(rng, n, dtype, scale=1.0) for _ in range(k)]
        v = [x.copy() for x in ins]
        if not binomial:
            for j in range(1, k):
                orc.reduce(v[0], v[j], dtype, op)
        else:
            mask = 1
            while mask < k:
                for r in range(0, k - mask, 2 * mask):
                    orc.reduce(v[r], v[r + mask], dtype, op)
                mask <<= 1
        d = [U.to_dev(x, dtype) for x in ins]
        out = torch.empty_like(d[0])
        plan = K.make_plan(dtype, k, op=op, topo=L().TOPO_BINOMIAL if binomial else L().TOPO_FOLD)
        K._q(None).fold(plan, [K.make_seg(out.data_ptr(), 0, [t.data_ptr() for t in d], n)])
        K.hip_sync()
        if dtype == F16:
            assert np.array_equal(U.bits(out), v[0]), (op, k)
        else:
            U.assert_same_bits(out, v[0], dtype, f"op={op} k={k} dtype={dtype} binomial={binomial}")


@pytest.mark.parametrize("k", range(1, 9))
@pytest.mark.parametrize("io", ["out_f32", "own_first", "own_last"])
@pytest.mark.parametrize("binomial", [False, True])
def test_fold_wire_modes(K, U, k, io, binomial):
    """fp32 tensors with the bf16 wire codec in one pass == encode, k-1 binary
    bf16 reduces, scale, decode."""
    if io == "own_last" and binomial:
        pytest.skip("the tree's owner is operand 0")
    rng = np.random.default_rng(100 * k + len(io))
    n = 30011
    own = U.rand_values(rng, n, F32, scale=1e-3, specials=True)
    peers = [U.rand_values(rng, n, BF16, scale=1e-3, specials=True) for _ in range(k - (io != "out_f32"))]
    if io == "out_f32":
        ops = peers
    elif io == "own_first":
        ops = [orc.encode_bf16(own)] + peers
    else:
        ops = peers + [orc.encode_bf16(own)]
    for scale in (None, 1.0 / 3):
        wbits = oracle_fold(ops, BF16, binomial, scale, orc.SCALE_VIEW)
        want = orc.decode_bf16(wbits)
        dp = [U.to_dev(p, BF16) for p in peers]
        down = U.to_dev(own, F32)
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        wire = torch.empty(n, dtype=torch.bfloat16, device="cuda")
        if io == "out_f32":
            ptrs, code = [t.data_ptr() for t in dp], L().IO_OUT_F32
        elif io == "own_first":
            ptrs, code = [down.data_ptr()] + [t.data_ptr() for t in dp], L().IO_OWN_FIRST_F32
        else:
            ptrs, code = [t.data_ptr() for t in dp] + [down.data_ptr()], L().IO_OWN_LAST_F32
        plan = K.make_plan(BF16, k, io=code, topo=L().TOPO_BINOMIAL if binomial else L().TOPO_FOLD,
                           scale_mode=L().SCALE_VIEW if scale else L().SCALE_NONE, scale=scale or 0.0)
        K._q(None).fold(plan, [K.make_seg(out.data_ptr(), wire.data_ptr(), ptrs, n)])
        K.hip_sync()
        U.assert_same_bits(out, want, F32, f"k={k} io={io} binomial={binomial} scale={scale}")
        assert np.array_equal(U.bits(wire), wbits)
        # in place: the fp32 output over the own operand
        if io != "out_f32":
            K._q(None).fold(plan, [K.make_seg(down.data_ptr(), 0, ptrs, n)])
            K.hip_sync()
            U.assert_same_bits(down, want, F32, "in place")


@pytest.mark.parametrize("k", [2, 3, 8])
def test_fold_f32_accumulate_mode_is_labelled_variant(K, U, k):
    """MCCLX_ACC_F32 (not the reference): one rounding at the end."""
    rng = np.random.default_rng(k)
    n = 40000
    ins = [U.rand_values(rng, n, BF16, scale=1e-2) for _ in range(k)]
    acc = orc.decode_bf16(ins[0]).copy()
    for x in ins[1:]:
        acc = acc + orc.decode_bf16(x)
    want = orc.encode_bf16(acc)
    d = [U.to_dev(x, BF16) for x in ins]
    out = torch.empty_like(d[0])
    plan = K.make_plan(BF16, k, acc=L().ACC_F32)
    K._q(None).fold(plan, [K.make_seg(out.data_ptr(), 0, [t.data_ptr() for t in d], n)])
    K.hip_sync()
    assert np.array_equal(U.bits(out), want)
    if k == 8:  # and it really differs from the per-step rounding somewhere
        assert not np.array_equal(want, oracle_fold(ins, BF16))


@pytest.mark.parametrize("nseg", [2, 8, 9, 100])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_fold_batched_ragged_segments(K, U, nseg, dtype):
    """By-value launch (<= 8 segments) and descriptor-table launch (> 8), with
    empty, tiny, tail-only and misaligned segments."""
    rng = np.random.default_rng(nseg)
    k = 3
    es = 4 if dtype == F32 else 2
    sizes = [int(s) for s in rng.choice([0, 1, 5, 8, 9, 1000, 8192, 8200, 20000, 70001], nseg)]
    sizes[0] = 70001
    total = sum(sizes) + 16 * nseg
    bufs = [U.rand_values(rng, total, dtype) for _ in range(k)]
    dbufs = [U.to_dev(b, dtype) for b in bufs]
    out_np = U.rand_values(rng, total, dtype)
    dout = U.to_dev(out_np, dtype)
    want = out_np.copy()
    segs = []
    off = 0
    for i, n in enumerate(sizes):
        shift = [int(x) for x in rng.integers(0, 8, k + 1)]  # element misalignment per pointer
        ins = [np.ascontiguousarray(bufs[j][off + shift[j]: off + shift[j] + n]) for j in range(k)]
        if n:
            want[off + shift[k]: off + shift[k] + n] = oracle_fold(ins, dtype)
        segs.append(K.make_seg(dout.data_ptr() + (off + shift[k]) * es, 0,
                               [dbufs[j].data_ptr() + (off + shift[j]) * es for j in range(k)], n))
        off += n + 16
    K._q(None).fold(K.make_plan(dtype, k), segs)
    K.hip_sync()
    U.assert_same_bits(dout, want, dtype, f"batched nseg={nseg}")  # gaps between segments untouched


def test_fold_uniform_table_4096_messages(K, U):
    """The tree path's shape: many equal 64 KiB messages, k = 3, one launch."""
    rng = np.random.default_rng(4)
    nmsg, n = 512, 16384
    ins = [rng.uniform(-1, 1, nmsg * n).astype(np.float32) for _ in range(3)]
    d = [U.to_dev(x, F32) for x in ins]
    segs = [K.make_seg(d[0].data_ptr() + m * n * 4, 0, [t.data_ptr() + m * n * 4 for t in d], n)
            for m in range(nmsg)]
    K._q(None).fold(K.make_plan(F32, 3), segs)
    K.hip_sync()
    want = (ins[0] + ins[1]) + ins[2]
    U.assert_same_bits(d[0], want, F32, "uniform table")


def test_plan_validation(K):
    from mccl_amd import MCCLError
    a = torch.ones(64, device="cuda")
    seg = K.make_seg(a.data_ptr(), 0, [a.data_ptr()] * 8, 64)
    for plan, msg in ((K.make_plan(F32, 0), "plan.k=0"), (K.make_plan(F32, 9), "plan.k=9"),
                      (K.make_plan(F32, 2, io=L().IO_OUT_F32), "bf16 wire dtype"),
                      (K.make_plan(BF16, 3, op=orc.MIN, io=L().IO_OUT_F32), "PURE, STEP"),
                      (K.make_plan(BF16, 3, op=orc.MAX, acc=L().ACC_F32), "PURE, STEP"),
                      (K.make_plan(F16, 3, acc=L().ACC_F32), "fp16 folds round after every step"),
                      (K.make_plan(F32, 2, op=6), "Unsupported ReduceOp: 6"),
                      (K.make_plan(7, 2), "No kernel for dtype")):
        with pytest.raises(MCCLError, match=msg):
            K._q(None).fold(plan, [seg])
    with pytest.raises(MCCLError, match="in\\[1\\] is null"):
        K._q(None).fold(K.make_plan(F32, 2), [K.make_seg(a.data_ptr(), 0, [a.data_ptr()], 64)])
    with pytest.raises(MCCLError, match="has no output"):
        K._q(None).fold(K.make_plan(F32, 1), [K.make_seg(0, 0, [a.data_ptr()], 64)])
    with pytest.raises(MCCLError, match="not element aligned"):
        K._q(None).fold(K.make_plan(F32, 1), [K.make_seg(a.data_ptr() + 2, 0, [a.data_ptr()], 8)])
