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
@pytest.mark.parametrize("io", ["out_f32", "own_first", "own_last", "all_f32"])
@pytest.mark.parametrize("binomial", [False, True])
def test_fold_wire_modes(K, U, k, io, binomial):
    """fp32 tensors with the bf16 wire codec in one pass == encode, k-1 binary
    bf16 reduces, scale, decode."""
    if io == "own_last" and binomial:
        pytest.skip("the tree's owner is operand 0")
    rng = np.random.default_rng(100 * k + len(io))
    n = 30011
    own = U.rand_values(rng, n, F32, scale=1e-3, specials=True)
    if io == "all_f32":  # every operand an fp32 tensor, each encoded in registers
        peers32 = [U.rand_values(rng, n, F32, scale=1e-3, specials=True) for _ in range(k - 1)]
        peers = [orc.encode_bf16(p) for p in peers32]
    else:
        peers = [U.rand_values(rng, n, BF16, scale=1e-3, specials=True) for _ in range(k - (io != "out_f32"))]
    if io == "out_f32":
        ops = peers
    elif io in ("own_first", "all_f32"):
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
        if io == "all_f32":
            dp = [U.to_dev(p, F32) for p in peers32]
            ptrs, code = [down.data_ptr()] + [t.data_ptr() for t in dp], L().IO_ALL_F32
        elif io == "out_f32":
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


@pytest.mark.parametrize("nseg", [2, 8, 9, 32, 33, 100])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_fold_batched_ragged_segments(K, U, nseg, dtype):
    """By-value launch (<= 32 segments) and descriptor-table launch (> 32), with
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


@pytest.mark.parametrize("io", ["encode", "decode", "own_first", "own_last"])
def test_wire_modes_at_odd_element_offsets(K, U, io):
    """Chunk starts are only element aligned (C2's second chunk starts 8 B past a
    16-byte boundary in fp32 and 12 B in bf16): every stream gets its own skew."""
    rng = np.random.default_rng(len(io))
    n = 20011
    for skew in ((0, 0, 0, 0), (1, 0, 0, 0), (0, 1, 2, 3), (3, 5, 7, 1), (2, 2, 2, 2), (31, 63, 1, 33)):
        own = U.rand_values(rng, n + 64, F32, scale=1e-2, specials=True)
        p1 = U.rand_values(rng, n + 64, BF16, scale=1e-2, specials=True)
        p2 = U.rand_values(rng, n + 64, BF16, scale=1e-2, specials=True)
        d_own, d1, d2 = U.to_dev(own, F32), U.to_dev(p1, BF16), U.to_dev(p2, BF16)
        o32 = torch.zeros(n + 64, dtype=torch.float32, device="cuda")
        o16 = torch.zeros(n + 64, dtype=torch.bfloat16, device="cuda")
        so, s1, s2, sd = skew
        a = own[so:so + n]
        if io == "encode":
            plan = K.make_plan(BF16, 1, io=L().IO_OWN_FIRST_F32)
            seg = K.make_seg(0, o16.data_ptr() + 2 * sd, [d_own.data_ptr() + 4 * so], n)
            want16 = orc.encode_bf16(a); want32 = None
        elif io == "decode":
            plan = K.make_plan(BF16, 1, io=L().IO_OUT_F32)
            seg = K.make_seg(o32.data_ptr() + 4 * sd, 0, [d1.data_ptr() + 2 * s1], n)
            want32 = orc.decode_bf16(p1[s1:s1 + n]); want16 = None
        else:
            first = io == "own_first"
            plan = K.make_plan(BF16, 3, io=L().IO_OWN_FIRST_F32 if first else L().IO_OWN_LAST_F32,
                               scale_mode=L().SCALE_VIEW, scale=1 / 3)
            peers = [d1.data_ptr() + 2 * s1, d2.data_ptr() + 2 * s2]
            ins = [d_own.data_ptr() + 4 * so] + peers if first else peers + [d_own.data_ptr() + 4 * so]
            seg = K.make_seg(o32.data_ptr() + 4 * sd, o16.data_ptr() + 2 * sd, ins, n)
            want32, want16 = orc.wire_fold_chunk(np.ascontiguousarray(a),
                                                 [np.ascontiguousarray(p1[s1:s1 + n]), np.ascontiguousarray(p2[s2:s2 + n])],
                                                 own_last=not first, scale_by=1 / 3, want_wire=True)
        K._q(None).fold(plan, [seg])
        K.hip_sync()
        if want32 is not None:
            full = np.zeros(n + 64, np.float32); full[sd:sd + n] = want32
            U.assert_same_bits(o32, full, F32, f"{io} skew {skew}")          # nothing outside the range is touched
        if want16 is not None:
            full = np.zeros(n + 64, np.uint16); full[sd:sd + n] = want16
            assert np.array_equal(U.bits(o16), full), (io, skew)


def test_many_table_launches_in_flight(K, U):
    """More descriptor-table launches than staging slots, queued without draining,
    with tables of growing size: slots are reused only after their launch finished."""
    rng = np.random.default_rng(99)
    q = K._q(None)
    n = 3001
    nseg_list = [33, 36, 40, 33, 300, 47, 1000, 34, 64, 33, 2000, 35]
    total = max(nseg_list) * n
    a = U.rand_values(rng, total, F32); b = U.rand_values(rng, total, F32)
    da, db = U.to_dev(a, F32), U.to_dev(b, F32)
    outs, wants = [], []
    plan = K.make_plan(F32, 2)
    K.hip_sync()
    for nseg in nseg_list:
        o = torch.zeros(total, device="cuda")
        outs.append(o)
        torch.cuda.synchronize()
        segs = [K.make_seg(o.data_ptr() + 4 * n * i, 0, [da.data_ptr() + 4 * n * i, db.data_ptr() + 4 * n * i], n)
                for i in range(nseg)]
        q.fold(plan, segs)                       # no drain between launches
        w = np.zeros(total, np.float32); w[:nseg * n] = (a + b)[:nseg * n]
        wants.append(w)
    q.drain()
    for o, w in zip(outs, wants):
        U.assert_same_bits(o, w, F32, "table launch")


def test_two_queues_from_two_threads(K, U):
    """Contexts are independent: two reduce queues driven from two host threads."""
    import threading
    rng = np.random.default_rng(5)
    n = 1_000_003
    data = [(U.rand_values(rng, n, BF16), U.rand_values(rng, n, BF16)) for _ in range(2)]
    res = [None, None]

    def work(i):
        q = K.ReduceQueue(0)
        a, b = U.to_dev(data[i][0], BF16), U.to_dev(data[i][1], BF16)
        torch.cuda.synchronize()
        for _ in range(20):
            K.hip_reduce_op_view(a.data_ptr(), b.data_ptr(), BF16, n, SUM, queue=q, drain=False)
        q.drain()
        res[i] = U.bits(a)
        q.close()

    ts = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    [t.start() for t in ts]
    [t.join(60) for t in ts]
    for i in range(2):
        want = data[i][0].copy()
        for _ in range(20):
            orc.reduce(want, data[i][1], BF16, SUM, threads=4)
        assert np.array_equal(res[i], want)


def test_one_long_segment_among_many_short_ones(K, U):
    """A launch of 9..32 segments travels by value unless its segments differ so much in
    length that most of the (longest x segments) grid would idle; either way the result
    is the same."""
    rng = np.random.default_rng(31)
    for nseg, long_n in ((12, 3_000_001), (32, 1_000_003), (6, 2_000_003)):
        counts = [long_n] + [int(c) for c in rng.integers(1, 300, nseg - 1)]
        total = sum(counts) + 16 * nseg
        a = U.rand_values(rng, total, BF16, scale=1e-2); b = U.rand_values(rng, total, BF16, scale=1e-2)
        da, db = U.to_dev(a, BF16), U.to_dev(b, BF16)
        out = torch.zeros(total, dtype=torch.bfloat16, device="cuda")
        want = np.zeros(total, np.uint16)
        segs, off = [], 0
        for n in counts:
            segs.append(K.make_seg(out.data_ptr() + 2 * off, 0, [da.data_ptr() + 2 * off, db.data_ptr() + 2 * off], n))
            x = a[off:off + n].copy(); orc.reduce(x, b[off:off + n].copy(), BF16, SUM)
            want[off:off + n] = x
            off += n + 16
        K._q(None).fold(K.make_plan(BF16, 2), segs)
        K.hip_sync()
        assert np.array_equal(U.bits(out), want), (nseg, long_n)


@pytest.mark.parametrize("k", [2, 3, 5, 8])
@pytest.mark.parametrize("binomial", [False, True])
def test_fold_bf16_nan_operands_of_any_payload(K, U, k, binomial):
    """The packet path rounds between operands without making NaNs canonical and fixes
    them once at the end.  Pinned here: operands holding every kind of bf16 NaN (quiet and
    signalling, either sign, payload in any bit), infinities of both signs (whose sum is a
    NaN born mid-fold) and zeros give what canonicalising after every step gives -- the
    oracle's result, bit for bit -- for every op, at every operand position."""
    rng = np.random.default_rng(4000 + k)
    n = 20011
    nans = np.array([0x7FC0, 0xFFC0, 0x7F81, 0xFF81, 0x7FFF, 0xFFFF, 0x7FA0, 0x7F80, 0xFF80, 0x0000, 0x8000, 0x3F80],
                    dtype=np.uint16)
    for op in (SUM, orc.PRODUCT, orc.MIN, orc.MAX):
        ins = []
        for _ in range(k):
            x = orc.encode_bf16((rng.standard_normal(n)).astype(np.float32))
            idx = rng.random(n) < 0.15
            x[idx] = nans[rng.integers(0, nans.size, int(idx.sum()))]
            ins.append(x)
        for scale in (None, 1.0 / 3):
            if scale is not None and op != SUM:
                continue
            v = [x.copy() for x in ins]
            if not binomial:
                for j in range(1, k):
                    orc.reduce(v[0], v[j], BF16, op)
            else:
                mask = 1
                while mask < k:
                    for r in range(0, k - mask, 2 * mask):
                        orc.reduce(v[r], v[r + mask], BF16, op)
                    mask <<= 1
            if scale is not None:
                orc.scale(v[0], BF16, scale, orc.SCALE_VIEW)
            d = [U.to_dev(x, BF16) for x in ins]
            out = torch.empty_like(d[0])
            plan = K.make_plan(BF16, k, op=op, topo=L().TOPO_BINOMIAL if binomial else L().TOPO_FOLD,
                               scale_mode=L().SCALE_VIEW if scale else L().SCALE_NONE, scale=scale or 0.0)
            K._q(None).fold(plan, [K.make_seg(out.data_ptr(), 0, [t.data_ptr() for t in d], n)])
            K.hip_sync()
            got = U.bits(out)
            assert np.array_equal(got, v[0]), f"op {op} k {k} binomial {binomial} scale {scale}: " \
                f"{int((got != v[0]).sum())} differ, first at {int(np.flatnonzero(got != v[0])[0])}"
    # one operand, no scale: bits move untouched (a decode keeps a NaN's payload)
    x = nans.repeat(700)
    d = U.to_dev(x, BF16)
    out = torch.empty(x.size, dtype=torch.float32, device="cuda")
    K._q(None).fold(K.make_plan(BF16, 1, io=L().IO_OUT_F32), [K.make_seg(out.data_ptr(), 0, [d.data_ptr()], x.size)])
    K.hip_sync()
    assert np.array_equal(U.bits(out), x.astype(np.uint32) << 16)


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("op", [SUM, orc.PRODUCT])
def test_scale_after_a_fold_keeps_the_sign_of_zero(K, U, dtype, op):
    """-0 * (1/N) is -0.  Sums of negative zeros and products that underflow produce
    negative zeros in bulk; the scale that follows (the AVG of AllreduceAlgos.cpp:88-91,
    the fused accumulate_scale kernels, shaders.metal:447-551) must hand them on."""
    rng = np.random.default_rng(77 + dtype + op)
    n = 20011
    for k in (1, 2, 3, 6):
        ins = [U.rand_values(rng, n, dtype, scale=1e-3) for _ in range(k)]
        zeros = rng.choice(n, size=n // 4, replace=False)
        for x in ins:                                  # a quarter of the elements: zeros of either sign
            sign = rng.random(zeros.size) < 0.8
            if dtype == F32:
                x[zeros] = np.where(sign, np.float32(-0.0), np.float32(0.0))
            else:
                x[zeros] = np.where(sign, np.uint16(0x8000), np.uint16(0))
        for scale, mode_o, mode_x in ((0.5, orc.SCALE_VIEW, L().SCALE_VIEW), (1.0 / 3, orc.SCALE_TENSOR, L().SCALE_TENSOR)):
            v = [x.copy() for x in ins]
            for j in range(1, k):
                orc.reduce(v[0], v[j], dtype, op)
            orc.scale(v[0], dtype, scale, mode_o)
            assert (U.np_bits(v[0]) == (0x80000000 if dtype == F32 else 0x8000)).sum() > n // 100, "the case needs -0 results"
            d = [U.to_dev(x, dtype) for x in ins]
            out = torch.empty_like(d[0])
            plan = K.make_plan(dtype, k, op=op, scale_mode=mode_x, scale=scale)
            K._q(None).fold(plan, [K.make_seg(out.data_ptr(), 0, [t.data_ptr() for t in d], n)])
            K.hip_sync()
            if dtype == F16:
                assert np.array_equal(U.bits(out), v[0]), (op, k, scale)
            else:
                U.assert_same_bits(out, v[0], dtype, f"dtype {dtype} op {op} k {k} scale {scale}")


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16", "own_first", "own_last", "all_f32"])
def test_fan_out_writes_the_result_to_every_destination(K, U, kind):
    """MCCLX_PLAN_FANOUT(n): what `out` receives also goes to in[k .. k+n-1] -- the owner of a
    chunk handing the reduced values to every other rank (AllreduceAlgos.cpp:77-86,185-200)
    without a second pass.  Every k and n that fit a segment, both topologies, misaligned
    destinations, a destination that is one of the operands, by-value and table launches."""
    rng = np.random.default_rng(len(kind) * 7)
    dtype = {"f32": F32, "bf16": BF16, "f16": F16}.get(kind, BF16)
    io = {"own_first": L().IO_OWN_FIRST_F32, "own_last": L().IO_OWN_LAST_F32,
          "all_f32": L().IO_ALL_F32}.get(kind, L().IO_PURE)
    odt = F32 if (dtype == F32 or io != L().IO_PURE) else dtype
    es = {F32: 4, F16: 2, BF16: 2}
    for k in range(2, 8):
        for fan in range(1, 9 - k):
            for binomial in ((False, True) if (k >= 4 and kind != "own_last") else (False,)):
                nseg = int(rng.choice([1, 3, 40]))
                segs, checks, keep = [], [], []
                for s in range(nseg):
                    n = int(rng.integers(1, 30000 if nseg < 10 else 3000))
                    ins, ptrs, dev = [], [], []
                    for j in range(k):
                        f32_in = (dtype == F32 or kind == "all_f32" or (kind == "own_first" and j == 0) or
                                  (kind == "own_last" and j == k - 1))
                        dt = F32 if f32_in else dtype
                        off = int(rng.integers(0, 5))
                        a = U.rand_values(rng, n + off + 4, dt, scale=1e-2, specials=(dt != F16))
                        t = U.to_dev(a, dt)
                        ins.append((np.ascontiguousarray(a[off:off + n]), dt))
                        dev.append(t)
                        ptrs.append(t.data_ptr() + off * es[dt])
                    ops = [orc.encode_bf16(a) if (dt == F32 and dtype == BF16) else a.copy() for a, dt in ins]
                    res = oracle_fold(ops, dtype, binomial and k >= 4, 1.0 / 3, orc.SCALE_VIEW)
                    want = orc.decode_bf16(res) if (odt == F32 and dtype == BF16) else res
                    outs = []
                    for f in range(fan + 1):
                        off = int(rng.integers(0, 5))
                        t = torch.full((n + off + 4,), 3.0, dtype=U.TORCH_DT[odt], device="cuda")
                        outs.append((t, off))
                    # one destination may be an operand of the output's form (reduced in place)
                    same_form = [j for j, (a, dt) in enumerate(ins) if dt == odt]
                    if same_form and rng.integers(0, 2):
                        j = int(rng.choice(same_form))
                        outs[-1] = (dev[j], (ptrs[j] - dev[j].data_ptr()) // es[odt])
                    dest = [t.data_ptr() + off * es[odt] for t, off in outs]
                    segs.append(K.make_seg(dest[0], 0, ptrs + dest[1:], n))
                    checks.append((outs, n, want))
                    keep.append(dev)
                plan = K.make_plan(dtype, k, io=io, topo=L().TOPO_BINOMIAL if binomial else L().TOPO_FOLD,
                                   scale_mode=L().SCALE_VIEW, scale=1.0 / 3, fanout=fan)
                torch.cuda.synchronize()
                K._q(None).fold(plan, segs)
                K.hip_sync()
                for outs, n, want in checks:
                    for f, (t, off) in enumerate(outs):
                        what = f"{kind} k={k} fan={fan} binomial={binomial} nseg={nseg} destination {f}"
                        if odt == F16:
                            assert np.array_equal(U.bits(t[off:off + n]), want), what
                        else:
                            U.assert_same_bits(t[off:off + n], want, odt, what)
                        if t.numel() == n + off + 4 and float(t[:1].float().cpu()) == 3.0:   # a fresh buffer: guards intact
                            assert torch.all(t[:off].float() == 3.0) and torch.all(t[off + n:].float() == 3.0), what


def test_fan_out_validation(K):
    q = K._q(None)
    t = torch.zeros(64, device="cuda")
    seg = lambda k, fan: [K.make_seg(t.data_ptr(), 0, [t.data_ptr()] * min(8, k + fan), 16)]
    for plan, fan, k, frag in ((K.make_plan(F32, 5, fanout=4), 4, 5, "k + fan <= 8"),
                               (K.make_plan(F32, 3, op=orc.MAX, fanout=2), 2, 3, "needs a sum"),
                               (K.make_plan(BF16, 3, acc=L().ACC_F32, fanout=2), 2, 3, "per-step rounding"),
                               (K.make_plan(BF16, 2, io=L().IO_OUT_F32, fanout=1), 1, 2, "fan-out"),
                               (K.make_plan(F32, 1, fanout=1), 1, 1, "fan-out")):
        with pytest.raises(Exception) as e:
            q.fold(plan, seg(k, fan))
        assert frag in str(e.value), str(e.value)
    with pytest.raises(Exception) as e:                                 # a destination is missing
        q.fold(K.make_plan(F32, 2, fanout=2), [K.make_seg(t.data_ptr(), 0, [t.data_ptr()] * 3, 16)])
    assert "fan-out destination in[3] is null" in str(e.value)
    with pytest.raises(Exception) as e:                                 # fan-out without `out`
        q.fold(K.make_plan(BF16, 2, fanout=1), [K.make_seg(0, t.data_ptr(), [t.data_ptr()] * 3, 16)])
    assert "fan-out needs `out`" in str(e.value)
    # a destination may BE an operand; one that overlaps an operand at another offset would be
    # read by some lanes after others have written it (checked under MCCLX_VALIDATE, which the tests set)
    a, b = torch.zeros(64, device="cuda"), torch.zeros(64, device="cuda")
    q.fold(K.make_plan(F32, 2, fanout=1), [K.make_seg(a.data_ptr(), 0, [a.data_ptr(), b.data_ptr(), b.data_ptr()], 16)])
    with pytest.raises(Exception) as e:
        q.fold(K.make_plan(F32, 2, fanout=1),
               [K.make_seg(a.data_ptr(), 0, [a.data_ptr(), b.data_ptr(), b.data_ptr() + 8], 16)])
    assert "overlaps operand in[1]" in str(e.value)
    K.hip_sync()
