"""The allocation-free batched fold (mcclx_fold_batched_noalloc) against
mcclx_fold_batched, through the C ABI: same plans, same segments, results
compared bit for bit -- on two calls in a row, the second with a smaller input,
because every call on a GPU shares one static descriptor table that keeps the
previous call's contents."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    from mccl_amd import _lib as L, kernels as K
    import gpu_util as U
    K.hip_kernels_init(0)
    return L, K, U


def _fold(L, q, plan, segs, noalloc):
    arr = (L.Seg * len(segs))(*segs)
    fn = L.lib().mcclx_fold_batched_noalloc if noalloc else L.lib().mcclx_fold_batched
    L.check(fn(q.handle, C.byref(plan), arr, len(segs)))


def _case(L, K, U, rng, nseg, counts, dtype, k, io, scale):
    """Builds inputs, runs both entry points, returns (got, want) bit patterns per segment."""
    tdt = {orc.F32: torch.float32, orc.BF16: torch.bfloat16}
    out_dt = torch.float32 if (dtype == orc.F32 or io != L.IO_PURE) else tdt[dtype]
    plan = K.make_plan(dtype, k, io=io, scale_mode=L.SCALE_VIEW if scale else L.SCALE_NONE, scale=scale or 0.0)
    ins, outs_a, outs_b, segs_a, segs_b = [], [], [], [], []
    for s in range(nseg):
        n = int(counts[s])
        ops = []
        for j in range(k):
            f32 = dtype == orc.F32 or (io == L.IO_OWN_FIRST_F32 and j == 0)
            ops.append(U.to_dev(U.rand_values(rng, max(n, 1), orc.F32 if f32 else dtype, scale=1e-2, specials=True),
                                orc.F32 if f32 else dtype))
        ins.append(ops)
        a = torch.zeros(max(n, 1), dtype=out_dt, device="cuda")
        b = torch.zeros(max(n, 1), dtype=out_dt, device="cuda")
        outs_a.append(a)
        outs_b.append(b)
        segs_a.append(K.make_seg(a.data_ptr(), 0, [t.data_ptr() for t in ops], n))
        segs_b.append(K.make_seg(b.data_ptr(), 0, [t.data_ptr() for t in ops], n))
    q = K._q(None)
    torch.cuda.synchronize()
    _fold(L, q, plan, segs_a, noalloc=False)
    _fold(L, q, plan, segs_b, noalloc=True)
    K.hip_sync()
    return [(U.bits(b), U.bits(a)) for a, b in zip(outs_a, outs_b)], ins


def _same(pairs, what):
    for s, (got, want) in enumerate(pairs):
        assert np.array_equal(got, want), f"{what}: segment {s} differs from mcclx_fold_batched"


def test_noalloc_matches_fold_batched_twice_in_a_row(env):
    L, K, U = env
    rng = np.random.default_rng(77)
    # call 1: 600 ragged segments (some empty), bf16 wire fold with an fp32 owner and the x(1/3) scale
    counts = rng.integers(0, 9000, size=600)
    counts[[3, 77, 599]] = 0
    counts[5] = 70001
    pairs, ins = _case(L, K, U, rng, 600, counts, orc.BF16, 3, L.IO_OWN_FIRST_F32, 1.0 / 3)
    _same(pairs, "600 ragged segments")
    # ... and against the oracle on a few segments, so that both being wrong alike cannot pass
    for s in (0, 5, 311):
        own = ins[s][0].cpu().numpy()
        peers = [U.bits(t) for t in ins[s][1:]]
        n = int(counts[s])
        want = orc.wire_fold_chunk(np.ascontiguousarray(own[:n]), [np.ascontiguousarray(p[:n]) for p in peers],
                                   scale_by=1.0 / 3)
        assert np.array_equal(pairs[s][0][:n], want.view(np.uint32)), f"segment {s} differs from the oracle"
    # call 2, smaller: 40 uniform segments of another plan; the table still holds call 1's descriptors behind them
    pairs, _ = _case(L, K, U, rng, 40, np.full(40, 16384), orc.F32, 3, L.IO_PURE, None)
    _same(pairs, "40 uniform segments after 600")
    # call 3: few enough to travel in the kernel arguments
    pairs, _ = _case(L, K, U, rng, 7, rng.integers(1, 5000, size=7), orc.BF16, 2, L.IO_PURE, None)
    _same(pairs, "7 segments by value")


def test_noalloc_limit_and_launch_only(env):
    L, K, U = env
    q = K._q(None)
    plan = K.make_plan(orc.F32, 2)
    t = torch.ones(64, device="cuda")
    segs = [K.make_seg(t.data_ptr(), 0, [t.data_ptr(), t.data_ptr()], 0)] * (L.NOALLOC_MAX_SEGS + 1)
    arr = (L.Seg * len(segs))(*segs)
    rc = L.lib().mcclx_fold_batched_noalloc(q.handle, C.byref(plan), arr, len(segs))
    assert rc == L.ERR_INVALID and "at most 1024" in L.last_error()
    # the largest launch it accepts, with device memory use unchanged across the call
    n = L.NOALLOC_MAX_SEGS
    a = torch.arange(n * 8, dtype=torch.float32, device="cuda")
    b = torch.ones(n * 8, dtype=torch.float32, device="cuda")
    out = torch.empty_like(a)
    segs = [K.make_seg(out.data_ptr() + 32 * i, 0, [a.data_ptr() + 32 * i, b.data_ptr() + 32 * i], 8) for i in range(n)]
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _fold(L, q, plan, segs, noalloc=True)
    K.hip_sync()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(out, a + 1)


def test_noalloc_ragged_launch_of_few_segments_takes_the_static_table(env):
    """Up to 32 segments travel in the kernel arguments only when they are of similar length:
    one long segment among many short ones would launch (longest x segments) blocks, most of
    them idle, so such a launch goes through the static table like mcclx_fold_batched's goes
    through an uploaded one (same rule).  Seen from outside: more than one kernel launch."""
    L, K, U = env
    rng = np.random.default_rng(5)
    q = K._q(None)
    counts = np.array([900_000] + [300] * 19)
    before = q.launch_count()
    pairs, _ = _case(L, K, U, rng, 20, counts, orc.F32, 2, L.IO_PURE, None)
    _same(pairs, "20 ragged segments")
    # fold_batched: 1 launch (its table is uploaded by a copy); noalloc: writer launch(es) + the fold
    assert q.launch_count() - before >= 3
    before = q.launch_count()
    pairs, _ = _case(L, K, U, rng, 20, np.full(20, 5000), orc.F32, 2, L.IO_PURE, None)
    _same(pairs, "20 even segments")
    assert q.launch_count() - before == 2, "even segments travel by value: one launch per entry point"


def test_noalloc_concurrent_entry_from_two_contexts_is_refused_not_interleaved(env):
    """Every context on a GPU shares the one static table.  A call that enters while another
    thread's call is still writing descriptors is refused with MCCLX_ERR_STATE instead of
    interleaving its writer launches with the other's.  Two threads, each with a context of its
    own, hammer the entry point with the SAME segments (what overlaps on the device -- which
    the host cannot see, and which the entry point leaves to its callers -- then writes the
    same bytes): every call returns OK or ERR_STATE, and the result is right throughout."""
    import threading
    L, K, U = env
    nseg, n, rounds = 40, 257, 150
    plan = K.make_plan(orc.F32, 2)
    a = torch.arange(nseg * n, dtype=torch.float32, device="cuda")
    b = torch.full((nseg * n,), 2.0, device="cuda")
    out = torch.zeros_like(a)
    segs = [K.make_seg(out.data_ptr() + 4 * n * i, 0, [a.data_ptr() + 4 * n * i, b.data_ptr() + 4 * n * i], n)
            for i in range(nseg)]
    arr = (L.Seg * nseg)(*segs)
    torch.cuda.synchronize()
    errs, codes = [], [set(), set()]
    start = threading.Barrier(2)

    def worker(w):
        try:
            torch.cuda.set_device(0)
            q = K.ReduceQueue(0)
            start.wait()
            for _ in range(rounds):
                rc = L.lib().mcclx_fold_batched_noalloc(q.handle, C.byref(plan), arr, nseg)
                codes[w].add(rc)
                if rc == L.ERR_STATE:
                    assert "static descriptor table" in L.last_error()
            q.drain()
            q.close()
        except BaseException as e:  # noqa: BLE001
            errs.append(e)

    ts = [threading.Thread(target=worker, args=(w,)) for w in range(2)]
    [t.start() for t in ts]
    [t.join(300) for t in ts]
    assert not errs, errs
    assert codes[0] | codes[1] <= {L.OK, L.ERR_STATE} and L.OK in codes[0] and L.OK in codes[1]
    torch.cuda.synchronize()
    assert torch.equal(out, a + 2.0)
