"""The c10d surface on the GPU: world-size-1 semantics (the reference's
tests/test_smoke.py) and N ranks as N threads of one process sharing the GPU,
checked bit for bit against the oracle's replay of the reference."""
import datetime
import gc
import os
import threading

import numpy as np
import pytest
import torch
import torch.distributed as dist

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG, MIN, MAX, PRODUCT, RING, TREE, BUTTERFLY

pytestmark = pytest.mark.gpu

TIMEOUT = datetime.timedelta(seconds=20)
OPS = {SUM: dist.ReduceOp.SUM, AVG: dist.ReduceOp.AVG, MIN: dist.ReduceOp.MIN, MAX: dist.ReduceOp.MAX,
       PRODUCT: dist.ReduceOp.PRODUCT}


@pytest.fixture(scope="module")
def CX():
    import mccl_amd
    from mccl_amd import _C
    return _C


@pytest.fixture(scope="module")
def U():
    import gpu_util
    return gpu_util


def run_ranks(CX, world, fn):
    """Create `world` backends over one HashStore, run fn(rank, pg) on one thread per rank."""
    store = dist.HashStore()
    out, errs = [None] * world, [None] * world

    def body(r):
        try:
            torch.cuda.set_device(0)
            pg = CX._create_process_group_mccl(store, r, world, TIMEOUT)
            out[r] = fn(r, pg)
        except BaseException as e:  # noqa: BLE001
            errs[r] = e

    ts = [threading.Thread(target=body, args=(r,)) for r in range(world)]
    for t in ts:
        t.start()
    for t in ts:
        t.join(60)
    assert not any(t.is_alive() for t in ts), "a rank thread hung"
    return out, errs


# ---- world size 1: tests/test_smoke.py:29-41 -------------------------------------

def test_world_one_is_a_no_op_with_real_work_objects(CX):
    pg = CX._create_process_group_mccl(dist.HashStore(), 0, 1, TIMEOUT)
    assert pg.name() == "mccl" and pg.rank() == 0 and pg.size() == 1
    t = torch.arange(16, dtype=torch.float32, device="cuda")
    ref = t.clone()
    w = pg.allreduce([t])
    assert w.is_completed() and w.is_success() and w.wait()
    assert torch.equal(t, ref)
    assert torch.equal(w.get_future().wait()[0], ref)
    out = torch.zeros(16, device="cuda")
    assert pg._allgather_base(out, t).wait() and torch.equal(out, ref)
    out.zero_()
    assert pg._reduce_scatter_base(out, t).wait() and torch.equal(out, ref)
    assert pg.barrier().wait()
    assert pg.broadcast([t]).wait()


def test_init_process_group_world_one(CX):
    if dist.is_initialized():
        dist.destroy_process_group()
    dist.init_process_group(backend="mccl", store=dist.HashStore(), rank=0, world_size=1,
                            timeout=TIMEOUT)
    try:
        assert dist.get_backend() == "mccl"
        t = torch.full((33,), 3.0, device="cuda")
        dist.all_reduce(t)
        assert torch.equal(t, torch.full((33,), 3.0, device="cuda"))
        o = torch.empty(33, device="cuda")
        dist.all_gather_into_tensor(o, t)
        assert torch.equal(o, t)
    finally:
        dist.destroy_process_group()


def test_distributed_data_parallel_over_the_backend_world_one(CX):
    """torch's DistributedDataParallel on top of backend "mccl" (the reference's
    tests/test_ddp.py:70-95 shape: a Linear layer, SGD, a few steps): parameter
    broadcast, bucket allreduce through Work/Future, and the same weights as plain training."""
    from torch.nn.parallel import DistributedDataParallel as DDP
    if dist.is_initialized():
        dist.destroy_process_group()
    dist.init_process_group(backend="mccl", store=dist.HashStore(), rank=0, world_size=1, timeout=TIMEOUT)
    try:
        torch.manual_seed(42)
        plain = torch.nn.Linear(16, 1, bias=False).cuda()
        wrapped = DDP(torch.nn.Linear(16, 1, bias=False).cuda())
        wrapped.module.load_state_dict(plain.state_dict())
        opt_a = torch.optim.SGD(plain.parameters(), lr=0.01)
        opt_b = torch.optim.SGD(wrapped.parameters(), lr=0.01)
        x = torch.randn(32, 16, device="cuda")
        y = torch.randn(32, 1, device="cuda")
        for _ in range(5):
            for model, opt in ((plain, opt_a), (wrapped, opt_b)):
                opt.zero_grad()
                torch.nn.functional.mse_loss(model(x), y).backward()
                opt.step()
        assert torch.equal(plain.weight, wrapped.module.weight)
    finally:
        wrapped = opt_b = model = opt = None   # a DDP module sits in reference cycles: collected here, while its group exists
        gc.collect()
        dist.destroy_process_group()


# ---- N ranks in one process -----------------------------------------------------------

@pytest.mark.parametrize("world", [2, 3, 4])
@pytest.mark.parametrize("algo_name,algo", [("ring", RING), ("butterfly", BUTTERFLY), ("tree", TREE), (None, None)])
@pytest.mark.parametrize("wire", [False, True])
def test_allreduce_threads_bit_exact(CX, U, monkeypatch, world, algo_name, algo, wire):
    if algo_name:
        monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", algo_name)
    else:
        monkeypatch.delenv("MCCL_ALLREDUCE_ALGO", raising=False)
    monkeypatch.delenv("MCCL_TREE_BELOW", raising=False)
    if wire:
        monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    else:
        monkeypatch.delenv("MCCL_WIRE_DTYPE", raising=False)
    rng = np.random.default_rng(world * 10 + (algo or 7))
    cases = [(F32, SUM, 40009), (F32, AVG, 1237), (BF16, SUM, 70001), (F32, SUM, 100003)]
    xs = {i: [U.rand_values(rng, n, dt, specials=True) for _ in range(world)] for i, (dt, op, n) in enumerate(cases)}

    def fn(r, pg):
        res, algos = [], []
        for i, (dt, op, n) in enumerate(cases):
            t = U.to_dev(xs[i][r], dt)
            o = dist.AllreduceOptions()
            o.reduceOp = OPS[op]
            w = pg.allreduce([t], o)
            assert w.is_completed() and w.wait()
            res.append(t)
            algos.append(CX._last_algo(pg))
        return res, algos

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for i, (dt, op, n) in enumerate(cases):
        want = [x.copy() for x in xs[i]]
        rc, used = orc.pg_allreduce(want, dt, op, wire_bf16=wire, env_algo=algo_name)
        assert rc == 0
        for r in range(world):
            assert out[r][1][i] == used, "algorithm selection differs from the reference's"
            U.assert_same_bits(out[r][0][i], want[r], dt, f"case {i} rank {r}")


def test_allreduce_min_max_product_fp16_and_tensor_lists(CX, U, monkeypatch):
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "butterfly")
    monkeypatch.delenv("MCCL_WIRE_DTYPE", raising=False)
    world = 3
    rng = np.random.default_rng(5)
    a = [U.rand_values(rng, 5003, F32) for _ in range(world)]
    b = [U.rand_values(rng, 777, F16) for _ in range(world)]

    def fn(r, pg):
        res = {}
        for op in (MIN, MAX, PRODUCT):
            t1, t2 = U.to_dev(a[r], F32), U.to_dev(b[r], F16)
            o = dist.AllreduceOptions(); o.reduceOp = OPS[op]
            pg.allreduce([t1, t2], o).wait()          # a list of tensors is handled one after another
            res[op] = (t1, t2)
        return res

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for op in (MIN, MAX, PRODUCT):
        wa = [x.copy() for x in a]; orc.allreduce(BUTTERFLY, wa, F32, op)
        wb = [x.copy() for x in b]; orc.allreduce(BUTTERFLY, wb, F16, op)
        for r in range(world):
            U.assert_same_bits(out[r][op][0], wa[r], F32, f"op {op}")
            assert np.array_equal(U.bits(out[r][op][1]), wb[r])


@pytest.mark.parametrize("world", [2, 3, 8])
def test_reduce_scatter_allgather_broadcast_barrier_threads(CX, U, world):
    rng = np.random.default_rng(world)
    CH = 4099
    ins = [U.rand_values(rng, CH * world, BF16) for _ in range(world)]
    f32 = [U.rand_values(rng, CH * world, F32) for _ in range(world)]

    def fn(r, pg):
        res = {}
        din = U.to_dev(ins[r], BF16)
        out = torch.empty(CH, dtype=torch.bfloat16, device="cuda")
        o = dist.ReduceScatterOptions(); o.reduceOp = dist.ReduceOp.AVG
        w = pg._reduce_scatter_base(out, din, o)          # asynchronous: a pending Work comes back
        assert w.wait()
        res["rs_base"] = out
        # list form, fp32, in place over the rank's own share
        full = U.to_dev(f32[r], F32)
        shares = [full.narrow(0, p * CH, CH) for p in range(world)]
        o2 = dist.ReduceScatterOptions(); o2.reduceOp = dist.ReduceOp.SUM
        assert pg.reduce_scatter([shares[r]], [shares], o2).wait()
        res["rs_list"] = shares[r].clone()
        # allgather, both forms
        g = torch.empty(CH * world, dtype=torch.bfloat16, device="cuda")
        assert pg._allgather_base(g, out).wait()
        res["ag_base"] = g
        outs = [torch.empty(CH, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
        fut = pg.allgather([outs], [out]).get_future()
        fut.wait()
        res["ag_list"] = torch.cat(outs)
        # broadcast from the last rank, then a barrier
        b = torch.full((1001,), float(r), device="cuda")
        bo = dist.BroadcastOptions(); bo.rootRank = world - 1
        assert pg.broadcast([b], bo).wait()
        res["bcast"] = b
        assert pg.barrier().wait()
        return res

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    want = [np.zeros(CH, dtype=np.uint16) for _ in range(world)]
    orc.reduce_scatter(want, ins, BF16, AVG)
    want32 = [np.zeros(CH, dtype=np.float32) for _ in range(world)]
    orc.reduce_scatter(want32, f32, F32, SUM)
    cat = np.concatenate(want)
    for r in range(world):
        U.assert_same_bits(out[r]["rs_base"], want[r], BF16, "reduce_scatter_base AVG")
        U.assert_same_bits(out[r]["rs_list"], want32[r], F32, "reduce_scatter list SUM")
        assert np.array_equal(U.bits(out[r]["ag_base"]), cat)
        assert np.array_equal(U.bits(out[r]["ag_list"]), cat)
        assert torch.equal(out[r]["bcast"], torch.full((1001,), float(world - 1), device="cuda"))


def test_error_paths(CX, U):
    world = 2

    def fn(r, pg):
        msgs = {}
        try:
            pg.allreduce([torch.ones(8)])                       # CPU tensor (test_mps_native.py:343-356)
        except RuntimeError as e:
            msgs["cpu"] = str(e)
        try:
            o = dist.AllreduceOptions(); o.reduceOp = dist.ReduceOp.BAND
            pg.allreduce([torch.ones(8, device="cuda")], o)
        except RuntimeError as e:
            msgs["op"] = str(e)
        try:
            pg.allreduce([torch.ones(8, device="cuda", dtype=torch.float64)])
        except RuntimeError as e:
            msgs["dtype"] = str(e)
        try:
            pg.allreduce([torch.ones(4, 4, device="cuda").t()])
        except RuntimeError as e:
            msgs["contig"] = str(e)
        # sizes that differ between ranks: every rank gets the leader's error
        try:
            pg.allreduce([torch.ones(8 + r, device="cuda")])
        except RuntimeError as e:
            msgs["mismatch"] = str(e)
        # asynchronous collectives report through the Work (ProcessGroupMCCL.cpp:60-68)
        w = pg._reduce_scatter_base(torch.ones(3, device="cuda"), torch.ones(8, device="cuda"))
        try:
            w.wait()
        except RuntimeError as e:
            msgs["rs_size"] = str(e)
        assert w.is_completed() and not w.is_success()
        try:
            pg.send([torch.ones(3, device="cuda")], r, 0)          # to itself (ProcessGroupMCCL.cpp:616-617)
        except RuntimeError as e:
            msgs["send"] = str(e)
        # the group still works afterwards
        t = torch.full((5,), float(r + 1), device="cuda")
        pg.allreduce([t]).wait()
        msgs["after"] = t.cpu().tolist()
        return msgs

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for m in out:
        assert "GPU-only; got CPU tensor" in m["cpu"]
        assert "Unsupported ReduceOp" in m["op"]
        assert "No HIP kernel for dtype" in m["dtype"]
        assert "must be contiguous" in m["contig"]
        assert "different size or dtype" in m["mismatch"]
        assert "input size != output * world" in m["rs_size"]
        assert "send: bad dst_rank" in m["send"]
        assert all(s.startswith("[MCCL] ") for k, s in m.items() if k != "after")
        assert m["after"] == [3.0] * 5


def test_divergent_argument_error_fails_every_rank_at_once(CX):
    """One rank passes a tensor its own checks refuse (CPU, non-contiguous, empty): that rank still
    goes to the meeting point, so its peers fail with its message instead of waiting for the
    group's timeout (20 s here)."""
    import time
    world = 3
    bad = {0: lambda: torch.ones(8), 1: lambda: torch.ones(4, 4, device="cuda").t(),
           2: lambda: torch.ones(0, device="cuda")}

    def fn(r, pg):
        msgs, took = [], []
        for culprit in range(world):
            t = bad[culprit]() if r == culprit else torch.ones(8, device="cuda")
            t0 = time.monotonic()
            try:
                pg.allreduce([t])
                msgs.append("no error")
            except RuntimeError as e:
                msgs.append(str(e))
            took.append(time.monotonic() - t0)
        ok = torch.full((5,), float(r + 1), device="cuda")
        pg.allreduce([ok]).wait()               # the group is still usable
        return msgs, took, ok.cpu().tolist()

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for r, (msgs, took, ok) in enumerate(out):
        assert "GPU-only; got CPU tensor" in msgs[0] and "must be contiguous" in msgs[1] and "empty tensors" in msgs[2]
        for culprit in range(world):
            if r != culprit:
                assert f"(raised on rank {culprit})" in msgs[culprit]
        assert max(took) < 5.0, took
        assert ok == [6.0] * 5


@pytest.mark.parametrize("spin_us", [None, "0", "1"])
def test_synchronous_allreduce_returns_with_the_result_whichever_way_it_drains(CX, U, monkeypatch, spin_us):
    """The synchronous allreduce leaves its drain when a word written behind the launch arrives in
    pinned host memory (the default), after a blocking drain (MCCL_DRAIN_SPIN_US=0), or after a
    blocking drain because the word did not come within the time allowed (1 us: a 25 MiB bucket
    takes longer).  Either way the tensors hold the oracle's bits when it returns: read by a kernel
    on the rank's stream, and by a copy to the host, at once."""
    if spin_us is None:
        monkeypatch.delenv("MCCL_DRAIN_SPIN_US", raising=False)
    else:
        monkeypatch.setenv("MCCL_DRAIN_SPIN_US", spin_us)
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "butterfly")
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    monkeypatch.delenv("MCCL_ALLREDUCE_ASYNC", raising=False)
    world = 3
    sizes = [6_553_600, 33, 1_000_003, 6_553_600, 70_001]
    rng = np.random.default_rng(41)
    xs = [[(rng.standard_normal(n) * 1e-3).astype(np.float32) for _ in range(world)] for n in sizes]

    def fn(r, pg):
        got = []
        for x in xs:
            t = U.to_dev(x[r], F32)
            torch.cuda.current_stream().synchronize()
            o = dist.AllreduceOptions(); o.reduceOp = dist.ReduceOp.AVG
            w = pg.allreduce([t], o)
            assert w.is_completed() and w.is_success()
            doubled = t * 2                       # a kernel on the rank's stream, straight away
            host = t.cpu()                        # and a copy to the host
            got.append((host, doubled.cpu()))
        return got

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for i, n in enumerate(sizes):
        want = [x.copy() for x in xs[i]]
        rc, used = orc.pg_allreduce(want, F32, AVG, wire_bf16=True, env_algo="butterfly", threads=orc.max_threads())
        assert rc == 0 and used == BUTTERFLY
        for r in range(world):
            U.assert_same_bits(out[r][i][0], want[r], F32, f"bucket {i} rank {r}")
            assert torch.equal(out[r][i][1], out[r][i][0] * 2)


@pytest.mark.parametrize("queues,direct", [(1, True), (2, True), (2, False)])
def test_allreduce_event_based_completion_and_bucket_coalescing(CX, U, monkeypatch, queues, direct):
    """MCCL_ALLREDUCE_ASYNC=1: allreduce returns a pending Work, wait() orders the caller's
    stream after the reduce queue without blocking the host, the Future settles from the
    completion ticket, and buckets issued while two earlier launches are still in flight go
    out together (one launch per phase for all of them).  With two queues (the default) the
    buckets alternate between them, up to two launches in flight on each.  Results are the oracle's,
    bit for bit.  By default the fold reads the ranks' fp32 tensors itself (one kernel per launch);
    MCCL_DIRECT=0 goes through bf16 copies (an encode in front of the fold)."""
    monkeypatch.setenv("MCCL_ALLREDUCE_ASYNC", "1")
    if direct:
        monkeypatch.delenv("MCCL_DIRECT", raising=False)
    else:
        monkeypatch.setenv("MCCL_DIRECT", "0")
    monkeypatch.setenv("MCCL_ASYNC_QUEUES", str(queues))
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "butterfly")
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    monkeypatch.setenv("MCCL_COALESCE_BELOW", "0")   # the queue mechanics alone (small buckets gather: see the next test)
    world = 3
    sizes = [6_553_600, 1_000_003, 70_001, 1_000_003, 33, 4097, 250_000]
    rng = np.random.default_rng(31)
    xs = [[(rng.standard_normal(n) * 1e-3).astype(np.float32) for _ in range(world)] for n in sizes]

    def fn(r, pg):
        ts = [U.to_dev(x[r], F32) for x in xs]
        big = torch.empty(1 << 30, dtype=torch.uint8, device="cuda") if r == 0 else None
        torch.cuda.current_stream().synchronize()
        before = (CX._async_stats(pg), CX._launch_count(pg))
        busy = None
        if r == 0:
            # the rank's stream is still busy (a backward pass would be): some 70 ms of copies in
            # front of the first bucket, so the later buckets find the reduce queue occupied
            for _ in range(300):
                big[: 1 << 29].copy_(big[1 << 29:])
            busy = torch.cuda.Event()
            busy.record()
        works = []
        for t in ts:
            o = dist.AllreduceOptions(); o.reduceOp = dist.ReduceOp.AVG
            works.append(pg.allreduce([t], o))
        pending_at_return = [not w.is_completed() for w in works]
        still_busy = busy is not None and not busy.query()   # else this thread was held up for longer than the copies ran
        for w in works:
            assert w.wait()                       # stream-ordered: does not block until the device is done
        doubled = [t * 2 for t in ts]             # torch work on this rank's stream, behind the reduction
        futs = [w.get_future().wait() for w in works]
        torch.cuda.current_stream().synchronize()
        assert all(w.is_completed() and w.is_success() for w in works)
        assert all(f[0].data_ptr() == t.data_ptr() for f, t in zip(futs, ts))
        after = (CX._async_stats(pg), CX._launch_count(pg))
        return ts, doubled, pending_at_return, before, after, still_busy

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for i, n in enumerate(sizes):
        want = [x.copy() for x in xs[i]]
        rc, used = orc.pg_allreduce(want, F32, AVG, wire_bf16=True, env_algo="butterfly", threads=orc.max_threads())
        assert rc == 0 and used == BUTTERFLY
        for r in range(world):
            U.assert_same_bits(out[r][0][i], want[r], F32, f"bucket {i} rank {r}")
            assert torch.equal(out[r][1][i], out[r][0][i] * 2)
    (l0, b0), k0 = out[0][3]
    (l1, b1), k1 = out[0][4]
    assert b1 - b0 == len(sizes)
    # with every bucket issued before the first launch has finished (the usual course, rank 0's
    # stream being busy for some 70 ms): one queue -- two buckets at once, the five behind them
    # together, 3 launches; two queues -- two at once on either queue, behind them buckets 4 and
    # 6 together and bucket 5, 6 launches.  A rank thread that is held up may split a group.
    assert (3 if queues == 1 else 6) <= l1 - l0 <= len(sizes)
    if out[0][5]:   # every bucket was issued while the first launch still waited for rank 0's stream
        assert l1 - l0 < len(sizes), "buckets were coalesced"
    assert k1 - k0 == (1 if direct else 2) * (l1 - l0), \
        "a launch of several buckets is one fold that also hands out the result (behind one encode without MCCL_DIRECT), once"
    assert all(all(out[r][2]) for r in range(world)), "a Work was complete when allreduce returned"


@pytest.mark.parametrize("below,launches", [(None, 2), ("0", None)])
def test_small_event_based_buckets_gather_behind_a_launch_in_flight(CX, U, monkeypatch, below, launches):
    """Buckets under MCCL_COALESCE_BELOW (8 MiB by default) take the main queue and are parked
    while ANY launch of it is in flight; what has gathered goes out as one launch.  Eight 1 MiB
    buckets issued behind a busy stream: the first goes out at once, the other seven together --
    two launches, against at least three with the gathering off (two launches in flight on each
    of two queues, the rest behind them).  Results are the oracle's, bit for bit, either way."""
    monkeypatch.setenv("MCCL_ALLREDUCE_ASYNC", "1")
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "butterfly")
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    if below is None:
        monkeypatch.delenv("MCCL_COALESCE_BELOW", raising=False)
    else:
        monkeypatch.setenv("MCCL_COALESCE_BELOW", below)
    world, nb, n = 3, 8, (1 << 20) // 4
    rng = np.random.default_rng(77)
    xs = [[(rng.standard_normal(n + 3 * i) * 1e-3).astype(np.float32) for _ in range(world)] for i in range(nb)]

    def fn(r, pg):
        ts = [U.to_dev(x[r], F32) for x in xs]
        big = torch.empty(1 << 30, dtype=torch.uint8, device="cuda") if r == 0 else None
        torch.cuda.current_stream().synchronize()
        before = CX._async_stats(pg)
        busy = None
        if r == 0:
            for _ in range(300):   # some 70 ms of copies: the first launch waits for this stream on the device
                big[: 1 << 29].copy_(big[1 << 29:])
            busy = torch.cuda.Event()
            busy.record()
        o = dist.AllreduceOptions(); o.reduceOp = dist.ReduceOp.AVG
        works = [pg.allreduce([t], o) for t in ts]
        still_busy = busy is not None and not busy.query()   # else this thread was held up for longer than the copies ran
        for w in works:
            assert w.wait(datetime.timedelta(seconds=60))   # with a timeout: blocks the host until settled
            assert w.is_completed() and w.is_success()
        torch.cuda.current_stream().synchronize()
        return ts, before, CX._async_stats(pg), still_busy

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for i in range(nb):
        want = [x.copy() for x in xs[i]]
        rc, used = orc.pg_allreduce(want, F32, AVG, wire_bf16=True, env_algo="butterfly", threads=orc.max_threads())
        assert rc == 0 and used == BUTTERFLY
        for r in range(world):
            U.assert_same_bits(out[r][0][i], want[r], F32, f"bucket {i} rank {r}")
    (l0, b0), (l1, b1) = out[0][1], out[0][2]
    assert b1 - b0 == nb
    if launches is not None and out[0][3]:
        assert l1 - l0 == launches, "the seven buckets behind the first went out together"
    else:
        assert 3 <= l1 - l0 <= nb


@pytest.mark.parametrize("queues", [1, 2])
def test_event_based_allreduces_that_share_memory_run_in_program_order(CX, U, monkeypatch, queues):
    """Event-based launches alternate between two queues and may overlap on the device; calls
    that touch the same tensor must still take effect one after another, also across other
    collectives issued in between, with nobody waiting on a Work until the end."""
    monkeypatch.setenv("MCCL_ALLREDUCE_ASYNC", "1")
    monkeypatch.setenv("MCCL_ASYNC_QUEUES", str(queues))
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "ring")
    monkeypatch.delenv("MCCL_WIRE_DTYPE", raising=False)
    world, n = 3, 700_001
    rng = np.random.default_rng(5)
    a = [(rng.standard_normal(n) * 1e-2).astype(np.float32) for _ in range(world)]
    b = [(rng.standard_normal(n) * 1e-2).astype(np.float32) for _ in range(world)]

    def fn(r, pg):
        ta, tb = U.to_dev(a[r], F32), U.to_dev(b[r], F32)
        gathered = torch.empty(world * n, dtype=torch.float32, device="cuda")
        big = torch.empty(1 << 28, dtype=torch.uint8, device="cuda") if r == 0 else None
        torch.cuda.current_stream().synchronize()
        if r == 0:                                   # keep the queues busy, so that launches pile up
            for _ in range(20):
                big[: 1 << 27].copy_(big[1 << 27:])
        works = []
        smax = dist.AllreduceOptions(); smax.reduceOp = dist.ReduceOp.MAX
        works.append(pg.allreduce([ta]))             # a = sum(a)
        works.append(pg.allreduce([tb], smax))       # b = max(b)                 (other queue, independent)
        works.append(pg.allreduce([ta]))             # a = 3 * sum(a)             (other queue than the first)
        works.append(pg.allreduce([ta, tb]))         # a = 9 * sum(a), b = 3 * max(b)
        bo = dist.BroadcastOptions(); bo.rootRank = 1
        works.append(pg.broadcast([tb], bo))         # on the main queue, behind all of the above
        works.append(pg.allreduce([tb]))             # b = 3 * (3 * max(b))
        works.append(pg._allgather_base(gathered, ta))
        for w in works:
            w.wait()
        torch.cuda.current_stream().synchronize()
        return ta, tb, gathered

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    wa = [x.copy() for x in a]
    wb = [x.copy() for x in b]
    for _ in range(3):
        assert orc.pg_allreduce(wa, F32, SUM, env_algo="ring")[0] == 0
    assert orc.pg_allreduce(wb, F32, MAX, env_algo="ring")[0] == 0
    assert orc.pg_allreduce(wb, F32, SUM, env_algo="ring")[0] == 0
    wb = [wb[1].copy() for _ in range(world)]
    assert orc.pg_allreduce(wb, F32, SUM, env_algo="ring")[0] == 0
    for r in range(world):
        U.assert_same_bits(out[r][0], wa[r], F32, f"a on rank {r}")
        U.assert_same_bits(out[r][1], wb[r], F32, f"b on rank {r}")
        U.assert_same_bits(out[r][2], np.concatenate(wa), F32, f"gathered on rank {r}")


@pytest.mark.parametrize("transport", ["host", "staged"])
@pytest.mark.parametrize("algo_name,algo", [("ring", RING), ("butterfly", BUTTERFLY), ("tree", TREE)])
def test_allreduce_over_the_host_wire_bit_exact(CX, U, monkeypatch, transport, algo_name, algo):
    """MCCL_WIRE=host|staged: every rank runs its own half of the collective and every chunk
    crosses the byte transport (send / recv on host memory) -- encoded into pinned memory and
    read by the owner's fold through the device alias, or staged through the pinned pool.
    Same bits as the oracle's replay of the reference, for every schedule, op and dtype."""
    monkeypatch.setenv("MCCL_WIRE", transport)
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", algo_name)
    monkeypatch.delenv("MCCL_ALLREDUCE_ASYNC", raising=False)
    rng = np.random.default_rng(70 + algo)
    cases = [(F32, SUM, 40009, True), (F32, AVG, 70001, True), (F32, SUM, 1237, False), (BF16, AVG, 5003, False),
             (F16, SUM, 777, False), (F32, MAX, 4099, True), (F32, MIN, 4099, False), (BF16, PRODUCT, 333, False),
             (F32, SUM, 5, True)]
    for world in (2, 3, 4):
        xs = {i: [U.rand_values(rng, n, dt, scale=1e-2, specials=(dt != F16)) for _ in range(world)]
              for i, (dt, op, n, wire) in enumerate(cases)}

        def fn(r, pg):
            res = []
            for i, (dt, op, n, wire) in enumerate(cases):
                if wire:
                    os.environ["MCCL_WIRE_DTYPE"] = "bf16"     # every rank sets the same value before the call
                else:
                    os.environ.pop("MCCL_WIRE_DTYPE", None)
                t = U.to_dev(xs[i][r], dt)
                o = dist.AllreduceOptions(); o.reduceOp = OPS[op]
                w = pg.allreduce([t], o)
                assert w.is_completed() and w.wait()
                res.append(t)
                pg.barrier().wait()                            # nobody changes the knob while a peer still reads it
            return res, CX._wire_stats(pg)

        out, errs = run_ranks(CX, world, fn)
        os.environ.pop("MCCL_WIRE_DTYPE", None)
        assert errs == [None] * world, errs
        for i, (dt, op, n, wire) in enumerate(cases):
            want = [x.copy() for x in xs[i]]
            rc, used = orc.pg_allreduce(want, dt, op, wire_bf16=wire, env_algo=algo_name)
            assert rc == 0
            for r in range(world):
                if dt == F16:
                    assert np.array_equal(U.bits(out[r][0][i]), want[r]), (world, i, r)
                else:
                    U.assert_same_bits(out[r][0][i], want[r], dt, f"{transport} {algo_name} world {world} case {i} rank {r}")
        assert all(st[0] == len(cases) for _, st in out)      # every call went over the wire


@pytest.mark.parametrize("transport", ["host", "staged"])
def test_host_wire_tensor_list_of_unequal_sizes(CX, U, monkeypatch, transport):
    """A list goes over the wire one tensor after another with no meeting in between
    (ProcessGroupMCCL.cpp:122-168): a rank may start on the next tensor while a peer still
    takes delivery of the last one, and consecutive tensors lay their chunks out differently."""
    monkeypatch.setenv("MCCL_WIRE", transport)
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "ring")
    rng = np.random.default_rng(91)
    world, sizes = 3, [300007, 11, 65536, 3, 200001, 4097]
    for op in (SUM, MAX):
        xs = [[U.rand_values(rng, n, F32, scale=1e-2) for n in sizes] for _ in range(world)]

        def fn(r, pg):
            ts = [U.to_dev(x, F32) for x in xs[r]]
            o = dist.AllreduceOptions(); o.reduceOp = OPS[op]
            for _ in range(3):                      # the same buffers again: results are idempotent only for MAX
                pg.allreduce([t.clone() for t in ts], o).wait()
            pg.allreduce(ts, o).wait()
            return ts

        out, errs = run_ranks(CX, world, fn)
        assert errs == [None] * world, errs
        for i, n in enumerate(sizes):
            want = [xs[r][i].copy() for r in range(world)]
            rc, _ = orc.pg_allreduce(want, F32, op, wire_bf16=True, env_algo="ring")
            assert rc == 0
            for r in range(world):
                U.assert_same_bits(out[r][i], want[r], F32, f"{transport} op {op} tensor {i} rank {r}")


def test_host_wire_error_paths(CX, monkeypatch):
    monkeypatch.setenv("MCCL_WIRE", "host")
    world = 2

    def fn(r, pg):
        msgs = {}
        try:
            pg.allreduce([torch.ones(8 + r, device="cuda")])          # sizes differ: found at the meeting point
        except RuntimeError as e:
            msgs["mismatch"] = str(e)
        os.environ["MCCL_WIRE"] = "carrier-pigeon"
        pg.barrier().wait()
        try:
            pg.allreduce([torch.ones(8, device="cuda")])
        except RuntimeError as e:
            msgs["knob"] = str(e)
        pg.barrier().wait()
        os.environ["MCCL_WIRE"] = "host"
        pg.barrier().wait()
        t = torch.full((5,), float(r + 1), device="cuda")
        pg.allreduce([t]).wait()
        msgs["after"] = t.cpu().tolist()
        return msgs

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for m in out:
        assert "different size or dtype" in m["mismatch"]
        assert "is not one of device, host, staged" in m["knob"]
        assert m["after"] == [3.0] * 5


def test_reference_collective_vectors(CX):
    """tests/collectives/test_allreduce.py:11-28 (128 x value rank+1, all ops, f32/f16/bf16)
    and tests/test_process_group_local.py:162-207 (3 ranks: SUM = 6, AVG = 2)."""
    world = 3
    os.environ.pop("MCCL_ALLREDUCE_ALGO", None)
    os.environ.pop("MCCL_WIRE_DTYPE", None)

    def fn(r, pg):
        res = {}
        for dt in (torch.float32, torch.float16, torch.bfloat16):
            for name, op in (("sum", dist.ReduceOp.SUM), ("avg", dist.ReduceOp.AVG), ("min", dist.ReduceOp.MIN),
                             ("max", dist.ReduceOp.MAX), ("prod", dist.ReduceOp.PRODUCT)):
                for n in (128, 1, 3, 7, 33, 997):
                    t = torch.full((n,), float(r + 1), dtype=dt, device="cuda")
                    o = dist.AllreduceOptions(); o.reduceOp = op
                    pg.allreduce([t], o).wait()
                    res[(dt, name, n)] = t.float().cpu()
        return res

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    exp = {"sum": 6.0, "avg": 2.0, "min": 1.0, "max": 3.0, "prod": 6.0}
    for m in out:
        for (dt, name, n), got in m.items():
            tol = 1e-4 if dt == torch.float32 else 1e-2            # tests/common.py:53-56
            assert torch.allclose(got, torch.full((n,), exp[name]), rtol=tol, atol=tol), (dt, name, n)


# ---- all-to-all and point-to-point: the reference's tests/collectives/test_alltoall.py
# ---- and test_p2p.py, with its values ----------------------------------------------

P2P_DTYPES = [torch.float32, torch.float16, torch.bfloat16, torch.int32, torch.int64, torch.uint8]


def seed_tensor(rank, n, dtype):
    """tests/common.py:136-147 of the reference."""
    if dtype in (torch.int8, torch.uint8):
        return torch.full((n,), (rank + 1) % 8, dtype=dtype, device="cuda")
    return torch.full((n,), rank + 1, dtype=dtype, device="cuda")


@pytest.mark.parametrize("world", [2, 3, 4])
def test_alltoall_base_even_uneven_and_in_place(CX, world):
    CH = 8

    def fn(r, pg):
        res = {}
        for dt in P2P_DTYPES:
            mk = lambda v, n: torch.full((n,), v, dtype=dt, device="cuda")
            inp = torch.cat([mk((r * 10 + p) % 120, CH) for p in range(world)])
            out = torch.empty(CH * world, dtype=dt, device="cuda")
            pg.alltoall_base(out, inp, [], []).wait()
            res[(dt, "even")] = out.cpu()
            same = inp.clone()
            pg.alltoall_base(same, same, [], []).wait()            # test_alltoall.py:19-23
            res[(dt, "in_place")] = same.cpu()
            in_sizes = [4 * (r + 1)] * world                        # test_alltoall.py:29-38
            out_sizes = [4 * (p + 1) for p in range(world)]
            inp = torch.cat([mk((r * 10 + p) % 120, in_sizes[p]) for p in range(world)])
            out = torch.empty(sum(out_sizes), dtype=dt, device="cuda")
            pg.alltoall_base(out, inp, out_sizes, in_sizes).wait()
            res[(dt, "uneven")] = out.cpu()
        # rows of a 2-d tensor: split sizes count rows
        inp = (torch.arange(world * 2 * 5, device="cuda", dtype=torch.float32) + 1000 * r).reshape(world * 2, 5)
        out = torch.empty_like(inp)
        pg.alltoall_base(out, inp, [2] * world, [2] * world).wait()
        res["rows"] = out.cpu()
        return res

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for r, res in enumerate(out):
        for dt in P2P_DTYPES:
            want = torch.cat([torch.full((CH,), (p * 10 + r) % 120, dtype=dt) for p in range(world)])
            assert torch.equal(res[(dt, "even")], want), (r, dt)
            assert torch.equal(res[(dt, "in_place")], want), (r, dt)
            want = torch.cat([torch.full((4 * (p + 1),), (p * 10 + r) % 120, dtype=dt) for p in range(world)])
            assert torch.equal(res[(dt, "uneven")], want), (r, dt)
        want = torch.cat([(torch.arange(world * 10, dtype=torch.float32) + 1000 * p).reshape(world * 2, 5)[2 * r:2 * r + 2]
                          for p in range(world)])
        assert torch.equal(res["rows"], want)


def test_alltoall_list_form_and_size_errors_reach_every_rank(CX):
    world = 3

    def fn(r, pg):
        res = {}
        ins = [torch.full((5 + p,), float(r * 100 + p), device="cuda") for p in range(world)]
        outs = [torch.empty(5 + r, device="cuda") for p in range(world)]
        pg.alltoall(outs, ins).wait()
        res["list"] = [o.cpu() for o in outs]
        # rank 1 expects more than its peers send: all ranks fail, at once, with one message
        import time
        t0 = time.time()
        out = torch.empty(8 * world + (1 if r == 1 else 0) * world, device="cuda")
        w = pg.alltoall_base(out, torch.ones(8 * world, device="cuda"), [], [])
        try:
            w.wait()
            res["err"] = None
        except RuntimeError as e:
            res["err"] = str(e)
        # a rank that fails its own argument check does not leave the others waiting
        w = pg.alltoall_base(torch.empty(9, device="cuda"), torch.ones(9 if r else 10, device="cuda"), [], [])
        try:
            w.wait()
            res["err2"] = None
        except RuntimeError as e:
            res["err2"] = str(e)
        res["secs"] = time.time() - t0
        t = torch.full((4,), float(r), device="cuda")
        pg.allreduce([t]).wait()
        res["after"] = t.cpu().tolist()
        return res

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for r, res in enumerate(out):
        for p in range(world):
            assert torch.equal(res["list"][p], torch.full((5 + r,), float(p * 100 + r)))
        assert "which expects" in res["err"] or "self chunk size mismatch" in res["err"], res["err"]
        assert "input not divisible by world" in res["err2"] and "raised on rank 0" in res["err2"], res["err2"]
        assert res["secs"] < 10                    # far below the group's 20 s timeout
        assert res["after"] == [3.0] * 4


@pytest.mark.parametrize("world", [2, 3, 4])
def test_send_recv_ring_tags_and_wildcard(CX, world):
    """test_p2p.py:8-49: even ranks send first, odd ranks receive first."""

    def fn(r, pg):
        nxt, prv = (r + 1) % world, (r - 1) % world
        res = {}
        for dt in P2P_DTYPES:
            for tag, want_tag in ((0, 0), (7, 7), (12345, 12345), (42, -1)):
                send_t = seed_tensor(r, 32, dt)
                recv_t = torch.empty(32, dtype=dt, device="cuda")
                if r % 2 == 0:
                    pg.send([send_t], nxt, tag).wait(); pg.recv([recv_t], prv, want_tag).wait()
                else:
                    pg.recv([recv_t], prv, want_tag).wait(); pg.send([send_t], nxt, tag).wait()
                res[(dt, tag)] = recv_t.cpu()
        return res

    # with an odd ring two neighbouring even ranks both send first; a send completes
    # without its receiver here, so no order of calls can deadlock
    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for r, res in enumerate(out):
        for (dt, tag), got in res.items():
            assert torch.equal(got, seed_tensor((r - 1) % world, 32, dt).cpu()), (r, dt, tag)


def test_send_recv_order_headers_and_reuse(CX):
    world = 2
    n = 1_000_003

    def fn(r, pg):
        res = {}
        peer = 1 - r
        # both ranks send first, several messages, then receive: FIFO per pair
        msgs = [torch.full((n,), float(10 * r + i), device="cuda") for i in range(3)]
        works = [pg.send([m], peer, i) for i, m in enumerate(msgs)]
        [w.wait() for w in works]
        for m in msgs:
            m.add_(1000.0)            # a finished send has taken its copy: the tensor is the sender's again
        got = [torch.empty(n, device="cuda") for _ in range(3)]
        rw = [pg.recv([g], peer, i) for i, g in enumerate(got)]
        [w.wait() for w in rw]
        res["fifo"] = [float(g[0]) for g in got] + [float(g[-1]) for g in got]
        # header checks (ProcessGroupMCCL.cpp:645-651)
        pg.send([torch.ones(4, device="cuda")], peer, 5).wait()
        try:
            pg.recv([torch.empty(4, device="cuda")], peer, 6).wait()
        except RuntimeError as e:
            res["tag"] = str(e)
        pg.send([torch.ones(4, device="cuda")], peer, 5).wait()
        try:
            pg.recv([torch.empty(3, device="cuda")], peer, 5).wait()
        except RuntimeError as e:
            res["size"] = str(e)
        # several tensors in one call
        a, b = torch.full((7,), 1.0 + r, device="cuda"), torch.full((9,), 5.0 + r, device="cuda", dtype=torch.float16)
        pg.send([a, b], peer, 1).wait()
        ra, rb = torch.empty(7, device="cuda"), torch.empty(9, device="cuda", dtype=torch.float16)
        pg.recv([ra, rb], peer, 1).wait()
        res["multi"] = (ra.cpu().tolist(), rb.float().cpu().tolist())
        return res

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for r, res in enumerate(out):
        p = 1 - r
        assert res["fifo"] == [10.0 * p + i for i in range(3)] * 2
        assert "recv: tag mismatch (expected 6 got 5)" in res["tag"]
        assert "recv: size mismatch (expected 12 got 16)" in res["size"]
        assert res["multi"] == ([1.0 + p] * 7, [5.0 + p] * 9)


def test_recv_times_out_when_nothing_was_sent(CX):
    store = dist.HashStore()
    short = datetime.timedelta(seconds=2)
    msgs = [None, None]

    def body(r):
        torch.cuda.set_device(0)
        pg = CX._create_process_group_mccl(store, r, 2, short)
        if r == 0:
            try:
                pg.recv([torch.empty(4, device="cuda")], 1, 0).wait()
            except RuntimeError as e:
                msgs[0] = str(e)
        # the mesh is still usable: a later message arrives
        if r == 1:
            import time; time.sleep(3.0)
            pg.send([torch.full((4,), 9.0, device="cuda")], 0, 3).wait()
            msgs[1] = "sent"
        else:
            t = torch.empty(4, device="cuda")
            for attempt in range(10):          # each attempt waits up to the group's 2 s
                try:
                    pg.recv([t], 1, 3).wait()
                    break
                except RuntimeError:
                    continue
            msgs.append(t.cpu().tolist())

    ts = [threading.Thread(target=body, args=(r,)) for r in range(2)]
    [t.start() for t in ts]
    [t.join(60) for t in ts]
    assert not any(t.is_alive() for t in ts)
    assert "Timeout" in msgs[0] and "nothing arrived from rank 1" in msgs[0]
    assert msgs[2] == [9.0] * 4


# ---- recorded allreduces ---------------------------------------------------------------

@pytest.mark.parametrize("wire", [False, True])
def test_repeated_allreduce_is_replayed_from_a_graph_and_stays_bit_exact(CX, U, monkeypatch, wire):
    """The same buffers reduced again and again (a DDP bucket): from the second time on the
    launches are recorded, later calls replay the graph.  Every call is checked against the
    oracle, with other work on torch's stream and other collectives between the replays."""
    world, n = 3, 300_007
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "butterfly")
    if wire:
        monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    else:
        monkeypatch.delenv("MCCL_WIRE_DTYPE", raising=False)
    monkeypatch.delenv("MCCL_GRAPH_CACHE", raising=False)
    monkeypatch.setenv("MCCL_GRAPH_MIN_LAUNCHES", "1")   # by default only allreduces of six launches or more are recorded
    rng = np.random.default_rng(77)
    rounds = 8
    data = [[U.rand_values(rng, n, F32, scale=1e-2, specials=(i == 3)) for _ in range(world)] for i in range(rounds)]

    def fn(r, pg):
        bucket = torch.empty(n, device="cuda")          # one address for every round
        other = torch.empty(1000, device="cuda")
        got = []
        for i in range(rounds):
            bucket.copy_(torch.from_numpy(data[i][r]))
            o = dist.AllreduceOptions(); o.reduceOp = dist.ReduceOp.AVG
            pg.allreduce([bucket], o).wait()
            got.append(U.bits(bucket).copy())
            other.fill_(float(i)).mul_(2.0)                # unrelated eager work between replays
            if i % 3 == 1:
                pg.broadcast([other], dist.BroadcastOptions()).wait()
        return got, CX._graph_hits(pg)

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for i in range(rounds):
        want = [x.copy() for x in data[i]]
        rc, used = orc.pg_allreduce(want, F32, AVG, wire_bf16=wire, env_algo="butterfly", threads=4)
        assert rc == 0 and used == BUTTERFLY
        for r in range(world):
            w = want[r].view(np.uint32)
            g = out[r][0][i]
            same = (g == w) | (np.isnan(g.view(np.float32)) & np.isnan(w.view(np.float32)))
            assert same.all(), (i, r, int((~same).sum()))
    assert out[0][1] >= rounds - 2          # first call eager, second records and replays


def test_graph_cache_can_be_switched_off(CX, monkeypatch):
    monkeypatch.setenv("MCCL_GRAPH_CACHE", "0")
    monkeypatch.delenv("MCCL_WIRE_DTYPE", raising=False)

    def fn(r, pg):
        t = torch.empty(4096, device="cuda")
        for i in range(5):
            t.fill_(float(r + i))
            pg.allreduce([t]).wait()
            assert float(t[0]) == 2.0 * i + 1.0
        return CX._graph_hits(pg)

    out, errs = run_ranks(CX, 2, fn)
    assert errs == [None, None], errs
    assert out == [0, 0]


def test_allreduce_of_a_long_tensor_list_goes_out_together(CX, U, monkeypatch):
    """The C4 shape through the c10d surface: one allreduce call over a list of 600 small
    messages (tree, since each is below MCCL_TREE_BELOW) plus a few larger ones (ring);
    every message bit-exact against the oracle's replay of the reference."""
    world = 3
    monkeypatch.delenv("MCCL_ALLREDUCE_ALGO", raising=False)
    monkeypatch.delenv("MCCL_WIRE_DTYPE", raising=False)
    monkeypatch.delenv("MCCL_TREE_BELOW", raising=False)
    rng = np.random.default_rng(404)
    sizes = [16384] * 200 + [int(n) for n in rng.integers(1, 5000, 400)] + [70000, 100003]
    host = [[U.rand_values(rng, n, F32, scale=1.0) for _ in range(world)] for n in sizes]

    def fn(r, pg):
        ts = [U.to_dev(msg[r], F32) for msg in host]
        pg.allreduce(ts).wait()
        return [U.bits(t) for t in ts]

    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, errs
    for i, (n, msg) in enumerate(zip(sizes, host)):
        want = [x.copy() for x in msg]
        rc, used = orc.pg_allreduce(want, F32, SUM)
        assert rc == 0 and used == (TREE if n * 4 <= 262144 else RING)
        for r in range(world):
            assert np.array_equal(out[r][i], want[r].view(np.uint32)), (i, n, r)
