"""The five measured configurations at their full sizes.

Where the oracle finishes in seconds the whole result is compared bit for bit;
at the largest sizes the check is (a) the fused schedule equals the stepwise one
(the reference's launches one by one, themselves pinned against the oracle at
small sizes) over every element, (b) the oracle on windows around every chunk
boundary, the ragged tail and the injected special values, and (c) the
invariants of the collective (all ranks identical, allgather = concatenation)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, BF16, SUM, AVG, RING, TREE, BUTTERFLY

pytestmark = pytest.mark.gpu

STEPWISE, FUSED = 0, 1


@pytest.fixture(scope="module")
def env():
    from mccl_amd import kernels, harness, workloads, _lib
    import gpu_util
    kernels.hip_kernels_init(0)
    return kernels, harness, workloads, _lib, gpu_util


def test_c1_ring_two_ranks_full(env):
    K, H, W, L, U = env
    xs = [W.c1_input(r) for r in range(2)]
    want = [x.copy() for x in xs]
    assert orc.allreduce(RING, want, F32, SUM, threads=8) == 0
    for mode in (STEPWISE, FUSED):
        d = [U.to_dev(x, F32) for x in xs]
        H.allreduce_replay(d, "sum", L.ALGO_RING, mode=mode)
        for r in range(2):
            U.assert_same_bits(d[r], want[r], F32, f"C1 mode {mode} rank {r}")


def test_c2_butterfly_bucket_full(env):
    K, H, W, L, U = env
    xs = [W.c2_input(r) for r in range(3)]
    want = [x.copy() for x in xs]
    rc, algo = orc.pg_allreduce(want, F32, AVG, wire_bf16=True, env_algo="butterfly", threads=8)
    assert rc == 0 and algo == BUTTERFLY
    assert np.array_equal(want[0], want[1]) and np.array_equal(want[1], want[2])
    for mode in (STEPWISE, FUSED, L.REPLAY_DIRECT):
        d = [U.to_dev(x, F32) for x in xs]
        H.allreduce_replay(d, "avg", L.ALGO_BUTTERFLY, wire_bf16=True, mode=mode)
        for r in range(3):
            U.assert_same_bits(d[r], want[r], F32, f"C2 mode {mode} rank {r}")
    # the outliers survive: +-1e2 dominates its element
    assert np.abs(want[0]).max() > 30.0


def _windows(chunks, numel, width=4096):
    """Index ranges around every chunk boundary, plus the start and the ragged end."""
    edges = {0, numel}
    for s, c, _, _ in chunks:
        edges.add(s)
        edges.add(s + c)
    out = []
    for e in sorted(edges):
        lo, hi = max(0, e - width), min(numel, e + width)
        if hi > lo:
            out.append((lo, hi))
    return out


def test_c3_ring_110m_ragged_hbm_and_pinned_host(env):
    K, H, W, L, U = env
    world, numel = 4, W.C3["numel"]
    g = torch.Generator(device="cuda").manual_seed(3)
    base = [torch.randn(numel, device="cuda", generator=g) * 1e-4 for _ in range(world)]
    chunks = H.chunkize(numel, 1, world)
    assert [c[1] for c in chunks] == [27500001] * 3 + [27499999]        # ragged tail
    fused = [t.clone() for t in base]
    H.allreduce_replay(fused, "sum", L.ALGO_RING, wire_bf16=True, mode=FUSED)
    step = [t.clone() for t in base]
    H.allreduce_replay(step, "sum", L.ALGO_RING, wire_bf16=True, mode=STEPWISE)
    for r in range(world):
        assert torch.equal(fused[r].view(torch.int32), step[r].view(torch.int32)), f"rank {r}: fused != stepwise"
        assert torch.equal(fused[r].view(torch.int32), fused[0].view(torch.int32)), "ranks differ"
    del step
    direct = [t.clone() for t in base]     # one launch: the fold reads the four fp32 tensors where they lie
    H.allreduce_replay(direct, "sum", L.ALGO_RING, wire_bf16=True, mode=L.REPLAY_DIRECT)
    for r in range(world):
        assert torch.equal(fused[r].view(torch.int32), direct[r].view(torch.int32)), f"rank {r}: fused != direct"
    del direct
    # oracle on windows: chunk c folds x_c, x_{c+1}, ..., owner last (AllreduceAlgos.cpp:62-75)
    for lo, hi in _windows(chunks, numel):
        host = [t[lo:hi].cpu().numpy() for t in base]
        want = [h.copy() for h in host]
        # inside one window all elements may belong to two chunks: fold per chunk
        for ch, (s, c, _, _) in enumerate(chunks):
            a, b = max(lo, s), min(hi, s + c)
            if b <= a:
                continue
            owner = (ch - 1) % world
            order = [(ch + j) % world for j in range(world)]
            peers = [orc.encode_bf16(np.ascontiguousarray(host[p][a - lo:b - lo])) for p in order[:-1]]
            res = orc.wire_fold_chunk(np.ascontiguousarray(host[owner][a - lo:b - lo]), peers, own_last=True)
            got = fused[0][a:b].cpu().numpy()
            assert np.array_equal(got.view(np.uint32), res.view(np.uint32)), (ch, a, b)
    # zero-copy variant: the peers' wire chunks live in pinned host memory and are read across PCIe
    q = K.hip_kernels_init(0)
    wires = [K.encode_bf16(t) for t in base]
    K.hip_sync()
    hbm_out = [torch.empty(c[1], device="cuda") for c in chunks]
    pin_out = [torch.empty(c[1], device="cuda") for c in chunks]
    host_bufs, dev_ptrs = [], []
    try:
        for w in wires:
            h, d = q.host_alloc(numel * 2)
            host_bufs.append(h)
            dev_ptrs.append(d)
            q.copy(d, w.data_ptr(), numel * 2)
        q.drain()
        plan = K.make_plan(L.BF16, world, io=L.IO_OWN_LAST_F32)
        for outs, wptr in ((hbm_out, [w.data_ptr() for w in wires]), (pin_out, dev_ptrs)):
            segs = []
            for ch, (s, c, _, _) in enumerate(chunks):
                o = (ch - 1) % world
                ins = [wptr[(ch + j) % world] + 2 * s for j in range(world - 1)] + [base[o].data_ptr() + 4 * s]
                segs.append(K.make_seg(outs[ch].data_ptr(), 0, ins, c))
            q.fold(plan, segs)
        q.drain()
    finally:
        for h in host_bufs:
            q.host_free(h)
    for ch, (s, c, _, _) in enumerate(chunks):
        assert torch.equal(hbm_out[ch].view(torch.int32), pin_out[ch].view(torch.int32)), "pinned != HBM"
        assert torch.equal(hbm_out[ch].view(torch.int32), fused[0][s:s + c].view(torch.int32))


def test_c3_ring_through_the_process_group_with_peers_in_pinned_host_memory(env, monkeypatch):
    """C3 at full size through the c10d surface: 4 ranks as 4 threads, MCCL_WIRE=host -- every rank
    encodes what it sends into pinned host memory, the transport delivers into the owner's pinned
    buffer, and the owner's fold reads its three peers across PCIe.  Same bits as the fused replay
    with everything in HBM (which the test above checks against the oracle)."""
    import datetime
    import threading
    import torch.distributed as dist
    from mccl_amd import _C as CX
    K, H, W, L, U = env
    world, numel = 4, W.C3["numel"]
    monkeypatch.setenv("MCCL_WIRE", "host")
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "ring")
    g = torch.Generator(device="cuda").manual_seed(3)
    base = [torch.randn(numel, device="cuda", generator=g) * 1e-4 for _ in range(world)]
    want = [t.clone() for t in base]
    H.allreduce_replay(want, "sum", L.ALGO_RING, wire_bf16=True, mode=FUSED)
    torch.cuda.synchronize()
    store = dist.HashStore()
    stats, errs = [None] * world, [None] * world

    def body(r):
        try:
            torch.cuda.set_device(0)
            pg = CX._create_process_group_mccl(store, r, world, datetime.timedelta(seconds=60))
            assert pg.allreduce([base[r]]).wait()
            stats[r] = CX._wire_stats(pg)
        except BaseException as e:  # noqa: BLE001
            errs[r] = e

    ts = [threading.Thread(target=body, args=(r,)) for r in range(world)]
    for t in ts:
        t.start()
    for t in ts:
        t.join(110)
    assert not any(t.is_alive() for t in ts), "a rank thread hung"
    assert errs == [None] * world, errs
    for r in range(world):
        assert torch.equal(base[r].view(torch.int32), want[r].view(torch.int32)), f"rank {r}"
    for calls, elems, peer_bytes, hbm_bytes, fold_ms, sent, *legs in stats:
        assert calls == 1 and elems in (27500001, 27499999)
        assert len(legs) == 5 and all(ms >= 0 for ms in legs) and sum(legs) > 0   # encode, scatter leg, fold, gather leg, casts
        assert peer_bytes == 3 * elems * 2 and fold_ms > 0
        print(f"C3 fold through the backend, peers in pinned host memory: {fold_ms:.2f} ms, "
              f"{peer_bytes / fold_ms / 1e6:.1f} GB/s over PCIe")


def test_c4_tree_4096_messages_one_launch(env):
    K, H, W, L, U = env
    m, n = W.C4["messages"], W.C4["numel"]
    g = torch.Generator(device="cuda").manual_seed(4)
    r = [torch.rand(m * n, device="cuda", generator=g) * 2 - 1 for _ in range(3)]
    host = [t.cpu().numpy() for t in r]
    out = torch.empty(m * n, device="cuda")
    segs = [K.make_seg(out.data_ptr() + 4 * n * i, 0, [t.data_ptr() + 4 * n * i for t in r], n) for i in range(m)]
    q = K.hip_kernels_init(0)
    q.fold(K.make_plan(L.F32, 3, topo=L.TOPO_BINOMIAL), segs)       # tree order for N=3: (x0 + x1) + x2
    q.drain()
    want = (host[0] + host[1]) + host[2]
    U.assert_same_bits(out, want, F32, "C4 batched")
    # and the same through the message-level scheduler: every message picks the tree (64 KiB <= 256 KiB)
    assert H.select_algo(None, None, n * 4, n, 3) == L.ALGO_TREE
    d = [t[:n * 8].clone() for t in r]
    for i in range(8):
        H.allreduce_replay([x[i * n:(i + 1) * n] for x in d], "sum", L.ALGO_TREE, mode=FUSED)
    for x in d:
        U.assert_same_bits(x, want[:n * 8], F32, "C4 per message")


def test_c5_reduce_scatter_allgather_512mib_bf16(env):
    K, H, W, L, U = env
    world, numel = 8, W.C5["numel"]
    ch = numel // world
    g = torch.Generator(device="cuda").manual_seed(5)
    sp = torch.tensor((W.C5_SPECIALS_F32 >> 16).astype(np.int64), device="cuda").to(torch.int16)
    ins = []
    for r in range(world):
        t = (torch.randn(numel, device="cuda", generator=g) * 1e-2).to(torch.bfloat16)
        idx = torch.arange(0, numel, 1_000_003, device="cuda")
        t.view(torch.int16)[idx] = sp[(torch.arange(idx.numel(), device="cuda") + r) % sp.numel()]
        ins.append(t)
    fused = [torch.empty(ch, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    H.reduce_scatter_replay(fused, ins, "sum", mode=FUSED)
    step = [torch.empty(ch, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    H.reduce_scatter_replay(step, ins, "sum", mode=STEPWISE)
    for r in range(world):
        assert torch.equal(fused[r].view(torch.int16), step[r].view(torch.int16)), f"rank {r}: fused != stepwise"
    del step
    # oracle: the first and last 2^20 elements of every rank's chunk, which hold injected specials
    Wn = 1 << 20
    for r in range(world):
        for lo in (0, ch - Wn):
            shares = [U.bits(ins[p][r * ch + lo: r * ch + lo + Wn]) for p in range(world)]
            acc = shares[r].copy()
            for p in range(world):
                if p != r:
                    orc.reduce(acc, shares[p], BF16, SUM, threads=8)
            got = U.bits(fused[r][lo:lo + Wn])
            assert np.array_equal(got, acc), (r, lo)
            spec = (np.arange(r * ch + lo, r * ch + lo + Wn) % 1_000_003) == 0
            assert spec.any()
    # NaN anywhere in a column poisons it to the canonical NaN; Inf - Inf likewise
    col0 = U.bits(fused[0][:1])[0]
    assert (col0 & 0x7FFF) > 0x7F80 and col0 == 0x7FC0
    # fp32-accumulate variant (not the reference) against its own oracle on a window
    f32acc = [torch.empty(ch, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    H.reduce_scatter_replay(f32acc, ins, "sum", mode=FUSED, acc=1)
    r = 3
    shares = [np.ascontiguousarray(U.bits(ins[p][r * ch: r * ch + Wn])) for p in range(world)]
    fake_ins = [np.concatenate([np.zeros(r * Wn, np.uint16), shares[p], np.zeros((world - 1 - r) * Wn, np.uint16)])
                for p in range(world)]
    want = [np.zeros(Wn, np.uint16) for _ in range(world)]
    orc.reduce_scatter_f32acc(want, fake_ins, SUM, threads=8)
    assert np.array_equal(U.bits(f32acc[r][:Wn]), want[r])
    del f32acc
    # allgather: every rank ends with the concatenation of the reduced chunks
    outs = [torch.empty(numel, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    H.allgather_replay(outs, fused)
    cat = torch.cat(fused)
    for o in outs:
        assert torch.equal(o.view(torch.int16), cat.view(torch.int16))


def test_graph_replays_match_eager(env):
    """Recorded launches (by-value and descriptor-table) replayed several times,
    with eager work and synchronisation in between, equal the eager result every time."""
    K, H, W, L, U = env
    q = K.hip_kernels_init(0)
    rng = np.random.default_rng(12)
    n = 50003
    a = [U.rand_values(rng, n * 12, F32) for _ in range(3)]
    d = [U.to_dev(x, F32) for x in a]
    out_few = torch.zeros(n * 12, device="cuda")
    out_tab = torch.zeros(n * 12, device="cuda")
    few = [K.make_seg(out_few.data_ptr() + 4 * n * i, 0, [t.data_ptr() + 4 * n * i for t in d], n) for i in range(3)]
    tab = [K.make_seg(out_tab.data_ptr() + 4 * n * i, 0, [t.data_ptr() + 4 * n * i for t in d], n) for i in range(12)]
    plan = K.make_plan(L.F32, 3, scale_mode=L.SCALE_VIEW, scale=1 / 3)
    K.hip_sync()
    q.graph_begin()
    q.fold(plan, few)
    q.fold(plan, tab)
    q.copy(out_few.data_ptr() + 4 * n * 6, out_tab.data_ptr() + 4 * n * 6, 4 * n)
    from mccl_amd import MCCLError
    with pytest.raises(MCCLError, match="not allowed between graph_begin and graph_end"):
        q.drain()
    graph = q.graph_end()
    want = ((a[0] + a[1]) + a[2]) * np.float32(1 / 3)
    for rep in range(4):
        out_few.zero_(); out_tab.zero_()
        torch.cuda.synchronize()
        q.graph_launch(graph)
        q.drain()
        U.assert_same_bits(out_tab, want, F32, f"table replay {rep}")
        assert np.array_equal(U.bits(out_few)[:3 * n], want.view(np.uint32)[:3 * n])
        assert np.array_equal(U.bits(out_few)[6 * n:7 * n], want.view(np.uint32)[6 * n:7 * n])
        # eager work of the program between replays
        e = torch.zeros(n * 3, device="cuda")
        q.fold(plan, [K.make_seg(e.data_ptr(), 0, [t.data_ptr() for t in d], n * 3)])
        q.drain()
        assert np.array_equal(U.bits(e), want.view(np.uint32)[:3 * n])
    q.graph_destroy(graph)


def test_counts_beyond_32_bits(env):
    """The reference narrows element counts to uint32 (MetalKernels.mm:156-163);
    here they are 64-bit: one launch over 2^32 + 4099 bf16 elements, checked
    against the oracle at the start, across the 2^32 boundary and at the ragged end."""
    K, H, W, L, U = env
    n = (1 << 32) + 4099
    g = torch.Generator(device="cuda").manual_seed(9)
    a = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    b = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    step = 1 << 28
    for lo in range(0, n, step):
        m = min(step, n - lo)
        a[lo:lo + m] = torch.randn(m, device="cuda", generator=g).to(torch.bfloat16)
        b[lo:lo + m] = torch.randn(m, device="cuda", generator=g).to(torch.bfloat16)
    windows = [(0, 1 << 16), ((1 << 32) - (1 << 15), (1 << 32) + 4099)]
    keep = [(U.bits(a[lo:hi]).copy(), U.bits(b[lo:hi]).copy()) for lo, hi in windows]
    K.hip_sync()
    K.hip_reduce_op_view(a.data_ptr(), b.data_ptr(), L.BF16, n, "sum")
    for (lo, hi), (wa, wb) in zip(windows, keep):
        orc.reduce(wa, wb, BF16, SUM, threads=8)
        assert np.array_equal(U.bits(a[lo:hi]), wa), (lo, hi)
    # a chunk boundary beyond 2^32 bytes: chunkize offsets are 64-bit too
    ch = H.chunkize(n, 2, 3)
    assert ch[2][2] == 2 * ch[2][0] > (1 << 32) and sum(c[1] for c in ch) == n
