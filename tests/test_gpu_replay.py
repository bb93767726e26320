"""GPU parity of the chunk scheduler: the N-virtual-rank replay of ring / tree /
butterfly allreduce, reduce_scatter and allgather (STEPWISE = the reference's
launches one by one, FUSED = one multi-input pass per chunk) against the
oracle's message-by-message replay of the reference."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG, PRODUCT, MIN, MAX, RING, TREE, BUTTERFLY

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from mccl_amd import kernels
    kernels.hip_kernels_init(0)
    return kernels


@pytest.fixture(scope="module")
def H():
    from mccl_amd import harness, kernels
    kernels.hip_kernels_init(0)
    return harness


@pytest.fixture(scope="module")
def U():
    import gpu_util
    return gpu_util


STEPWISE, FUSED, DIRECT = 0, 1, 2


def run_case(H, U, algo, world, dtype, op, wire, mode, numel, seed, specials=False):
    rng = np.random.default_rng(seed)
    xs = [U.rand_values(rng, numel, dtype, scale=10.0 ** rng.integers(-3, 2), specials=specials)
          for _ in range(world)]
    want = [x.copy() for x in xs]
    rc = orc.allreduce(algo, want, dtype, op) if not wire else \
        orc.pg_allreduce(want, dtype, op, wire_bf16=True, env_algo={RING: "ring", TREE: "tree", BUTTERFLY: "butterfly"}[algo])[0]
    assert rc == 0
    d = [U.to_dev(x, dtype) for x in xs]
    H.allreduce_replay(d, op, algo, wire_bf16=wire, mode=mode)
    for r in range(world):
        if dtype == F16:
            assert np.array_equal(U.bits(d[r]), want[r]), (algo, world, r)
        else:
            U.assert_same_bits(d[r], want[r], dtype, f"algo={algo} world={world} rank={r} op={op} wire={wire} mode={mode}")


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
@pytest.mark.parametrize("world", [2, 3, 4, 5, 8])
@pytest.mark.parametrize("mode", [STEPWISE, FUSED, DIRECT])
@pytest.mark.parametrize("dtype,wire", [(F32, False), (BF16, False), (F32, True)])
def test_allreduce_sum_avg(H, U, algo, world, mode, dtype, wire):
    for op in (SUM, AVG):
        for numel in (world, 1237, 40009):   # numel == world: one element per chunk
            run_case(H, U, algo, world, dtype, op, wire, mode, numel, seed=world * 100 + algo * 10 + op,
                     specials=(numel > 1000 and dtype != F16))


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
@pytest.mark.parametrize("op", [PRODUCT, MIN, MAX])
@pytest.mark.parametrize("mode", [STEPWISE, FUSED, DIRECT])
def test_allreduce_other_ops_and_fp16(H, U, algo, op, mode):
    for world in (2, 3, 4):
        for dtype, wire in ((F32, False), (BF16, False), (F16, False), (F32, True)):
            run_case(H, U, algo, world, dtype, op, wire, mode, 5003, seed=world + op)
    run_case(H, U, algo, 3, F16, SUM, False, mode, 5003, seed=1)
    run_case(H, U, algo, 3, F16, AVG, False, mode, 5003, seed=2)


def tie_and_nan_values(rng, n, dtype, world):
    """Operands on which MIN / MAX depend on which side is dst: +0 against -0 (a tie
    keeps dst) and NaN against numbers (a NaN on either side keeps dst), at positions
    that differ from rank to rank, between ordinary values.  fp16 gets the zeros only
    (the payload of an fp16 NaN is hardware-defined)."""
    pool = np.array([0.0, -0.0, 1.0, -1.0, 0.0, -0.0] + ([] if dtype == F16 else [np.nan, -np.nan, np.nan]),
                    dtype=np.float32)
    out = []
    for _ in range(world):
        x = pool[rng.integers(0, pool.size, n)]
        plain = rng.random(n) < 0.2
        x[plain] = rng.standard_normal(int(plain.sum())).astype(np.float32)
        if dtype == F32:
            out.append(x)
        elif dtype == BF16:
            out.append(orc.encode_bf16(x))
        else:
            out.append(x.astype(np.float16).view(np.uint16))
    return out


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
@pytest.mark.parametrize("op", [MIN, MAX])
def test_min_max_operand_roles_on_ties_and_nans(H, U, algo, op):
    """The reference's min/max keep dst on a +0/-0 tie and when an operand is NaN
    (shaders.metal:65-72), and each schedule decides which operand is dst: the ring
    reduces the travelling partial result into the receiver's own chunk
    (AllreduceAlgos.cpp:72-74), the others reduce received data into the partial result.
    FUSED == STEPWISE == oracle, bit for bit, for every schedule."""
    rng = np.random.default_rng(500 + 10 * algo + op)
    names = {RING: "ring", TREE: "tree", BUTTERFLY: "butterfly"}
    for world in (2, 3, 4, 5, 9, 12):
        for dtype, wire in ((F32, False), (BF16, False), (F16, False), (F32, True)):
            xs = tie_and_nan_values(rng, 6007, dtype, world)
            want = [x.copy() for x in xs]
            rc = orc.allreduce(algo, want, dtype, op) if not wire else \
                orc.pg_allreduce(want, dtype, op, wire_bf16=True, env_algo=names[algo])[0]
            assert rc == 0
            got = {}
            for mode in (STEPWISE, FUSED):
                d = [U.to_dev(x, dtype) for x in xs]
                H.allreduce_replay(d, op, algo, wire_bf16=wire, mode=mode)
                got[mode] = [U.bits(t) for t in d]
                for r in range(world):
                    w = U.np_bits(np.ascontiguousarray(want[r]))
                    assert np.array_equal(got[mode][r], w), \
                        f"{names[algo]} world={world} dtype={dtype} wire={wire} mode={mode} rank={r}: " \
                        f"{int((got[mode][r] != w).sum())} elements differ from the oracle"
            for r in range(world):
                assert np.array_equal(got[STEPWISE][r], got[FUSED][r])


@pytest.mark.parametrize("op", [MIN, MAX])
def test_reduce_scatter_min_max_on_ties_and_nans(H, U, op):
    rng = np.random.default_rng(600 + op)
    CH = 3001
    for world in (2, 3, 8, 11):
        for dtype in (F32, BF16, F16):
            ins = tie_and_nan_values(rng, CH * world, dtype, world)
            want = [np.zeros(CH, dtype=ins[0].dtype) for _ in range(world)]
            assert orc.reduce_scatter(want, ins, dtype, op) == 0
            for mode in (STEPWISE, FUSED):
                din = [U.to_dev(x, dtype) for x in ins]
                dout = [torch.empty(CH, dtype=din[0].dtype, device="cuda") for _ in range(world)]
                H.reduce_scatter_replay(dout, din, op, mode=mode)
                for r in range(world):
                    assert np.array_equal(U.bits(dout[r]), U.np_bits(np.ascontiguousarray(want[r]))), \
                        (world, dtype, mode, r)


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
def test_worlds_wider_than_one_fold(H, U, algo):
    """More ranks than one fold takes operands: ring and butterfly chain folds (8 operands, then
    the partial result + 7 more, ...), the tree folds blocks of 8 ranks and then the blocks; all bit-exact."""
    run_case(H, U, algo, 11, F32, SUM, True, FUSED, 2003, seed=11)
    run_case(H, U, algo, 16, BF16, AVG, False, FUSED, 2003, seed=16)
    run_case(H, U, algo, 9, F32, AVG, False, FUSED, 40009, seed=9, specials=True)
    run_case(H, U, algo, 23, F32, AVG, True, FUSED, 5003, seed=23, specials=True)
    run_case(H, U, algo, 10, BF16, MAX, False, FUSED, 3001, seed=10)
    run_case(H, U, algo, 12, F32, PRODUCT, True, FUSED, 3001, seed=12)
    if algo == TREE:     # a tree of 8-rank trees up to 64 ranks, the stepwise schedule beyond
        for world, dtype, op, wire in ((17, F32, AVG, False), (33, F32, SUM, True), (64, BF16, SUM, False),
                                       (57, F32, MIN, True), (65, F32, AVG, True)):
            run_case(H, U, algo, world, dtype, op, wire, FUSED, 1237, seed=world)


def test_tree_with_fewer_elements_than_ranks(H, U):  # ProcessGroupMCCL.cpp:143-145 -> tree
    for mode in (STEPWISE, FUSED):
        run_case(H, U, TREE, 5, F32, SUM, False, mode, 3, seed=3)
        run_case(H, U, TREE, 4, F32, AVG, True, mode, 1, seed=4)


def test_preconditions(H):
    from mccl_amd import MCCLError
    t = [torch.ones(2, device="cuda") for _ in range(3)]
    for algo in (RING, BUTTERFLY):
        with pytest.raises(MCCLError, match="numel must be >= world"):   # AllreduceAlgos.cpp:55,137
            H.allreduce_replay(t, SUM, algo)
    with pytest.raises(MCCLError, match="Unsupported ReduceOp: 5"):
        H.allreduce_replay(t, 5, TREE)
    with pytest.raises(MCCLError, match="empty tensor list"):
        H.allreduce_replay([], SUM, TREE)
    one = [torch.full((4,), 7.0, device="cuda")]
    H.allreduce_replay(one, AVG, RING)                                   # world == 1: no-op (PG.cpp:107)
    assert torch.equal(one[0], torch.full((4,), 7.0, device="cuda"))


def test_env_semantics(H, U, monkeypatch):
    """MCCL_ALLREDUCE_ALGO / MCCL_TREE_BELOW / MCCL_WIRE_DTYPE are re-read per call."""
    rng = np.random.default_rng(9)

    def go(numel, world=3, dtype=F32):
        xs = [U.rand_values(rng, numel, dtype) for _ in range(world)]
        d = [U.to_dev(x, dtype) for x in xs]
        used = H.allreduce(d, "sum")
        return xs, d, used

    for k in ("MCCL_ALLREDUCE_ALGO", "MCCL_TREE_BELOW", "MCCL_WIRE_DTYPE"):
        monkeypatch.delenv(k, raising=False)
    assert go(65536)[2] == TREE            # 262144 B <= default threshold (inclusive)
    assert go(65537)[2] == RING
    monkeypatch.setenv("MCCL_TREE_BELOW", "1000")
    assert go(300)[2] == RING and go(250)[2] == TREE
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    assert go(500)[2] == TREE              # threshold applies to the bf16 byte size
    assert go(500, dtype=BF16)[2] == TREE and go(501, dtype=BF16)[2] == RING
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "butterfly")
    xs, d, used = go(999)
    assert used == BUTTERFLY
    want = [x.copy() for x in xs]
    assert orc.pg_allreduce(want, F32, SUM, wire_bf16=True, env_algo="butterfly", tree_below=1000) == (0, BUTTERFLY)
    U.assert_same_bits(d[1], want[1], F32, "env butterfly + wire")
    assert go(2)[2] == TREE                # numel < world
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "nonsense")
    assert go(100000)[2] == TREE
    monkeypatch.setenv("MCCL_WIRE_DTYPE", "fp16")   # only "bf16" switches the codec on
    monkeypatch.setenv("MCCL_ALLREDUCE_ALGO", "ring")
    xs, d, used = go(999)
    want = [x.copy() for x in xs]; orc.allreduce(RING, want, F32, SUM)
    U.assert_same_bits(d[0], want[0], F32, "no wire")


@pytest.mark.parametrize("world", [2, 3, 8, 10, 17])
@pytest.mark.parametrize("dtype", [F32, BF16, F16])
@pytest.mark.parametrize("mode", [STEPWISE, FUSED])
def test_reduce_scatter_allgather(H, U, world, dtype, mode):
    rng = np.random.default_rng(world)
    CH = 4099
    for op in (SUM, AVG, MIN, MAX, PRODUCT):
        ins = [U.rand_values(rng, CH * world, dtype) for _ in range(world)]
        want = [np.zeros(CH, dtype=ins[0].dtype) for _ in range(world)]
        assert orc.reduce_scatter(want, ins, dtype, op) == 0
        din = [U.to_dev(x, dtype) for x in ins]
        dout = [torch.empty(CH, dtype=din[0].dtype, device="cuda") for _ in range(world)]
        H.reduce_scatter_replay(dout, din, op, mode=mode)
        for r in range(world):
            if dtype == F16:
                assert np.array_equal(U.bits(dout[r]), want[r])
            else:
                U.assert_same_bits(dout[r], want[r], dtype, f"reduce_scatter op={op} rank={r}")
    # in place: out is the rank's own slice of its input (tests/collectives/test_reduce_scatter.py:24-29)
    ins = [U.rand_values(rng, CH * world, dtype) for _ in range(world)]
    want = [np.zeros(CH, dtype=ins[0].dtype) for _ in range(world)]
    orc.reduce_scatter(want, ins, dtype, SUM)
    din = [U.to_dev(x, dtype) for x in ins]
    dout = [din[r].narrow(0, r * CH, CH) for r in range(world)]
    H.reduce_scatter_replay(dout, din, SUM, mode=mode)
    for r in range(world):
        if dtype == F16:
            assert np.array_equal(U.bits(dout[r]), want[r])
        else:
            U.assert_same_bits(dout[r], want[r], dtype, "in place")
    # allgather of the results (tests/collectives/allgather.py)
    gout = [torch.empty(CH * world, dtype=din[0].dtype, device="cuda") for _ in range(world)]
    H.allgather_replay(gout, [o.contiguous() for o in dout])
    cat = np.concatenate([U.bits(o) for o in dout])
    for g in gout:
        assert np.array_equal(U.bits(g), cat)


def test_reduce_scatter_reference_vectors(H, U):
    """tests/collectives/test_reduce_scatter.py:14-44: value (p+1)*10+rank, CHUNK=32."""
    world, CH = 4, 32
    for dtype, tdt in ((F32, torch.float32), (BF16, torch.bfloat16), (F16, torch.float16)):
        ins = [torch.cat([torch.full((CH,), float((p + 1) * 10 + r), dtype=tdt, device="cuda")
                          for p in range(world)]) for r in range(world)]
        outs = [torch.empty(CH, dtype=tdt, device="cuda") for _ in range(world)]
        H.reduce_scatter_replay(outs, ins, "sum")
        for r in range(world):
            exp = sum((r + 1) * 10 + q for q in range(world))
            assert torch.allclose(outs[r].float().cpu(), torch.full((CH,), float(exp)), rtol=1e-2, atol=1e-2)
        H.reduce_scatter_replay(outs, ins, "max")
        for r in range(world):
            assert torch.equal(outs[r].float().cpu(), torch.full((CH,), float((r + 1) * 10 + world - 1)))


def test_f32acc_reduce_scatter_variant(H, U):
    """The fp32-accumulate mode (not the reference) equals its own oracle and
    stays within one bf16 ulp of the exact sum."""
    rng = np.random.default_rng(8)
    world, CH = 8, 10007
    ins = [U.rand_values(rng, CH * world, BF16, scale=1e-2) for _ in range(world)]
    want = [np.zeros(CH, dtype=np.uint16) for _ in range(world)]
    orc.reduce_scatter_f32acc(want, ins, SUM)
    din = [U.to_dev(x, BF16) for x in ins]
    dout = [torch.empty(CH, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    H.reduce_scatter_replay(dout, din, SUM, mode=FUSED, acc=1)
    for r in range(world):
        assert np.array_equal(U.bits(dout[r]), want[r])
    # AVG: the factor 1/world stays fp32 as well (1/7 is not a bf16 value), one rounding at the end
    for world in (3, 7):
        ins = [U.rand_values(rng, CH * world, BF16, scale=1e-2, specials=True) for _ in range(world)]
        want = [np.zeros(CH, dtype=np.uint16) for _ in range(world)]
        orc.reduce_scatter_f32acc(want, ins, AVG)
        din = [U.to_dev(x, BF16) for x in ins]
        dout = [torch.empty(CH, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
        H.reduce_scatter_replay(dout, din, AVG, mode=FUSED, acc=1)
        for r in range(world):
            U.assert_same_bits(dout[r], want[r], BF16, f"f32acc AVG world {world} rank {r}")


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
@pytest.mark.parametrize("dtype,wire", [(F32, False), (BF16, False), (F32, True)])
def test_many_messages_in_one_replay_equal_single_replays(H, U, algo, dtype, wire):
    """A list of allreduces issued together (one launch per phase for all of them) gives
    what the oracle gives for each message on its own: mixed sizes, more messages than fit
    the kernel arguments, world 3."""
    world = 3
    rng = np.random.default_rng(17 + algo)
    sizes = [3, 5, 64, 997, 4099, 16384, 16384, 33, 70001] + [int(n) for n in rng.integers(3, 3000, 40)]
    host = [[U.rand_values(rng, n, dtype, scale=1e-2, specials=(n > 64)) for _ in range(world)] for n in sizes]
    groups = [[U.to_dev(x, dtype) for x in msg] for msg in host]
    H.allreduce_replay_many(groups, "avg" if dtype == F32 else "sum", algo, wire_bf16=wire)
    for n, msg, g in zip(sizes, host, groups):
        want = [x.copy() for x in msg]
        op = AVG if dtype == F32 else SUM
        rc = orc.allreduce(algo, want, dtype, op) if not wire else \
            orc.pg_allreduce(want, dtype, op, wire_bf16=True, env_algo={RING: "ring", TREE: "tree", BUTTERFLY: "butterfly"}[algo])[0]
        assert rc == 0
        for r in range(world):
            U.assert_same_bits(g[r], want[r], dtype, f"algo {algo} n {n} rank {r}")


def test_list_replay_with_a_tensor_named_twice_runs_in_order(H, U):
    """A list whose entries share memory cannot be issued phase by phase: the second
    allreduce of the same tensors must see the first one's result, as in the reference's
    one-by-one loop (ProcessGroupMCCL.cpp:173-177)."""
    world = 3
    rng = np.random.default_rng(44)
    for dtype, wire in ((F32, False), (F32, True), (BF16, False)):
        a = [U.rand_values(rng, 5003, dtype, scale=1e-2) for _ in range(world)]
        b = [U.rand_values(rng, 777, dtype, scale=1e-2) for _ in range(world)]
        da, db = [U.to_dev(x, dtype) for x in a], [U.to_dev(x, dtype) for x in b]
        H.allreduce_replay_many([da, db, da, da], "sum", BUTTERFLY, wire_bf16=wire)
        wa, wb = [x.copy() for x in a], [x.copy() for x in b]
        for bufs, times in ((wa, 3), (wb, 1)):
            for _ in range(times):
                rc = orc.allreduce(BUTTERFLY, bufs, dtype, SUM) if not wire else \
                    orc.pg_allreduce(bufs, dtype, SUM, wire_bf16=True, env_algo="butterfly")[0]
                assert rc == 0
        for r in range(world):
            U.assert_same_bits(da[r], wa[r], dtype, f"tensor reduced three times, rank {r}")
            U.assert_same_bits(db[r], wb[r], dtype, f"tensor reduced once, rank {r}")


def test_copy_batched_many_small_and_a_few_large(K, U):
    rng = np.random.default_rng(3)
    q = K._q(None)
    for sizes in ([int(n) for n in rng.integers(1, 70000, 300)], [1, 2, 3, 15, 16, 17], [20_000_001, 9_000_003, 5, 0, 7]):
        total = sum(sizes) + 64 * len(sizes)
        src = torch.randint(0, 256, (total,), dtype=torch.uint8, device="cuda")
        dst = torch.zeros(total, dtype=torch.uint8, device="cuda")
        want = np.zeros(total, np.uint8)
        hs = src.cpu().numpy()
        triples, off = [], 0
        for i, n in enumerate(sizes):
            so, do = off + int(rng.integers(0, 16)), off + int(rng.integers(0, 16))
            triples.append((dst.data_ptr() + do, src.data_ptr() + so, n))
            want[do:do + n] = hs[so:so + n]
            off += n + 64
        torch.cuda.synchronize()
        q.copy_batched(triples)
        q.drain()
        assert np.array_equal(dst.cpu().numpy(), want), sizes[:5]


def test_launch_counts_of_the_fused_schedules(H, K, U):
    """What "fused" means in launches.  Up to four ranks a sum needs no allgather launch: the
    owner's fold stores the reduced chunk into every rank's tensor, so butterfly over the wire =
    encode + fold (2) and without the wire one fold (1); the other reduce ops, and five ranks or
    more, keep the separate cast / copy launch (3, or 1 fold + the allgather copies); a list of
    200 tree messages = 1 launch; the stepwise replay of the same butterfly issues the
    reference's sequence."""
    from mccl_amd import _lib as L
    q = K._q(None)
    world, n = 3, 300_000
    rng = np.random.default_rng(8)

    def launches(fn):
        before = q.launch_count()
        fn()
        return q.launch_count() - before

    mk = lambda: [U.to_dev(U.rand_values(rng, n, F32), F32) for _ in range(world)]
    for op in ("avg", "min", "max", "product"):
        t = mk()
        assert launches(lambda: H.allreduce_replay(t, op, BUTTERFLY, wire_bf16=True, mode=FUSED)) == (2 if op == "avg" else 3), op
    t = mk()
    assert launches(lambda: H.allreduce_replay(t, "sum", BUTTERFLY, mode=FUSED)) == 1
    t = mk()
    assert launches(lambda: H.allreduce_replay(t, "max", BUTTERFLY, mode=FUSED)) == 1 + 1   # 6 copies of 400 KB: one launch
    # DIRECT: the fold reads the ranks' fp32 tensors itself -- the whole wire allreduce of up to
    # four ranks is one launch, of five to eight a fold and the casts on arrival
    for algo in (RING, TREE, BUTTERFLY):
        t = mk()
        assert launches(lambda: H.allreduce_replay(t, "avg", algo, wire_bf16=True, mode=DIRECT)) == 1
    t = mk()
    assert launches(lambda: H.allreduce_replay(t, "max", BUTTERFLY, wire_bf16=True, mode=DIRECT)) == 3
    five = [U.to_dev(U.rand_values(rng, n, F32), F32) for _ in range(5)]
    assert launches(lambda: H.allreduce_replay(five, "avg", RING, wire_bf16=True, mode=DIRECT)) == 2
    assert launches(lambda: H.allreduce_replay(five, "sum", RING, mode=FUSED)) == 1 + 1
    assert launches(lambda: H.allreduce_replay(five, "avg", RING, wire_bf16=True, mode=FUSED)) == 3
    t = mk()
    stepwise = launches(lambda: H.allreduce_replay(t, "avg", BUTTERFLY, wire_bf16=True, mode=STEPWISE))
    assert stepwise >= 3 + 2 * 3 * 2 + 3 + 3       # encodes, (copy + reduce) per peer and rank, scales, ..., decodes
    groups = [[U.to_dev(U.rand_values(rng, 5000 + 7 * i, F32), F32) for _ in range(world)] for i in range(200)]
    assert launches(lambda: H.allreduce_replay_many(groups, "sum", TREE)) == 1
    wide = [U.to_dev(U.rand_values(rng, n, F32), F32) for _ in range(16)]     # 16 ranks: folds of 8, 8 and 2 operands
    assert launches(lambda: H.allreduce_replay(wide, "avg", RING, wire_bf16=True, mode=FUSED)) == 1 + 3 + 1
    small = [U.to_dev(U.rand_values(rng, 1000, F32), F32) for _ in range(20)]  # tree of 20: blocks 8 + 8 + 4, then 3
    assert launches(lambda: H.allreduce_replay(small, "sum", TREE, mode=FUSED)) == 3 + 1
