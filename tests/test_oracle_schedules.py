"""Pins the oracle's chunking and schedules: the reference's own chunkize
(compiled from its checkout when present), the reference's unit-test cases,
hand-derived fold orders per algorithm, and schedule invariants."""
import ctypes as C
import itertools

import numpy as np
import pytest

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG, PRODUCT, MIN, MAX, RING, TREE, BUTTERFLY

WORLDS = (2, 3, 4, 8, 16, 30)                       # tests/internal/test_ring_chunks.cpp:25
NUMELS = (100, 1024, 1025, 1 << 20, 1234567)        # :26


# ---- chunkize ---------------------------------------------------------

@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("numel", NUMELS)
def test_chunks_cover_exactly(world, numel):  # test_ring_chunks.cpp:24-38
    ch = orc.chunkize(numel, 4, world)
    assert sum(c[1] for c in ch) == numel
    for s, n, off, ln in ch:
        assert 0 <= n and s + n <= numel and off == 4 * s and ln == 4 * n


def test_chunks_contiguous():  # :40-45
    ch = orc.chunkize(1000, 4, 7)
    for a, b in zip(ch, ch[1:]):
        assert b[0] == a[0] + a[1]


def test_chunks_degenerate():  # :59-73
    ch = orc.chunkize(3, 4, 5)
    assert len(ch) == 5 and sum(c[1] for c in ch) == 3
    assert sum(1 for c in ch if c[1] == 0) > 0


def test_config_chunk_sizes():
    assert [c[1] for c in orc.chunkize(6553600, 2, 3)] == [2184534, 2184534, 2184532]
    assert [c[1] for c in orc.chunkize(110000002, 2, 4)] == [27500001] * 3 + [27499999]
    assert [c[1] for c in orc.chunkize(1048576, 4, 2)] == [524288, 524288]


def test_chunkize_equals_reference_code():
    R = orc.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    assert R.ref_ring_chunks_selftest() == 0
    rng = np.random.default_rng(1)
    cases = list(itertools.product(WORLDS + (1, 5, 7), NUMELS + (0, 1, 2, 3, 5, 31, 6553600, 110000002)))
    cases += [(int(w), int(n)) for w, n in zip(rng.integers(1, 64, 200), rng.integers(0, 1 << 33, 200))]
    for world, numel in cases:
        for esize in (2, 4):
            out = (C.c_int64 * (4 * world))()
            R.ref_chunkize(numel, world, esize, out)
            mine = orc.chunkize(numel, esize, world)
            for i, (s, n, off, ln) in enumerate(mine):
                assert (s, s + n, off, ln) == tuple(out[4 * i:4 * i + 4]), (world, numel, esize, i)


# ---- hand-derived fold orders -------------------------------------------
# Each helper below states, independently of the oracle's message-passing
# replay, which operands meet in which order (derived by tracing
# AllreduceAlgos.cpp by hand; see the docstrings).

def f32add(a, b):
    return (a.astype(np.float32) + b.astype(np.float32)).astype(np.float32)


def bf16add(a, b):
    return orc.encode_bf16(orc.decode_bf16(a) + orc.decode_bf16(b))


def expected_ring(xs, add):
    """Chunk c is folded left to right starting at rank c:
    (((x_c + x_{c+1}) + x_{c+2}) + ...), indices mod N (AllreduceAlgos.cpp:62-75:
    at step k rank r adds the partial sum arriving from r-1 into its chunk
    r-k-1, dst being its own data -- fp add is commutative, so only the
    grouping matters)."""
    N = len(xs)
    out = xs[0].copy()
    for c, (s, n, _, _) in enumerate(orc.chunkize(xs[0].size, xs[0].itemsize, N)):
        acc = xs[c][s:s + n]
        for j in range(1, N):
            acc = add(acc, xs[(c + j) % N][s:s + n])
        out[s:s + n] = acc
    return out


def expected_butterfly(xs, add):
    """Chunk R is reduced at rank R: own data first, then peers in ascending
    rank order (AllreduceAlgos.cpp:155-180)."""
    N = len(xs)
    out = xs[0].copy()
    for R, (s, n, _, _) in enumerate(orc.chunkize(xs[0].size, xs[0].itemsize, N)):
        acc = xs[R][s:s + n]
        for p in range(N):
            if p != R:
                acc = add(acc, xs[p][s:s + n])
        out[s:s + n] = acc
    return out


def expected_tree(xs, add):
    """Binomial tree (AllreduceAlgos.cpp:100-114): value(r, span) =
    ((x_r + value(r+1)) + value(r+2)) + value(r+4) ... for children inside
    the world."""
    N = len(xs)

    def value(r, limit):
        acc = xs[r]
        m = 1
        while m < limit and r + m < N:
            if r & m:
                break
            acc = add(acc, value(r + m, m))
            m <<= 1
        return acc

    top = 1
    while top < N:
        top <<= 1
    return value(0, top)


EXPECT = {RING: expected_ring, BUTTERFLY: expected_butterfly, TREE: expected_tree}


def rand_inputs(world, numel, seed, dtype):
    rng = np.random.default_rng(seed)
    xs = [rng.standard_normal(numel).astype(np.float32) * np.float32(10.0 ** rng.integers(-3, 3))
          for _ in range(world)]
    if dtype == BF16:
        xs = [orc.encode_bf16(x) for x in xs]
    return xs


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
@pytest.mark.parametrize("world", [2, 3, 4, 5, 7, 8])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_fold_order(algo, world, dtype):
    numel = 1237  # ragged for every world above
    xs = rand_inputs(world, numel, 100 * world + algo, dtype)
    want = EXPECT[algo](xs, f32add if dtype == F32 else bf16add)
    bufs = [x.copy() for x in xs]
    assert orc.allreduce(algo, bufs, dtype, SUM) == 0
    for r in range(world):
        assert np.array_equal(bufs[r], want), (algo, world, r)
    # the three orders genuinely differ for world >= 3 on random data, so a
    # swapped schedule cannot pass by accident
    if world >= 4:
        others = [EXPECT[a](xs, f32add if dtype == F32 else bf16add) for a in EXPECT if a != algo]
        assert any(not np.array_equal(o, want) for o in others)


def test_tree_shapes_written_out():
    xs = rand_inputs(4, 64, 5, F32)
    a = f32add
    bufs = [x.copy() for x in xs]
    orc.allreduce(TREE, bufs, F32, SUM)
    assert np.array_equal(bufs[3], a(a(xs[0], xs[1]), a(xs[2], xs[3])))   # N=4: (x0+x1)+(x2+x3)
    xs = rand_inputs(3, 64, 6, F32)
    bufs = [x.copy() for x in xs]
    orc.allreduce(TREE, bufs, F32, SUM)
    assert np.array_equal(bufs[2], a(a(xs[0], xs[1]), xs[2]))             # N=3: (x0+x1)+x2
    xs = rand_inputs(6, 64, 7, F32)
    bufs = [x.copy() for x in xs]
    orc.allreduce(TREE, bufs, F32, SUM)
    want = a(a(a(xs[0], xs[1]), a(xs[2], xs[3])), a(xs[4], xs[5]))
    assert np.array_equal(bufs[5], want)


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
def test_two_ranks_all_algorithms_coincide(algo):
    xs = rand_inputs(2, 1001, 3, F32)
    bufs = [x.copy() for x in xs]
    orc.allreduce(algo, bufs, F32, SUM)
    assert np.array_equal(bufs[0], xs[0] + xs[1]) and np.array_equal(bufs[1], bufs[0])


@pytest.mark.parametrize("algo", [RING, TREE, BUTTERFLY])
@pytest.mark.parametrize("world", [2, 3, 5, 8])
def test_exact_integer_sums_and_reference_vectors(algo, world):
    # small integers add exactly in any order: a dropped or doubled chunk shows
    rng = np.random.default_rng(world)
    xs = [rng.integers(-1000, 1000, 4099).astype(np.float32) for _ in range(world)]
    bufs = [x.copy() for x in xs]
    assert orc.allreduce(algo, bufs, F32, SUM) == 0
    want = np.sum(np.stack(xs).astype(np.int64), 0)
    for b in bufs:
        assert np.array_equal(b.astype(np.int64), want)
    # tests/collectives/test_allreduce.py:11-28 -- 128 elements of value rank+1
    for dtype, enc in ((F32, lambda v: v), (BF16, orc.encode_bf16),
                       (F16, lambda v: v.astype(np.float16).view(np.uint16))):
        for op, fn in ((SUM, np.sum), (MIN, np.min), (MAX, np.max), (PRODUCT, np.prod)):
            bufs = [enc(np.full(128, r + 1.0, dtype=np.float32)) for r in range(world)]
            assert orc.allreduce(algo, bufs, dtype, op) == 0
            want = enc(np.full(128, fn(np.arange(1.0, world + 1)), dtype=np.float32))
            for b in bufs:
                assert np.array_equal(b, want), (dtype, op)
        bufs = [enc(np.full(128, r + 1.0, dtype=np.float32)) for r in range(world)]
        orc.allreduce(algo, bufs, dtype, AVG)
        got = bufs[0].astype(np.float64) if dtype == F32 else (
            orc.decode_bf16(bufs[0]) if dtype == BF16 else bufs[0].view(np.float16).astype(np.float64))
        assert np.allclose(got, (world + 1) / 2, rtol=1e-2, atol=1e-2)  # tests/common.py:53-56


@pytest.mark.parametrize("n", [1, 3, 7, 33, 997, 13])
def test_three_rank_sum_avg(n):  # tests/test_process_group_local.py:162-207,250-315
    for algo in (RING, TREE, BUTTERFLY):
        if algo != TREE and n < 3:
            bufs = [np.full(n, r + 1.0, np.float32) for r in range(3)]
            assert orc.allreduce(algo, bufs, F32, SUM) == -1  # AllreduceAlgos.cpp:55,137
            continue
        bufs = [np.full(n, r + 1.0, np.float32) for r in range(3)]
        orc.allreduce(algo, bufs, F32, SUM)
        assert all(np.array_equal(b, np.full(n, 6.0, np.float32)) for b in bufs)
        bufs = [np.full(n, r + 1.0, np.float32) for r in range(3)]
        orc.allreduce(algo, bufs, F32, AVG)
        assert all(np.allclose(b, 2.0, rtol=1e-6) for b in bufs)


# ---- ProcessGroup-level logic ---------------------------------------------

def test_select_algo():  # ProcessGroupMCCL.cpp:134-145
    S = orc.select_algo
    assert S(None, None, 262144, 65536, 3) == TREE       # inclusive threshold
    assert S(None, None, 262145, 65537, 3) == RING
    assert S("auto", None, 65536, 16384, 3) == TREE
    assert S("auto", 0, 8, 2, 2) == RING                 # MCCL_TREE_BELOW=0
    assert S("auto", 1 << 30, 1 << 26, 1 << 24, 4) == TREE
    assert S("ring", None, 8, 2, 3) == TREE              # numel < world
    assert S("ring", None, 12, 3, 3) == RING
    assert S("butterfly", None, 8, 2, 3) == TREE
    assert S("butterfly", None, 12, 3, 3) == BUTTERFLY
    assert S("tree", None, 1 << 30, 1 << 28, 4) == TREE
    assert S("bogus", None, 1 << 30, 1 << 28, 4) == TREE  # :173-176 else branch


@pytest.mark.parametrize("algo_name,algo", [("ring", RING), ("butterfly", BUTTERFLY), ("tree", TREE)])
@pytest.mark.parametrize("op", [SUM, AVG])
def test_wire_bf16_allreduce_recipe(algo_name, algo, op):
    """fp32 in, bf16 wire: every operand (own included) is encoded, every step
    rounds, AVG multiplies by the truncated constant, output is the decode."""
    world, numel = 3, 1000
    xs = rand_inputs(world, numel, 42, F32)
    bufs = [x.copy() for x in xs]
    rc, used = orc.pg_allreduce(bufs, F32, op, wire_bf16=True, env_algo=algo_name)
    assert rc == 0 and used == algo
    hs = [orc.encode_bf16(x) for x in xs]
    want = EXPECT[algo](hs, bf16add)
    if op == AVG:
        s = np.array([0x3EAA], dtype=np.uint16)
        want = orc.encode_bf16(orc.decode_bf16(want) * orc.decode_bf16(s)[0])
    for b in bufs:
        assert np.array_equal(b.view(np.uint32), orc.decode_bf16(want).view(np.uint32))
    # without the wire flag the same call is plain fp32
    bufs = [x.copy() for x in xs]
    orc.pg_allreduce(bufs, F32, SUM, wire_bf16=False, env_algo=algo_name)
    assert np.array_equal(bufs[0], EXPECT[algo](xs, f32add))


def test_auto_threshold_uses_wire_bytes():
    xs = rand_inputs(3, 100000, 1, F32)            # 400000 B fp32, 200000 B bf16
    bufs = [x.copy() for x in xs]
    assert orc.pg_allreduce(bufs, F32, SUM, wire_bf16=False)[1] == RING
    bufs = [x.copy() for x in xs]
    assert orc.pg_allreduce(bufs, F32, SUM, wire_bf16=True)[1] == TREE
    bufs = [x.copy() for x in xs]
    assert orc.pg_allreduce(bufs, F32, SUM, wire_bf16=True, tree_below=1000)[1] == RING


@pytest.mark.parametrize("world", [2, 3, 8])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_reduce_scatter_and_allgather(world, dtype):
    CH = 32  # tests/collectives/test_reduce_scatter.py:14-21: value (p+1)*10+rank
    enc = (lambda v: v) if dtype == F32 else orc.encode_bf16
    ins = [enc(np.concatenate([np.full(CH, (p + 1) * 10.0 + r, np.float32) for p in range(world)]))
           for r in range(world)]
    for op, fn in ((SUM, np.sum), (MIN, np.min), (MAX, np.max)):
        outs = [np.zeros(CH, dtype=ins[0].dtype) for _ in range(world)]
        assert orc.reduce_scatter(outs, ins, dtype, op) == 0
        for r in range(world):
            exact = fn([(r + 1) * 10.0 + q for q in range(world)])
            if dtype == F32 or op != SUM:
                assert np.array_equal(outs[r], enc(np.full(CH, exact, np.float32)))
            else:  # bf16 rounds after every step: the reference's own tolerance (tests/common.py:53-56)
                assert np.allclose(orc.decode_bf16(outs[r]), exact, rtol=1e-2, atol=1e-2)
    # random data: own share first, then ascending peers; AVG uses the RNE constant
    rng = np.random.default_rng(world)
    ins = [enc(rng.standard_normal(CH * world).astype(np.float32)) for _ in range(world)]
    outs = [np.zeros(CH, dtype=ins[0].dtype) for _ in range(world)]
    orc.reduce_scatter(outs, ins, dtype, AVG)
    add = f32add if dtype == F32 else bf16add
    for r in range(world):
        acc = ins[r][r * CH:(r + 1) * CH]
        for p in range(world):
            if p != r:
                acc = add(acc, ins[p][r * CH:(r + 1) * CH])
        if dtype == F32:
            acc = acc * np.float32(1.0 / world)
        else:
            s = orc.decode_bf16(orc.encode_bf16(np.array([np.float32(1.0 / world)])))[0]
            acc = orc.encode_bf16(orc.decode_bf16(acc) * s)
        assert np.array_equal(outs[r], acc)
    # allgather: concatenation by rank (tests/collectives/allgather.py)
    gouts = [np.zeros(CH * world, dtype=ins[0].dtype) for _ in range(world)]
    orc.allgather(gouts, outs)
    for g in gouts:
        assert np.array_equal(g, np.concatenate(outs))


def test_wire_fold_chunk_equals_full_allreduce():
    world, numel = 3, 1000
    xs = rand_inputs(world, numel, 8, F32)
    hs = [orc.encode_bf16(x) for x in xs]
    bufs = [x.copy() for x in xs]
    orc.pg_allreduce(bufs, F32, AVG, wire_bf16=True, env_algo="butterfly")
    for R, (s, n, _, _) in enumerate(orc.chunkize(numel, 2, world)):
        peers = [np.ascontiguousarray(hs[p][s:s + n]) for p in range(world) if p != R]
        out = orc.wire_fold_chunk(np.ascontiguousarray(xs[R][s:s + n]), peers, scale_by=1.0 / world)
        assert np.array_equal(out.view(np.uint32), bufs[0][s:s + n].view(np.uint32))
    bufs = [x.copy() for x in xs]
    orc.pg_allreduce(bufs, F32, SUM, wire_bf16=True, env_algo="ring")
    for c, (s, n, _, _) in enumerate(orc.chunkize(numel, 2, world)):
        owner = (c - 1) % world
        order = [(c + j) % world for j in range(world)]
        assert order[-1] == owner
        peers = [np.ascontiguousarray(hs[p][s:s + n]) for p in order[:-1]]
        out = orc.wire_fold_chunk(np.ascontiguousarray(xs[owner][s:s + n]), peers, own_last=True)
        assert np.array_equal(out.view(np.uint32), bufs[0][s:s + n].view(np.uint32))


def test_reference_progress_engine_order():
    R = orc.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    order = (C.c_int * 100)()
    assert R.ref_progress_order(100, 0, order) == 100 and list(order) == list(range(100))
    assert R.ref_progress_order(3, 0b001, order) == 2 and list(order[:2]) == [1, 2]
