"""Seeded random parity runs on the GPU: plans, segment shapes, alignments and
schedules drawn at random and checked bit for bit against the oracle -- the
combinations the hand-written cases do not enumerate (a fold plan has six
parameters, a segment five pointers with their own misalignment, a replay a
world size, an algorithm, an op, a dtype, a wire codec and a mode)."""
import ctypes as C
import datetime
import threading

import numpy as np
import pytest
import torch
import torch.distributed as dist

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, AVG, MIN, MAX, PRODUCT, RING, TREE, BUTTERFLY

pytestmark = pytest.mark.gpu

ES = {F32: 4, F16: 2, BF16: 2}
OPS = {SUM: dist.ReduceOp.SUM, AVG: dist.ReduceOp.AVG, MIN: dist.ReduceOp.MIN, MAX: dist.ReduceOp.MAX,
       PRODUCT: dist.ReduceOp.PRODUCT}
TIMEOUT = datetime.timedelta(seconds=30)
NAMES = {RING: "ring", TREE: "tree", BUTTERFLY: "butterfly"}


@pytest.fixture(scope="module")
def env():
    from mccl_amd import kernels, harness, _lib
    import gpu_util
    kernels.hip_kernels_init(0)
    return kernels, harness, _lib, gpu_util


def chain(ops, dtype, op, binomial, acc_is_src):
    v = [x.copy() for x in ops]
    k = len(v)
    if not binomial or k < 4:
        acc = v[0]
        for j in range(1, k):
            if acc_is_src:
                d = v[j].copy(); orc.reduce(d, acc, dtype, op); acc = d
            else:
                orc.reduce(acc, v[j], dtype, op)
        return acc
    mask = 1
    while mask < k:
        for r in range(0, k - mask, 2 * mask):
            orc.reduce(v[r], v[r + mask], dtype, op)
        mask <<= 1
    return v[0]


def fold_case(case, rng, K, L, U):
    dtype = int(rng.choice([F32, BF16, BF16, F16]))
    io = L.IO_PURE if dtype != BF16 else int(rng.choice([L.IO_PURE, L.IO_OUT_F32, L.IO_OWN_FIRST_F32, L.IO_OWN_LAST_F32]))
    k = int(rng.integers(1, 9))
    op = SUM if io != L.IO_PURE else int(rng.choice([SUM, SUM, MIN, MAX, PRODUCT]))
    binomial = bool(rng.integers(0, 2)) and io != L.IO_OWN_LAST_F32
    flags = L.PLAN_ACC_IS_SRC if (rng.integers(0, 3) == 0 and not (binomial and k >= 4)) else 0
    scale_mode = int(rng.choice([L.SCALE_NONE, L.SCALE_VIEW, L.SCALE_TENSOR]))
    scale = float(rng.choice([1 / 3, 0.5, 1 / 7, 0.125]))
    shape = int(rng.integers(0, 4))
    nseg = [1, int(rng.integers(2, 5)), int(rng.integers(5, 33)), int(rng.integers(33, 120))][shape]
    big = [200000, 60000, 9000, 3000][shape]
    out_f32 = dtype == F32 or io != L.IO_PURE
    want_wire = dtype != F32 and io != L.IO_PURE and bool(rng.integers(0, 2))
    segs, keep, checks = [], [], []
    uniform = bool(rng.integers(0, 3) == 0)
    n0 = int(rng.integers(0, big))
    for s in range(nseg):
        n = n0 if uniform else int(rng.choice([0, 1, int(rng.integers(1, 70)), int(rng.integers(1, big))], p=[.05, .05, .2, .7]))
        ins_np, ins_dev, ptrs = [], [], []
        for j in range(k):
            f32_in = dtype == F32 or (io == L.IO_OWN_FIRST_F32 and j == 0) or (io == L.IO_OWN_LAST_F32 and j == k - 1)
            dt = F32 if f32_in else dtype
            off = int(rng.integers(0, 9))
            a = U.rand_values(rng, n + off + 8, dt, scale=10.0 ** int(rng.integers(-3, 2)), specials=(dt != F16))
            if dt == F16 and a.size >= 16:      # zeros of both signs, denormals
                idx = rng.choice(a.size, size=a.size // 8, replace=False)
                a[idx] = np.resize(np.array([0, 0x8000, 1, 0x8001, 0x03FF, 0x83FF, 0x3C00, 0xBC00], dtype=np.uint16), idx.size)
            t = U.to_dev(a, dt)
            ins_np.append((a[off:off + n], dt)); ins_dev.append(t)
            ptrs.append(t.data_ptr() + off * ES[dt])
        # expected
        ops = [orc.encode_bf16(a) if (dt == F32 and dtype == BF16) else a.copy() for a, dt in ins_np]
        if n:
            res = chain(ops, dtype, op, binomial, bool(flags))
            if scale_mode != L.SCALE_NONE:
                orc.scale(res, dtype, scale, orc.SCALE_VIEW if scale_mode == L.SCALE_VIEW else orc.SCALE_TENSOR)
        else:
            res = ops[0][:0]
        want_out = orc.decode_bf16(res) if (out_f32 and dtype == BF16) else res
        odt = F32 if out_f32 else dtype
        ooff = int(rng.integers(0, 9))
        inplace = rng.integers(0, 4) == 0 and n > 0
        target = None
        if inplace:   # over an operand of the output's dtype
            cand = [j for j, (a, dt) in enumerate(ins_np) if dt == odt]
            if cand:
                target = int(rng.choice(cand))
        if target is not None:
            out_t, out_ptr, ooff_e = ins_dev[target], ptrs[target], (ptrs[target] - ins_dev[target].data_ptr()) // ES[odt]
        else:
            out_t = torch.full((n + ooff + 8,), 7.0, dtype=U.TORCH_DT[odt], device="cuda")
            out_ptr, ooff_e = out_t.data_ptr() + ooff * ES[odt], ooff
        wire_t = wire_ptr = None
        if want_wire:
            woff = int(rng.integers(0, 9))
            wire_t = torch.full((n + woff + 8,), 5.0, dtype=torch.bfloat16, device="cuda")
            wire_ptr = wire_t.data_ptr() + woff * 2
            checks.append((wire_t, woff, n, res, BF16, f"seg {s} wire"))
        checks.append((out_t, ooff_e, n, want_out, odt, f"seg {s} out"))
        segs.append(K.make_seg(out_ptr, wire_ptr or 0, ptrs, n))
        keep.append((ins_dev, out_t, wire_t))
    plan = K.make_plan(dtype, k, io=io, topo=L.TOPO_BINOMIAL if binomial else L.TOPO_FOLD, op=op,
                       scale_mode=scale_mode, scale=scale, flags=flags)
    desc = f"case {case}: dtype {dtype} io {io} k {k} op {op} binom {binomial} flags {flags} scale {scale_mode}/{scale:.4f} nseg {nseg} uniform {uniform} wire {want_wire}"
    q = K._q(None)
    arr = (L.Seg * len(segs))(*segs)
    noalloc = nseg <= L.NOALLOC_MAX_SEGS and rng.integers(0, 3) == 0
    fn = L.lib().mcclx_fold_batched_noalloc if noalloc else L.lib().mcclx_fold_batched
    torch.cuda.synchronize()
    L.check(fn(q.handle, C.byref(plan), arr, len(segs)))
    K.hip_sync()
    for t, off, n, want, dt, what in checks:
        got = t[off:off + n]
        U.assert_same_bits(got, want, dt, desc + " " + what + (" noalloc" if noalloc else ""))


def values(rng, U, n, dtype):
    a = U.rand_values(rng, n, dtype, scale=10.0 ** int(rng.integers(-3, 1 if dtype == F16 else 2)), specials=(dtype != F16 and rng.integers(0, 2) == 0))
    if n >= 8 and rng.integers(0, 2) == 0:       # zeros of both signs, ties
        idx = rng.choice(n, size=max(1, n // 6), replace=False)
        if dtype == F32:
            a[idx] = np.resize(np.array([0.0, -0.0, 1.0, -1.0], dtype=np.float32), idx.size)
        elif dtype == BF16:
            a[idx] = np.resize(np.array([0, 0x8000, 0x3F80, 0xBF80], dtype=np.uint16), idx.size)
        else:
            a[idx] = np.resize(np.array([0, 0x8000, 0x3C00, 0xBC00, 1, 0x8001], dtype=np.uint16), idx.size)
    return a


def check(U, d, want, dtype, what):
    for r in range(len(d)):
        if dtype == F16:
            assert np.array_equal(U.bits(d[r]), want[r]), what + f" rank {r}"
        else:
            U.assert_same_bits(d[r], want[r], dtype, what + f" rank {r}")


def numel_for(rng, world, algo):
    n = int(rng.choice([1, world, world + 1, int(rng.integers(1, 200)), int(rng.integers(200, 70000)), int(rng.integers(70000, 400000))],
                       p=[.05, .1, .1, .25, .4, .1]))
    if algo != TREE:
        n = max(n, world)
    return n


def allreduce_case(case, rng, H, U):
    algo = int(rng.choice([RING, TREE, BUTTERFLY]))
    world = int(rng.choice([2, 3, 4, 5, 7, 8, 9, 12, 17]))
    dtype, wire = [(F32, False), (BF16, False), (F16, False), (F32, True)][int(rng.integers(0, 4))]
    op = int(rng.choice([SUM, AVG, MIN, MAX, PRODUCT]))
    mode = int(rng.integers(0, 2))
    if mode == 1 and case % 2:   # FUSED, or DIRECT (over the wire codec: the ranks' fp32 tensors read in place)
        mode = 2
    many = rng.integers(0, 3) == 0
    groups = int(rng.integers(2, 7)) if many else 1
    desc = f"case {case}: allreduce algo {NAMES[algo]} world {world} dtype {dtype} wire {wire} op {op} mode {mode} groups {groups}"
    xs, wants, ds = [], [], []
    for g in range(groups):
        n = numel_for(rng, world, algo)
        x = [values(rng, U, n, dtype) for _ in range(world)]
        w = [a.copy() for a in x]
        rc = orc.allreduce(algo, w, dtype, op) if not wire else orc.pg_allreduce(w, dtype, op, wire_bf16=True, env_algo=NAMES[algo])[0]
        assert rc == 0
        xs.append(x); wants.append(w); ds.append([U.to_dev(a, dtype) for a in x])
        desc += f" n{g}={n}"
    if many:
        H.allreduce_replay_many(ds, op, algo, wire_bf16=wire, mode=mode)
    else:
        H.allreduce_replay(ds[0], op, algo, wire_bf16=wire, mode=mode)
    for g in range(groups):
        check(U, ds[g], wants[g], dtype, desc + f" group {g}")


def reduce_scatter_case(case, rng, K, H, U):
    world = int(rng.choice([2, 3, 4, 8, 9, 16]))
    dtype = int(rng.choice([F32, BF16, F16]))
    op = int(rng.choice([SUM, AVG, MIN, MAX, PRODUCT]))
    mode = int(rng.integers(0, 2))
    chunk = int(rng.choice([1, int(rng.integers(1, 100)), int(rng.integers(100, 50000))]))
    desc = f"case {case}: reduce_scatter world {world} dtype {dtype} op {op} mode {mode} chunk {chunk}"
    ins = [values(rng, U, chunk * world, dtype) for _ in range(world)]
    outs = [np.zeros(chunk, dtype=ins[0].dtype) for _ in range(world)]
    assert orc.reduce_scatter(outs, ins, dtype, op) == 0
    din = [U.to_dev(a, dtype) for a in ins]
    dout = [torch.empty(chunk, dtype=U.TORCH_DT[dtype], device="cuda") for _ in range(world)]
    H.reduce_scatter_replay(dout, din, op, mode=mode)
    check(U, dout, outs, dtype, desc)
    # allgather of the results
    gout = [torch.empty(chunk * world, dtype=U.TORCH_DT[dtype], device="cuda") for _ in range(world)]
    H.allgather_replay(gout, dout)
    K.hip_sync()
    cat = np.concatenate([U.bits(o) for o in dout])   # the device's own results (NaN payloads are the GPU's)
    for r in range(world):
        assert np.array_equal(U.bits(gout[r]), cat), desc + f" allgather rank {r}"


def run_ranks(CX, world, fn):
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
        t.join(90)
    assert not any(t.is_alive() for t in ts), "a rank thread hung"
    return out, errs


def collective_mix_case(case, rng, monkeypatch, CX, U):
    world = int(rng.choice([2, 3, 4]))
    dtype = int(rng.choice([F32, BF16]))
    asyn = bool(rng.integers(0, 4))
    queues = str(int(rng.integers(1, 3)))
    chunk = int(rng.choice([int(rng.integers(1, 50)), int(rng.integers(50, 60000))]))
    n = chunk * world
    ntens = 3
    steps = []
    for _ in range(int(rng.integers(3, 10))):
        kind = int(rng.choice([0, 0, 0, 1, 2, 3]))
        steps.append((kind, int(rng.integers(0, ntens)), int(rng.integers(0, ntens)), int(rng.choice([SUM, MAX, MIN, AVG]))))
    wire = dtype == F32 and case % 2 == 1            # the bf16 wire codec on the allreduces ...
    direct = case % 4 != 3                           # ... whose fold reads the fp32 tensors itself, or bf16 copies
    desc = f"case {case}: world {world} dtype {dtype} async {asyn} queues {queues} chunk {chunk} wire {wire} direct {direct} steps {steps}"
    for k in ("MCCL_ALLREDUCE_ALGO", "MCCL_WIRE", "MCCL_ALLREDUCE_ASYNC", "MCCL_WIRE_DTYPE", "MCCL_DIRECT"):
        monkeypatch.delenv(k, raising=False)
    if wire:
        monkeypatch.setenv("MCCL_WIRE_DTYPE", "bf16")
    if not direct:
        monkeypatch.setenv("MCCL_DIRECT", "0")
    monkeypatch.setenv("MCCL_ASYNC_QUEUES", queues)
    if asyn:
        monkeypatch.setenv("MCCL_ALLREDUCE_ASYNC", "1")
    big = [[U.rand_values(rng, n, dtype, scale=1e-2) for _ in range(ntens)] for _ in range(world)]     # world*chunk tensors
    small = [[U.rand_values(rng, chunk, dtype, scale=1e-2) for _ in range(ntens)] for _ in range(world)]
    def fn(r, pg):
        B = [U.to_dev(x, dtype) for x in big[r]]
        S = [U.to_dev(x, dtype) for x in small[r]]
        works = []
        for kind, i, j, op in steps:
            o = dist.AllreduceOptions(); o.reduceOp = OPS[op]
            if kind == 0:
                works.append(pg.allreduce([B[i]], o))
            elif kind == 1:
                works.append(pg.allreduce([S[j], B[i]], o))
            elif kind == 2:
                ro = dist.ReduceScatterOptions(); ro.reduceOp = OPS[op]
                works.append(pg._reduce_scatter_base(S[j], B[i], ro))
            else:
                works.append(pg._allgather_base(B[i], S[j]))
        for w in works:
            w.wait()
        torch.cuda.current_stream().synchronize()
        return B, S
    out, errs = run_ranks(CX, world, fn)
    assert errs == [None] * world, (desc, errs)
    WB = [[big[r][t].copy() for r in range(world)] for t in range(ntens)]
    WS = [[small[r][t].copy() for r in range(world)] for t in range(ntens)]
    for kind, i, j, op in steps:
        if kind == 0:
            assert orc.pg_allreduce(WB[i], dtype, op, wire_bf16=wire)[0] == 0
        elif kind == 1:
            assert orc.pg_allreduce(WS[j], dtype, op, wire_bf16=wire)[0] == 0
            assert orc.pg_allreduce(WB[i], dtype, op, wire_bf16=wire)[0] == 0
        elif kind == 2:
            assert orc.reduce_scatter(WS[j], WB[i], dtype, op) == 0
        else:
            orc.allgather(WB[i], WS[j])
    for r in range(world):
        for t in range(ntens):
            U.assert_same_bits(out[r][0][t], WB[t][r], dtype, desc + f" big {t} rank {r}")
            U.assert_same_bits(out[r][1][t], WS[t][r], dtype, desc + f" small {t} rank {r}")


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_fold_plans_segments_and_alignments(env, seed):
    K, H, L, U = env
    rng = np.random.default_rng(seed)
    for case in range(150):
        fold_case(case, rng, K, L, U)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_schedules(env, seed):
    K, H, L, U = env
    rng = np.random.default_rng(seed)
    for case in range(150):
        if rng.integers(0, 4):
            allreduce_case(case, rng, H, U)
        else:
            reduce_scatter_case(case, rng, K, H, U)


@pytest.mark.parametrize("seed", [31, 32])
def test_random_mixes_of_collectives_on_shared_tensors_through_the_process_group(env, monkeypatch, seed):
    """allreduce (synchronous or event-based on one or two queues, single tensors and lists),
    reduce_scatter and allgather issued back to back on tensors they share, with no Work waited
    on before the end: every call must see the result of the calls before it."""
    from mccl_amd import _C as CX
    K, H, L, U = env
    rng = np.random.default_rng(seed)
    for case in range(60):
        collective_mix_case(case, rng, monkeypatch, CX, U)
