"""GPU parity of the hold form of the fold launches: all loads first, results kept in
registers, stores once the launch's reads are through (a time the host works out from the
bytes read).  Same bits as the plain form and as the oracle for every plan that has it, for
ragged, misaligned and in-place segments, for each of its block shapes, and whatever the gate."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16

pytestmark = pytest.mark.gpu

ES = {F32: 4, F16: 2, BF16: 2}
KINDS = ["f32", "out_f32", "own_first", "own_last", "all_f32", "bf16", "f16"]
PURE16 = {"bf16": BF16, "f16": F16}


@pytest.fixture(scope="module")
def env():
    from mccl_amd import _lib, kernels
    import gpu_util
    from test_gpu_fold import oracle_fold
    kernels.hip_kernels_init(0)
    return kernels, _lib, gpu_util, oracle_fold


def queue_with(K, **knobs):
    """A reduce queue made under the given environment knobs (they are read when it is made)."""
    old = {k: os.environ.get(k) for k in knobs}
    try:
        for k, v in knobs.items():
            os.environ[k] = str(v)
        return K.ReduceQueue(0)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


@pytest.fixture(scope="module")
def queues(env):
    K = env[0]
    held = queue_with(K, MCCLX_HOLD_MIN_BYTES=0)      # every launch that fits one generation holds
    plain = queue_with(K, MCCLX_HOLD=0)
    yield held, plain
    held.close()
    plain.close()


def io_of(L, kind):
    return {"f32": L.IO_PURE, "out_f32": L.IO_OUT_F32, "own_first": L.IO_OWN_FIRST_F32,
            "own_last": L.IO_OWN_LAST_F32, "all_f32": L.IO_ALL_F32, "bf16": L.IO_PURE, "f16": L.IO_PURE}[kind]


def in_dtype(kind, j, k):
    if kind in PURE16:
        return PURE16[kind]
    if kind in ("f32", "all_f32") or (kind == "own_first" and j == 0) or (kind == "own_last" and j == k - 1):
        return F32
    return BF16


def build_case(env, rng, kind, k, fan, counts, in_place=False):
    """Segments with misaligned operands; returns (plan, segs for a queue, checks, keep-alive)."""
    K, L, U, oracle_fold = env
    W = F32 if kind == "f32" else PURE16.get(kind, BF16)
    odt = PURE16.get(kind, F32)          # the form of the outputs
    segs, checks, keep = [], [], []
    for n in counts:
        ins, ptrs, dev = [], [], []
        for j in range(k):
            dt = in_dtype(kind, j, k)
            off = int(rng.integers(0, 5))
            a = U.rand_values(rng, n + off + 4, dt, scale=1e-2, specials=(dt != F16))
            t = U.to_dev(a, dt)
            ins.append((np.ascontiguousarray(a[off:off + n]), dt))
            dev.append(t)
            ptrs.append(t.data_ptr() + off * ES[dt])
        ops = [orc.encode_bf16(a) if (dt == F32 and W == BF16) else a.copy() for a, dt in ins]
        res = oracle_fold(ops, W, False, 1.0 / 3, orc.SCALE_VIEW)
        want = orc.decode_bf16(res) if (W == BF16 and odt == F32) else res
        outs = []
        for f in range(fan + 1):
            off = int(rng.integers(0, 5))
            t = torch.full((n + off + 4,), 3.0, dtype=U.TORCH_DT[odt], device="cuda")
            outs.append((t, off))
        if in_place:  # the result over an operand of the output's form
            j = next(j for j, (_, dt) in enumerate(ins) if dt == odt)
            outs[0] = (dev[j], (ptrs[j] - dev[j].data_ptr()) // ES[odt])
        dest = [t.data_ptr() + off * ES[odt] for t, off in outs]
        segs.append(K.make_seg(dest[0], 0, ptrs + dest[1:], n))
        checks.append((outs, n, want, odt))
        keep.append(dev)
    plan = K.make_plan(W, k, io=io_of(L, kind), scale_mode=L.SCALE_VIEW, scale=1.0 / 3, fanout=fan)
    return plan, segs, checks, keep


def check_outputs(U, checks, what, guards=True):
    for outs, n, want, odt in checks:
        for f, (t, off) in enumerate(outs):
            if odt == F16:
                assert np.array_equal(U.bits(t[off:off + n]), want), f"{what} destination {f}"
            else:
                U.assert_same_bits(t[off:off + n], want, odt, f"{what} destination {f}")
            if guards and t.numel() == n + off + 4 and float(t[:1].float().cpu()) == 3.0:
                assert torch.all(t[:off].float() == 3.0) and torch.all(t[off + n:].float() == 3.0), what + ": wrote outside its range"


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("k", [2, 3, 4])
def test_hold_form_gives_the_oracles_bits(env, queues, kind, k):
    """Every plan with a hold form, with and without fan-out, one and three segments, sizes
    from one element to a few hundred thousand, misaligned operands, in place."""
    K, L, U, _ = env
    held, plain = queues
    if kind == "out_f32" and k < 2:
        pytest.skip("no such plan")
    rng = np.random.default_rng(1000 + 10 * KINDS.index(kind) + k)
    fans = [0] if kind == "out_f32" else [0, min(2, 8 - k)]
    if kind == "f16":
        fans = [0, 1]
    for fan in fans:
        for counts in ([1], [7], [4099], [300_007], [33, 70_001, 5], [70_001, 0, 9], [120_000, 120_001, 119_999]):
            for in_place in ((False, True) if kind != "out_f32" and fan == 0 else (False,)):
                plan, segs, checks, keep = build_case(env, rng, kind, k, fan, counts, in_place)
                before = held.hold_launch_count()
                torch.cuda.synchronize()     # the buffers were filled on torch's stream
                held.fold(plan, segs)
                held.drain()
                assert held.hold_launch_count() == before + 1, "the launch did not take the hold form"
                check_outputs(U, checks, f"{kind} k={k} fan={fan} counts={counts} in_place={in_place}", guards=not in_place)
    assert plain.hold_launch_count() == 0


@pytest.mark.parametrize("kind,k,count", [("bf16", 3, 13_107_200),        # a 25 MiB bucket of bf16 gradients
                                          ("own_first", 3, 8_000_000),    # four packets per lane
                                          ("own_first", 3, 9_500_000),    # five
                                          ("all_f32", 3, 6_553_600),      # the one-launch allreduce of a 25 MiB bucket
                                          ("own_last", 4, 10_000_000),
                                          ("f32", 2, 7_000_003)])
def test_hold_form_block_shapes_against_the_plain_form(env, queues, kind, k, count):
    """Launches near what one generation holds, where more packets per lane take over: the
    same bits as the plain form of the same launch."""
    K, L, U, _ = env
    held, plain = queues
    g = torch.Generator(device="cuda").manual_seed(count % 1000 + k)
    W = F32 if kind == "f32" else PURE16.get(kind, BF16)
    odt = PURE16.get(kind, F32)
    ins = []
    for j in range(k):
        t = torch.randn(count + 3, device="cuda", generator=g) * 1e-2
        ins.append(t if in_dtype(kind, j, k) == F32 else t.to(U.TORCH_DT[in_dtype(kind, j, k)]))
    ptrs = [t.data_ptr() + ES[in_dtype(kind, j, k)] for j, t in enumerate(ins)]   # one element past the start
    plan = K.make_plan(W, k, io=io_of(L, kind), scale_mode=L.SCALE_VIEW, scale=1.0 / 3)
    got = []
    for q in (held, plain):
        out = torch.full((count + 2,), 7.0, dtype=U.TORCH_DT[odt], device="cuda")
        before = q.hold_launch_count()
        torch.cuda.synchronize()
        q.fold(plan, [K.make_seg(out.data_ptr() + ES[odt], 0, ptrs, count)])
        q.drain()
        assert q.hold_launch_count() == before + (1 if q is held else 0)
        assert float(out[0].float().cpu()) == 7.0 and float(out[-1].float().cpu()) == 7.0
        got.append(out)
    view = torch.int32 if odt == F32 else torch.int16
    assert torch.equal(got[0].view(view), got[1].view(view))


def test_a_launch_wider_than_one_generation_takes_the_plain_form(env, queues):
    K, L, U, _ = env
    held, _ = queues
    n = 20_000_000
    g = torch.Generator(device="cuda").manual_seed(4)
    own = torch.randn(n, device="cuda", generator=g) * 1e-2
    peers = [(torch.randn(n, device="cuda", generator=g) * 1e-2).to(torch.bfloat16) for _ in range(2)]
    out = torch.empty(n, device="cuda")
    plan = K.make_plan(BF16, 3, io=L.IO_OWN_FIRST_F32)
    before = held.hold_launch_count()
    torch.cuda.synchronize()
    held.fold(plan, [K.make_seg(out.data_ptr(), 0, [own.data_ptr()] + [p.data_ptr() for p in peers], n)])
    held.drain()
    assert held.hold_launch_count() == before
    want = (own.to(torch.bfloat16) + peers[0]) + peers[1]      # torch rounds after every add as well
    assert torch.equal(out, want.float())


def test_default_threshold_and_the_switch(env):
    """By default a launch holds from 10 MiB read on; mcclx_set_hold switches the form off and on."""
    K, L, U, _ = env
    q = queue_with(K)
    try:
        plan = K.make_plan(BF16, 3, io=L.IO_OWN_FIRST_F32, scale_mode=L.SCALE_VIEW, scale=1.0 / 3)

        def run(n):
            g = torch.Generator(device="cuda").manual_seed(n % 97)
            own = torch.randn(n, device="cuda", generator=g) * 1e-2
            peers = [(torch.randn(n, device="cuda", generator=g) * 1e-2).to(torch.bfloat16) for _ in range(2)]
            out = torch.empty(n, device="cuda")
            before = q.hold_launch_count()
            torch.cuda.synchronize()
            q.fold(plan, [K.make_seg(out.data_ptr(), 0, [own.data_ptr()] + [p.data_ptr() for p in peers], n)])
            q.drain()
            return q.hold_launch_count() - before, out

        assert run(262_144)[0] == 0            # 2 MiB read: the plain form
        took, a = run(2_184_534)               # one chunk of a 25 MiB bucket: 17.5 MB read
        assert took == 1
        q.set_hold(False)
        took, b = run(2_184_534)
        assert took == 0 and torch.equal(a.view(torch.int32), b.view(torch.int32))
        q.set_hold(True)
        assert run(2_184_534)[0] == 1
    finally:
        q.close()


@pytest.mark.parametrize("knobs", [dict(MCCLX_HOLD_BYTES_PER_TICK=1000),                  # a gate far too late (capped at 1 ms)
                                   dict(MCCLX_HOLD_BYTES_PER_TICK=1000000, MCCLX_HOLD_LATENCY_TICKS=0)])  # none to speak of
def test_results_do_not_depend_on_the_gate(env, queues, knobs):
    K, L, U, _ = env
    q = queue_with(K, MCCLX_HOLD_MIN_BYTES=0, **knobs)
    try:
        rng = np.random.default_rng(5)
        plan, segs, checks, keep = build_case(env, rng, "own_first", 3, 2, [200_003, 7, 65_536])
        before = q.hold_launch_count()
        torch.cuda.synchronize()
        q.fold(plan, segs)
        q.drain()
        assert q.hold_launch_count() == before + 1
        check_outputs(U, checks, f"gate knobs {knobs}")
    finally:
        q.close()


def test_the_gate_follows_the_device_and_the_knobs_override_it(monkeypatch):
    """The rate behind the hold form's gate is measured when the first context of the process
    is made (two read-only launches over scratch memory): on MI355X it lands near 70,000 bytes
    per 10 ns tick.  MCCLX_HOLD_BYTES_PER_TICK overrides it for contexts made afterwards, and
    MCCLX_HOLD_CALIBRATE=0 cannot undo a measurement already cached for the device."""
    from mccl_amd import kernels as K
    q = K.ReduceQueue(0)
    lat, bpt, measured = q.hold_model()
    q.close()
    assert measured and lat == 40 and 50_000 <= bpt <= 95_000, (lat, bpt, measured)
    monkeypatch.setenv("MCCLX_HOLD_BYTES_PER_TICK", "65432")
    q = K.ReduceQueue(0)
    assert q.hold_model() == (40, 65432, False)
    q.close()
    monkeypatch.delenv("MCCLX_HOLD_BYTES_PER_TICK")
    q = K.ReduceQueue(0)
    assert q.hold_model() == (lat, bpt, True), "one measurement per device and process"
    q.close()


def test_the_wire_encode_has_a_hold_form_too(env, queues):
    """fp32 -> bf16 of whole tensors (the first launch of every schedule that sends bf16 copies):
    reads first, results kept in registers, stores behind the gate -- from three tensors on (on one
    or two the plain form is as fast or faster).  Bit for bit the oracle's round-to-nearest-even,
    specials included, on ragged, misaligned segments; the size threshold is off in this queue."""
    K, L, U, _ = env
    held, plain = queues
    rng = np.random.default_rng(9)
    plan = K.make_plan(BF16, 1, io=L.IO_OWN_FIRST_F32)
    for counts, takes in (([1], False), ([6_000_001], False), ([300_001, 299_999], False), ([70_003, 5, 123_457], True),
                          ([2_000_003, 1_500_001, 1_999_999], True), ([1_200_001] * 5 + [7], True)):
        segs, want, outs = [], [], []
        for n in counts:
            off_i, off_o = int(rng.integers(0, 5)), int(rng.integers(0, 5))
            a = U.rand_values(rng, n + off_i + 4, F32, scale=1e-2, specials=True)
            t = U.to_dev(a, F32)
            o = torch.full((n + off_o + 4,), 3.0, dtype=torch.bfloat16, device="cuda")
            segs.append(K.make_seg(0, o.data_ptr() + 2 * off_o, [t.data_ptr() + 4 * off_i], n))
            want.append(orc.encode_bf16(np.ascontiguousarray(a[off_i:off_i + n])))
            outs.append((o, off_o, n, t))
        torch.cuda.synchronize()
        before = held.hold_launch_count()
        held.fold(plan, segs)
        held.drain()
        assert held.hold_launch_count() == before + int(takes), f"encode of {counts}: hold form {'not ' if takes else ''}taken"
        for (o, off, n, _), w in zip(outs, want):
            assert np.array_equal(U.bits(o[off:off + n]), w), f"encode, hold form, counts {counts}"
            assert torch.all(o[:off].float() == 3.0) and torch.all(o[off + n:].float() == 3.0), "wrote outside its range"


@pytest.mark.parametrize("with_out,with_wire,scaled", [(True, False, False), (True, True, True), (False, True, True), (True, True, False)])
def test_one_operand_plans_in_the_hold_form_match_the_plain_form(env, queues, with_out, with_wire, scaled):
    """The encode's plan (one fp32 operand, rounded to bf16) with any of its outputs -- the fp32
    form of the rounded value, the bf16 form, both -- and with a scale: the hold form writes what
    the plain form writes, bit for bit, and nothing outside, on ragged segments that include an
    empty one and one shorter than the head peel."""
    K, L, U, _ = env
    held, plain = queues
    rng = np.random.default_rng(77 + 4 * with_out + 2 * with_wire + scaled)
    plan = K.make_plan(BF16, 1, io=L.IO_OWN_FIRST_F32, scale_mode=L.SCALE_VIEW if scaled else L.SCALE_NONE, scale=1.0 / 3)
    for counts in ([70_003, 0, 123_457], [3, 500_001, 17, 250_000], [1_000_003] * 3):
        ins = []
        for n in counts:
            off = int(rng.integers(0, 5))
            a = U.rand_values(rng, n + off + 4, F32, scale=1e-2, specials=True)
            ins.append((U.to_dev(a, F32), off, n))
        got = []
        for q in (held, plain):
            outs, segs = [], []
            for t, off, n in ins:
                oo, ow = int(rng.integers(0, 5)), int(rng.integers(0, 5))
                o = torch.full((n + oo + 4,), 3.0, device="cuda") if with_out else None
                w = torch.full((n + ow + 4,), 3.0, dtype=torch.bfloat16, device="cuda") if with_wire else None
                segs.append(K.make_seg(o.data_ptr() + 4 * oo if with_out else 0, w.data_ptr() + 2 * ow if with_wire else 0,
                                       [t.data_ptr() + 4 * off], n))
                outs.append((o, oo, w, ow, n))
            torch.cuda.synchronize()
            before = q.hold_launch_count()
            q.fold(plan, segs)
            q.drain()
            assert q.hold_launch_count() == before + (1 if q is held else 0)
            for o, oo, w, ow, n in outs:
                if with_out:
                    assert torch.all(o[:oo] == 3.0) and torch.all(o[oo + n:] == 3.0), "wrote outside its range"
                if with_wire:
                    assert torch.all(w[:ow].float() == 3.0) and torch.all(w[ow + n:].float() == 3.0), "wrote outside its range"
            got.append([(o[oo:oo + n].clone() if with_out else None, w[ow:ow + n].clone() if with_wire else None) for o, oo, w, ow, n in outs])
        for (ho, hw), (po, pw) in zip(*got):
            if with_out:
                assert torch.equal(ho.view(torch.int32), po.view(torch.int32)), f"fp32 output, counts {counts}"
            if with_wire:
                assert torch.equal(hw.view(torch.int16), pw.view(torch.int16)), f"bf16 output, counts {counts}"
