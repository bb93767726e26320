"""Randomised parity of mcclx_fold_batched against the oracle: random plans (dtype, io
mode, k, topology, op, scale constant), 1..70 segments per launch with random lengths
(empty ones included) and element-granular offsets of every stream, outputs checked
bit for bit including the untouched bytes around every segment.  MCCLX_FUZZ_ROUNDS
raises the number of launches (default 60, a few seconds)."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM

pytestmark = pytest.mark.gpu

ROUNDS = int(os.environ.get("MCCLX_FUZZ_ROUNDS", "60"))


@pytest.fixture(scope="module")
def K():
    from mccl_amd import kernels
    kernels.hip_kernels_init(0)
    return kernels


@pytest.fixture(scope="module")
def U():
    import gpu_util
    return gpu_util


def fold_chain(v, dtype, op, binomial):
    v = [x.copy() for x in v]
    k = len(v)
    if not binomial:
        for j in range(1, k):
            orc.reduce(v[0], v[j], dtype, op)
    else:
        mask = 1
        while mask < k:
            for r in range(0, k - mask, 2 * mask):
                orc.reduce(v[r], v[r + mask], dtype, op)
            mask <<= 1
    return v[0]


def random_plan(rng, L):
    """A plan the library supports, as (dtype, io, k, binomial, op, scale, scale_mode)."""
    kind = rng.integers(0, 4)
    k = int(rng.integers(1, 9))
    binomial = bool(rng.integers(0, 2))
    scale, mode = None, L.SCALE_NONE
    if kind == 0:      # plain SUM in fp32 or bf16, maybe scaled
        dtype, io, op = (F32, BF16)[rng.integers(0, 2)], L.IO_PURE, SUM
    elif kind == 1:    # MIN / MAX / PRODUCT, or fp16
        dtype, io = (F32, F16, BF16)[rng.integers(0, 3)], L.IO_PURE
        op = (orc.MIN, orc.MAX, orc.PRODUCT, SUM)[rng.integers(0, 4 if dtype == F16 else 3)]
        k = max(k, 2)
    else:              # bf16 wire codec around fp32 tensors
        dtype, op = BF16, SUM
        io = (L.IO_OUT_F32, L.IO_OWN_FIRST_F32, L.IO_OWN_LAST_F32)[rng.integers(0, 3)]
        if io == L.IO_OWN_LAST_F32:
            binomial = False
    if op == SUM and dtype != F16 and rng.integers(0, 2):
        scale = 1.0 / float(rng.integers(2, 9))
        mode = (L.SCALE_VIEW, L.SCALE_TENSOR)[rng.integers(0, 2)]
    return dtype, io, k, binomial, op, scale, mode


def test_random_plans_segments_and_offsets(K, U):
    from mccl_amd import _lib as L
    rng = np.random.default_rng(20240611)
    q = K._q(None)
    GUARD = 70   # elements kept free on both sides of every stream's range
    for rnd in range(ROUNDS):
        dtype, io, k, binomial, op, scale, mode = random_plan(rng, L)
        nseg = int(rng.choice([1, 2, 3, 8, 9, 17, 32, 33, 40, 70]))
        big = rnd % 10 == 0
        counts = [int(c) for c in rng.choice([0, 1, 3, 63, 64, 65, 511, 2047, 2048, 2049, 8191, 30011,
                                              262147 if big else 4099], size=nseg)]
        in_f32 = [dtype == F32 or (io == L.IO_OWN_FIRST_F32 and i == 0) or (io == L.IO_OWN_LAST_F32 and i == k - 1)
                  for i in range(k)]
        out_f32 = dtype == F32 or io != L.IO_PURE
        want_wire = dtype != F32 and io != L.IO_PURE and bool(rng.integers(0, 2))
        # one pool per stream; every segment gets its own slice at a random element offset
        stride = max(counts) + 2 * GUARD + 16
        host_in = [U.rand_values(rng, nseg * stride, F32 if in_f32[i] else dtype,
                                 scale=10.0 ** rng.integers(-3, 2), specials=(op == SUM)) for i in range(k)]
        dev_in = [U.to_dev(host_in[i], F32 if in_f32[i] else dtype) for i in range(k)]
        out = torch.full((nseg * stride,), 7.0, dtype=torch.float32 if out_f32 else U.TORCH_DT[dtype], device="cuda")
        wire = torch.full((nseg * stride,), 7.0, dtype=torch.bfloat16, device="cuda") if want_wire else None
        want_out = U.bits(out).copy()
        want_wire_bits = U.bits(wire).copy() if want_wire else None
        segs = []
        for s, n in enumerate(counts):
            offs = [s * stride + GUARD + int(rng.integers(0, 16)) for _ in range(k + 2)]
            ops = []
            for i in range(k):
                a = host_in[i][offs[i]:offs[i] + n]
                ops.append(orc.encode_bf16(np.ascontiguousarray(a)) if (in_f32[i] and dtype != F32) else a.copy())
            if n:
                acc = fold_chain(ops, dtype, op, binomial)
                if scale is not None:
                    orc.scale(acc, dtype, scale, orc.SCALE_VIEW if mode == L.SCALE_VIEW else orc.SCALE_TENSOR)
                if out_f32 and dtype != F32:
                    want_out[offs[k]:offs[k] + n] = orc.decode_bf16(acc).view(np.uint32)
                elif dtype == F32:
                    want_out[offs[k]:offs[k] + n] = acc.view(np.uint32)
                else:
                    want_out[offs[k]:offs[k] + n] = acc
                if want_wire:
                    want_wire_bits[offs[k + 1]:offs[k + 1] + n] = acc
            es_out = 4 if out_f32 else 2
            segs.append(K.make_seg(out.data_ptr() + es_out * offs[k],
                                   wire.data_ptr() + 2 * offs[k + 1] if want_wire else 0,
                                   [dev_in[i].data_ptr() + (4 if in_f32[i] else 2) * offs[i] for i in range(k)], n))
        plan = K.make_plan(dtype, k, io=io, op=op, topo=L.TOPO_BINOMIAL if binomial else L.TOPO_FOLD,
                           scale_mode=mode, scale=scale or 0.0)
        what = f"round {rnd}: dtype={dtype} io={io} k={k} binomial={binomial} op={op} scale={scale} mode={mode} nseg={nseg}"
        torch.cuda.synchronize()
        q.fold(plan, segs)
        q.drain()
        got = U.bits(out)
        bad = got != want_out
        if dtype == F32:   # fp32 arithmetic: the payload of a produced NaN is the hardware's
            gn, wn = np.isnan(got.view(np.float32)), np.isnan(want_out.view(np.float32))
            assert np.array_equal(gn, wn), what
            bad &= ~gn
        if dtype == F16:   # fp16 NaN payloads are the hardware's too; bf16 NaNs are canonical (0x7FC0)
            gn, wn = np.isnan(got.view(np.float16)), np.isnan(want_out.view(np.float16))
            assert np.array_equal(gn, wn), what
            bad &= ~gn
        if bad.any():
            i = int(np.flatnonzero(bad)[0])
            raise AssertionError(f"{what}: {int(bad.sum())} elements differ, first at {i}: "
                                 f"got {int(got[i]):#x} want {int(want_out[i]):#x}")
        if want_wire:
            assert np.array_equal(U.bits(wire), want_wire_bits), what + " (wire_out)"
