"""The golden vectors of tests/golden/reference_kats.json against the oracle
(CPU) and against the HIP kernels through the C ABI (GPU)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as orc
from oracle.oracle import F32, F16, BF16, SUM, MIN, MAX, PRODUCT

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
BIN = {"accumulate": SUM, "min": MIN, "max": MAX, "product": PRODUCT}


def f32(v):
    return np.array(v, dtype=np.float32)


def test_oracle_codec_vectors():
    for src, want in G["bf16_encode_bits"]["cases"]:
        x = np.array([int(src, 16)], dtype=np.uint32).view(np.float32)
        assert orc.encode_bf16(x)[0] == int(want, 16), src


def test_oracle_kernel_vectors():
    for name, op in BIN.items():
        a = f32(G[name]["a"])
        orc.reduce(a, f32(G[name]["b"]), F32, op)
        assert np.array_equal(a, f32(G[name]["out"])), name
    t = G["accumulate_tail_sizes"]
    for n in t["sizes"]:
        a = np.full(n, t["a"], np.float32)
        orc.reduce(a, np.full(n, t["b"], np.float32), F32, SUM)
        assert np.array_equal(a, np.full(n, t["out"], np.float32))
    a = f32(G["scale"]["a"]); orc.scale(a, F32, G["scale"]["s"])
    assert np.array_equal(a, f32(G["scale"]["out"]))
    a = f32(G["accumulate_scale"]["a"]); orc.accumulate_scale(a, f32(G["accumulate_scale"]["b"]), F32, G["accumulate_scale"]["s"])
    assert np.array_equal(a, f32(G["accumulate_scale"]["out"]))
    for c in G["scale_constants_bits"]["cases"]:
        w = c["world"]
        if "f32" in c:
            assert orc.scale_constant_bits(F32, 1 / w, 0) == int(c["f32"], 16)
        if "f16" in c:
            assert orc.scale_constant_bits(F16, 1 / w, 0) == int(c["f16"], 16)
        assert orc.scale_constant_bits(BF16, 1 / w, orc.SCALE_VIEW) == int(c["bf16_view"], 16)
        assert orc.scale_constant_bits(BF16, 1 / w, orc.SCALE_TENSOR) == int(c["bf16_tensor"], 16)
    for c in G["chunk_sizes"]["cases"]:
        assert [x[1] for x in orc.chunkize(c["numel"], 4, c["world"])] == c["counts"]


def test_oracle_collective_vectors():
    t = G["three_rank_sum_avg"]
    for n in t["sizes"]:
        for algo in (orc.RING, orc.TREE, orc.BUTTERFLY):
            if algo != orc.TREE and n < 3:
                continue
            b = [np.full(n, r + 1.0, np.float32) for r in range(3)]
            orc.allreduce(algo, b, F32, SUM)
            assert all(np.array_equal(x, np.full(n, t["sum"], np.float32)) for x in b)
            b = [np.full(n, r + 1.0, np.float32) for r in range(3)]
            orc.allreduce(algo, b, F32, orc.AVG)
            assert all(np.allclose(x, t["avg"], rtol=1e-6) for x in b)


@pytest.mark.gpu
def test_gpu_golden_vectors():
    import torch
    import gpu_util as U
    from mccl_amd import kernels as K, harness as H, _lib as L
    K.hip_kernels_init(0)
    x = np.array([int(s, 16) for s, _ in G["bf16_encode_bits"]["cases"]], dtype=np.uint32).view(np.float32)
    e = K.encode_bf16(U.to_dev(x, F32)); K.hip_sync()
    assert [int(v) for v in U.bits(e)] == [int(w, 16) for _, w in G["bf16_encode_bits"]["cases"]]
    for name, op in BIN.items():
        for dt in (torch.float32, torch.float16, torch.bfloat16):
            a = torch.tensor(G[name]["a"], dtype=dt, device="cuda")
            K.hip_reduce_op(a, torch.tensor(G[name]["b"], dtype=dt, device="cuda"), op); K.hip_sync()
            assert torch.equal(a, torch.tensor(G[name]["out"], dtype=dt, device="cuda")), (name, dt)
    a = torch.tensor(G["scale"]["a"], device="cuda")
    K.hip_scale_inplace(a, G["scale"]["s"]); K.hip_sync()
    assert torch.equal(a, torch.tensor(G["scale"]["out"], device="cuda"))
    a = torch.tensor(G["accumulate_scale"]["a"], device="cuda")
    K.hip_accumulate_and_scale(a, torch.tensor(G["accumulate_scale"]["b"], device="cuda"), G["accumulate_scale"]["s"]); K.hip_sync()
    assert torch.equal(a, torch.tensor(G["accumulate_scale"]["out"], device="cuda"))
    for c in G["scale_constants_bits"]["cases"]:
        w = c["world"]
        one = U.to_dev(np.array([0x3F80] * 8, dtype=np.uint16), BF16)           # 1.0 * s == s
        K.hip_scale_inplace_view(one.data_ptr(), L.BF16, 8, 1 / w)
        assert U.bits(one)[0] == int(c["bf16_view"], 16)
        one = U.to_dev(np.array([0x3F80] * 8, dtype=np.uint16), BF16)
        K.hip_scale_inplace(one, 1 / w); K.hip_sync()
        assert U.bits(one)[0] == int(c["bf16_tensor"], 16)
    for c in G["chunk_sizes"]["cases"]:
        assert [x[1] for x in H.chunkize(c["numel"], 4, c["world"])] == c["counts"]
    t = G["three_rank_sum_avg"]
    for n in t["sizes"]:
        for algo in (L.ALGO_RING, L.ALGO_TREE, L.ALGO_BUTTERFLY):
            if algo != L.ALGO_TREE and n < 3:
                continue
            b = [torch.full((n,), r + 1.0, device="cuda") for r in range(3)]
            H.allreduce_replay(b, "sum", algo)
            assert all(torch.equal(x, torch.full((n,), t["sum"], device="cuda")) for x in b)
