"""Host-buffer interop on the GPU: pinned device-mapped memory (zero-copy) and
the staging path (stage_for_send / unstage_from_recv, MPSInterop.mm:365-435)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle.oracle import F32, BF16, SUM

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    from mccl_amd import kernels, _lib
    import gpu_util
    return kernels, _lib, gpu_util, kernels.hip_kernels_init(0)


def host_view(addr, nbytes):
    return np.ctypeslib.as_array((C.c_uint8 * nbytes).from_address(addr))


def test_zero_copy_operands_in_pinned_host_memory(env):
    K, L, U, q = env
    n = 1_000_003
    rng = np.random.default_rng(1)
    a = U.rand_values(rng, n, F32); b = U.rand_values(rng, n, BF16)
    h, d = q.host_alloc(n * 2)
    try:
        host_view(h, n * 2)[:] = b.view(np.uint8)          # "the wire" writes into host memory
        own = U.to_dev(a, F32)
        plan = K.make_plan(L.BF16, 2, io=L.IO_OWN_FIRST_F32)
        q.fold(plan, [K.make_seg(own.data_ptr(), 0, [own.data_ptr(), d], n)])   # the kernel reads it in place
        q.drain()
        want = orc.wire_fold_chunk(a, [b])
        U.assert_same_bits(own, want, F32, "zero-copy peer")
        # and a result written straight into host memory
        q.fold(K.make_plan(L.BF16, 1, io=L.IO_OWN_FIRST_F32), [K.make_seg(0, d, [own.data_ptr()], n)])
        q.drain()
        assert np.array_equal(host_view(h, n * 2).view(np.uint16), orc.encode_bf16(want))
    finally:
        q.host_free(h)
    from mccl_amd import MCCLError
    with pytest.raises(MCCLError, match="was not returned by mcclx_host_alloc"):
        q.host_free(12345)


def test_stage_for_send_and_unstage_from_recv(env):
    K, L, U, q = env
    rng = np.random.default_rng(2)
    for nbytes in (1, 4099, (8 << 20) - 1, (8 << 20) + 1, 40_000_003):     # below / across the 8 MiB staging chunks
        src = rng.integers(0, 256, nbytes, dtype=np.uint8)
        t = torch.from_numpy(src).cuda()
        torch.cuda.synchronize()
        hp = q.stage_for_send(t.data_ptr(), nbytes)                          # device -> pinned staging, blocking
        assert np.array_equal(host_view(hp, nbytes), src)
        back = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        q.unstage_from_recv(back.data_ptr(), src.ctypes.data, nbytes)       # pageable host -> device, pipelined
        q.drain()
        assert torch.equal(back.cpu(), torch.from_numpy(src))
    # pinned source: single asynchronous copy; host-visible "device" source: returned without a copy
    h, d = q.host_alloc(1 << 20)
    try:
        host_view(h, 1 << 20)[:] = 7
        back = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        q.unstage_from_recv(back.data_ptr(), h, 1 << 20)
        q.drain()
        assert bool((back == 7).all())
        assert q.stage_for_send(d, 1 << 20) == h
    finally:
        q.host_free(h)


def test_received_bytes_then_reduce_matches_reference_order(env):
    """The reference's reduce_scatter leg: recv into host memory, unstage into a
    device scratch, binary reduce (ProcessGroupMCCL.cpp:378-383)."""
    K, L, U, q = env
    rng = np.random.default_rng(3)
    n = 500_009
    own = U.rand_values(rng, n, BF16); peer = U.rand_values(rng, n, BF16)
    d_own = U.to_dev(own, BF16)
    scratch = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    q.unstage_from_recv(scratch.data_ptr(), peer.ctypes.data, n * 2)
    K.hip_reduce_op_view(d_own.data_ptr(), scratch.data_ptr(), L.BF16, n, "sum")
    want = own.copy(); orc.reduce(want, peer, BF16, SUM)
    U.assert_same_bits(d_own, want, BF16, "unstage + reduce")


def test_ticket_stays_pollable_while_another_thread_waits(env):
    """A ticket another thread is waiting on must not read as complete before the device work is."""
    import threading
    from mccl_amd import kernels
    q = kernels.ReduceQueue(0)
    n = 1 << 30
    buf = torch.empty(2 * n, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    for _ in range(6):
        q.copy(buf.data_ptr() + n, buf.data_ptr(), n)      # about 2 ms of queued work
    ticket = q.record()
    seen_done_early = []
    waiter = threading.Thread(target=lambda: q.wait(ticket))
    waiter.start()
    while waiter.is_alive():
        done = q.query(ticket)
        if done and waiter.is_alive():
            # complete by the library's word: then the waiter must be about to return
            waiter.join(1.0)
            seen_done_early.append(waiter.is_alive())
    waiter.join()
    assert not any(seen_done_early)
    assert q.query(ticket)                                  # retired tickets read as complete
    q.close()


def test_table_launch_refuses_a_capture_it_did_not_start_and_noalloc_records(env):
    """A context on the caller's stream: while the caller records that stream into a graph, a launch
    that needs a descriptor table is refused (its staging ring would be replayed stale), and the
    allocation-free entry point -- kernel launches only -- records and replays correctly."""
    import ctypes as C
    from mccl_amd import _lib as L, kernels
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        q = kernels.ReduceQueue(0, on_torch_stream=True)
        nseg, n = 40, 3001
        a = torch.arange(nseg * n, dtype=torch.float32, device="cuda")
        b = torch.ones(nseg * n, dtype=torch.float32, device="cuda")
        out = torch.zeros_like(a)
        plan = kernels.make_plan(L.F32, 2)
        segs = [kernels.make_seg(out.data_ptr() + 4 * n * i, 0, [a.data_ptr() + 4 * n * i, b.data_ptr() + 4 * n * i], n)
                for i in range(nseg)]
        arr = (L.Seg * nseg)(*segs)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            rc = L.lib().mcclx_fold_batched(q.handle, C.byref(plan), arr, nseg)
            msg = L.last_error()
            rc2 = L.lib().mcclx_fold_batched_noalloc(q.handle, C.byref(plan), arr, nseg)
        assert rc == L.ERR_STATE and "did not start" in msg
        assert rc2 == L.OK
        for rep in range(3):
            out.zero_()
            b.fill_(float(rep + 1))
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, a + (rep + 1)), rep
        q.close()
