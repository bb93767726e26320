"""torch's DistributedDataParallel over backend "mccl" with several ranks, as the
reference's tests/test_ddp.py runs it (two and three ranks; a Linear layer, an
MLP, SGD for five steps, per-rank batches; gradients and weights the same on
every rank; here also the same weights as one process training on the ranks'
batches put together, which a random batch's loss going down does not show).  The ranks are threads of this process sharing the one GPU: torch's
own thread-local world (the one its MultiThreadedTestCase installs) lets every
thread call dist.init_process_group(backend="mccl") and own a default group.

Stronger than the reference's allclose checks where arithmetic allows: ranks
must agree bit for bit, and with two ranks (one commutative add per element) the
synchronised gradient must equal the oracle's allreduce of the local gradients."""
import datetime
import gc
import threading

import numpy as np
import pytest
import torch
import torch.distributed as dist
import torch.nn as nn

pytestmark = pytest.mark.gpu

TIMEOUT = datetime.timedelta(seconds=20)


@pytest.fixture(scope="module")
def CX():
    import mccl_amd
    from mccl_amd import _C
    return _C


def run_default_groups(world, fn):
    """fn(rank, world) on one thread per rank, each inside its own default process group."""
    import torch._C._distributed_c10d as c10d
    from torch.testing._internal.distributed import multi_threaded_pg as mtpg
    assert not dist.is_initialized()
    mtpg._install_threaded_pg()           # dist's world becomes thread-local
    c10d._set_thread_isolation_mode(True)  # group names are registered per thread
    store = dist.HashStore()
    out, errs = [None] * world, [None] * world

    def body(r):
        try:
            torch.cuda.set_device(0)
            dist.init_process_group(backend="mccl", store=store, rank=r, world_size=world, timeout=TIMEOUT)
            try:
                # The autograd engine has one worker thread per device; with every rank on
                # cuda:0 the ranks' backward passes would queue behind each other's blocking
                # collectives.  The switch is thread-local: each rank runs its own backward.
                with torch.autograd.set_multithreading_enabled(False):
                    out[r] = fn(r, world)
            finally:
                # DDP modules sit in reference cycles: collect them here, on the rank's own thread and
                # while its group exists, not whenever and wherever the collector next runs
                gc.collect()
                dist.destroy_process_group()
        except BaseException as e:  # noqa: BLE001
            errs[r] = e

    try:
        ts = [threading.Thread(target=body, args=(r,)) for r in range(world)]
        for t in ts:
            t.start()
        for t in ts:
            t.join(90)
        assert not any(t.is_alive() for t in ts), "a rank thread hung"
    finally:
        c10d._set_thread_isolation_mode(False)
        mtpg._uninstall_threaded_pg()
    for e in errs:
        if e is not None:
            raise e
    return out


def batch(n_in, seed, step, world, rank):
    g = torch.Generator(device="cpu").manual_seed(seed + step * world + rank)
    return torch.randn(8, n_in, generator=g).cuda(), torch.ones(8, 1, device="cuda")


def train(model, rank, world, seed, steps=5, **ddp_kwargs):
    from torch.nn.parallel import DistributedDataParallel as DDP
    ddp = DDP(model, **ddp_kwargs)
    opt = torch.optim.SGD(ddp.parameters(), lr=0.01)
    n_in = next(model.parameters()).shape[1]
    losses = []
    for step in range(steps):
        x, y = batch(n_in, seed, step, world, rank)
        opt.zero_grad()
        loss = nn.functional.mse_loss(ddp(x), y)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    return losses


def train_alone(model, world, seed, steps=5):
    """The same training in one process on the ranks' batches put together: the mean loss
    over all samples has the mean of the ranks' gradients."""
    opt = torch.optim.SGD(model.parameters(), lr=0.01)
    n_in = next(model.parameters()).shape[1]
    for step in range(steps):
        xs, ys = zip(*[batch(n_in, seed, step, world, r) for r in range(world)])
        opt.zero_grad()
        nn.functional.mse_loss(model(torch.cat(xs)), torch.cat(ys)).backward()
        opt.step()
    return snapshot(model)


def snapshot(model):
    return [p.detach().cpu().numpy().copy() for p in model.parameters()]


def fresh(make, seed=42):
    with torch.random.fork_rng(devices=[]):
        torch.manual_seed(seed)
        return make().cuda()


@pytest.mark.parametrize("world,make", [
    (2, lambda: nn.Linear(16, 1, bias=False)),                                        # test_ddp.py:74-106
    (2, lambda: nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 1))),       # test_ddp.py:140-176
    (3, lambda: nn.Linear(16, 1, bias=False)),                                        # test_ddp.py:182-213
], ids=["linear-2", "mlp-2", "linear-3"])
def test_ddp_training_keeps_ranks_identical(CX, world, make):
    lock = threading.Lock()

    def fn(rank, world):
        with lock:                       # torch's global RNG is shared by the threads
            model = fresh(make)
        assert dist.get_backend() == "mccl" and dist.get_world_size() == world and dist.get_rank() == rank
        losses = train(model, rank, world, seed=1000)
        return losses, snapshot(model)

    out = run_default_groups(world, fn)
    for _, params in out[1:]:
        for a, b in zip(out[0][1], params):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    start = snapshot(fresh(make))
    alone = train_alone(fresh(make), world, seed=1000)
    for a, b, c in zip(out[0][1], alone, start):
        assert np.allclose(a, b, rtol=1e-5, atol=1e-6)
        assert not np.allclose(a, c, rtol=1e-3, atol=1e-4)      # and it did train


def test_ddp_gradient_is_the_oracles_allreduce_of_the_local_gradients(CX):
    """test_ddp.py:112-134 (different inputs per rank, same gradients after backward),
    against the arithmetic: DDP divides each local gradient by the world size and
    allreduces with SUM; with two ranks that is one add per element in any schedule."""
    from torch.nn.parallel import DistributedDataParallel as DDP
    from oracle import oracle as orc
    lock = threading.Lock()

    def fn(rank, world):
        with lock:
            model = fresh(lambda: nn.Linear(8, 4, bias=True))
            local = fresh(lambda: nn.Linear(8, 4, bias=True))
        g = torch.Generator(device="cpu").manual_seed(100 + rank)
        x = torch.randn(4, 8, generator=g).cuda()
        y = torch.randn(4, 4, generator=g).cuda()
        nn.functional.mse_loss(local(x), y).backward()
        ddp = DDP(model)
        nn.functional.mse_loss(ddp(x), y).backward()
        return ([p.grad.detach().cpu().numpy().copy() for p in model.parameters()],
                [p.grad.detach().cpu().numpy().copy() for p in local.parameters()])

    out = run_default_groups(2, fn)
    for i in range(len(out[0][0])):
        halves = [np.ascontiguousarray((out[r][1][i] / np.float32(2)).astype(np.float32).ravel()) for r in range(2)]
        rc, _ = orc.pg_allreduce(halves, orc.F32, orc.SUM)
        assert rc == 0
        for r in range(2):
            assert np.array_equal(out[r][0][i].ravel().view(np.uint32), halves[r].view(np.uint32))


@pytest.mark.parametrize("knob", [None, "MCCL_ALLREDUCE_ASYNC=1", "MCCL_WIRE=host"],
                         ids=["sync", "event-based", "host-wire"])
def test_ddp_many_buckets(CX, monkeypatch, knob):
    """Six 1 MiB gradient buckets per step: the reference's synchronous allreduce,
    event-based completion, and peers' chunks travelling through pinned host memory."""
    if knob:
        monkeypatch.setenv(*knob.split("="))
    lock = threading.Lock()
    make = lambda: nn.Sequential(*[m for _ in range(5) for m in (nn.Linear(512, 512), nn.ReLU())], nn.Linear(512, 1))

    def fn(rank, world):
        with lock:
            model = fresh(make)
        losses = train(model, rank, world, seed=7000, steps=4, bucket_cap_mb=1)
        return losses, snapshot(model)

    out = run_default_groups(3, fn)
    for _, params in out[1:]:
        for a, b in zip(out[0][1], params):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    alone = train_alone(fresh(make), 3, seed=7000, steps=4)
    for a, b in zip(out[0][1], alone):
        assert np.allclose(a, b, rtol=1e-4, atol=1e-6)
