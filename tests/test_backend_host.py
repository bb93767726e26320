"""Host-side behaviour of the c10d backend pieces, no GPU needed: the FIFO
engine (the reference's tests/internal/test_progress.cpp cases, and the
reference's own engine from oracle/_ref run on the same cases), the Work
object (csrc/backend/WorkMCCL.cpp), the in-process mesh, registration."""
import ctypes as C
import datetime
import os

import pytest

from oracle import oracle as orc


@pytest.fixture(scope="module")
def CX():
    from mccl_amd import _C
    return _C


# ---- Progress: tests/internal/test_progress.cpp:12-63 --------------------

def test_fifo_order_across_many_tasks(CX):
    assert CX._test_progress_order(100, 0, False) == list(range(100))


def test_destructor_drains_the_queue(CX):
    assert CX._test_progress_order(50, 0, True) == list(range(50))


def test_exception_does_not_poison_the_engine(CX):
    assert CX._test_progress_order(3, 0b001, False) == [1, 2]
    assert CX._test_progress_order(10, 0b1000010000, False) == [0, 1, 2, 3, 5, 6, 7, 8]


def test_submit_does_not_wait_for_a_running_task(CX):
    assert CX._test_progress_submit_latency_us() < 1000


def test_same_observable_order_as_the_reference_engine(CX):
    R = orc.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    for n, mask in ((100, 0), (7, 0b0101010), (64, 0xF0F0F0F0F0F0F0F0)):
        buf = (C.c_int * n)()
        k = R.ref_progress_order(n, mask, buf)
        assert CX._test_progress_order(n, mask, False) == list(buf[:k])


# ---- the engine shut down from its own worker thread ---------------------------------------
# (the reference leaves this open; a join of the calling thread throws inside a destructor and
# std::terminate ends the process with SIGABRT on a native thread)

def test_a_task_may_hold_the_last_reference_to_its_own_engine(CX):
    """The engine is destroyed on its own worker, by the task that owned it: the tasks queued
    behind that one still run, in order, and nothing aborts."""
    assert CX._test_progress_self_shutdown("task_owns_engine") == [1, 2, 3]


def test_a_future_callback_may_drop_the_owner_of_the_engine_it_runs_on(CX):
    """An owner of an engine (as a process group is) dies on that engine's thread, when the
    Future of a Work completed there drops the callback that kept it alive: the callback runs
    (1), the owner's destructor shuts the engine down from its own thread, which runs the
    queued task there and then (3) while the owner's members are still whole (9), and the
    task that completed the Work goes on to its end (2)."""
    assert CX._test_progress_self_shutdown("callback_drops_owner") == [1, 3, 9, 2]


def test_an_uncaught_exception_on_a_native_thread_is_named_in_the_abort_file(tmp_path):
    """std::terminate on a worker thread: the message and the native stack go to the file
    MCCL_ABORT_BACKTRACE names (file descriptor 2 may belong to a test runner's capture)."""
    import subprocess
    import sys
    log = tmp_path / "abort.txt"
    env = dict(os.environ, MCCL_ABORT_BACKTRACE=str(log))
    r = subprocess.run([sys.executable, "-c",
                        "from mccl_amd import _C; _C._test_terminate('engine thread blew up')"],
                       env=env, capture_output=True, text=True, timeout=120,
                       cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == -6, (r.returncode, r.stderr[-500:])
    text = log.read_text()
    assert "std::terminate called with an uncaught exception: [MCCL] engine thread blew up" in text
    assert "SIGABRT: native stack of the aborting thread" in text


# ---- WorkMCCL: csrc/backend/WorkMCCL.cpp:46-104 --------------------------------

def test_work_completion_states(CX):
    assert CX._test_work("finish", 1000) == (True, True, "")
    done, ok, msg = CX._test_work("fail", 1000)
    assert done and not ok and msg == "[MCCL] engine task failed"      # wait() rethrows (:57-59)
    done, ok, msg = CX._test_work("sync_cb_throws", 1000)
    assert done and not ok and msg == "[MCCL] drain failed"            # finish() -> sync cb throws (:71-78)
    assert CX._test_work("late", 2000) == (True, True, "")
    assert CX._test_work("never", 50) == (False, False, "timeout")     # wait(timeout) returns false (:51-55)


# ---- in-process mesh ----------------------------------------------------------

def test_mesh_meets_every_round_with_slots_by_rank(CX):
    assert CX._test_mesh(4, 5, -1, 5000, False) == ["ok:5"] * 4
    assert CX._test_mesh(1, 3, -1, 5000, False) == ["ok:3"]


def test_mesh_times_out_when_a_rank_is_missing(CX):
    out = CX._test_mesh(3, 1, 1, 150, False)
    assert out[1] == "absent"
    assert all(o.startswith("[MCCL] Timeout: ") for i, o in enumerate(out) if i != 1)


def test_a_rank_that_arrives_after_its_peers_gave_up_finds_the_mesh_broken(CX):
    """The peers' arrivals were taken back when their wait timed out: the late rank does not become
    the leader of a collective whose other members have left (their buffers may be gone)."""
    out = CX._test_mesh(3, 1, 1, 100, False, 400)
    assert out[0].startswith("[MCCL] Timeout: ") and out[2].startswith("[MCCL] Timeout: ")
    assert "broken" in out[1] or out[1].startswith("[MCCL] Timeout: "), out
    assert not out[1].startswith("ok"), "the leader ran with contributions of ranks that had left"
    # arriving while the others still wait is fine, however close to their limit
    assert CX._test_mesh(3, 2, 1, 2000, False, 300) == ["ok:2"] * 3


def test_a_rank_arriving_as_its_peers_time_out_is_served_by_all_or_by_none(CX):
    """The late rank arrives at about the moment the others' wait runs out.  Whichever way each round
    falls, it falls one way for everybody: either the collective ran with all three (a rank that
    could not take its arrival back any more waited for the leader), or nobody's did."""
    all_ok = none_ok = 0
    for i in range(150):
        out = CX._test_mesh(3, 1, i % 3, 4, False, 4)
        oks = [o.startswith("ok") for o in out]
        assert all(oks) or not any(oks), out
        all_ok += all(oks)
        none_ok += not any(oks)
    assert all_ok + none_ok == 150


def test_mesh_leader_error_reaches_every_rank(CX):
    assert CX._test_mesh(3, 2, -1, 5000, True) == ["[MCCL] leader failed"] * 3


# ---- the byte transport with PeerMesh's interface (PeerMesh.hpp:12-31) --------------------

@pytest.mark.parametrize("world", [2, 3, 5])
def test_peer_send_recv_ring_exchange(CX, world):
    assert CX._test_peer_wire("ring", world, 8) == ["ok:0"] * world


def test_peer_send_kept_hands_the_buffer_over_and_lets_go_of_it(CX):
    assert CX._test_peer_wire("kept", 3, 8) == ["ok:0"] * 3


def test_peer_recv_refuses_a_message_of_another_length(CX):
    out = CX._test_peer_wire("short", 2)
    assert all("expects 4 bytes" in o and "which sent 3" in o for o in out), out


def test_peer_recv_times_out_and_the_mesh_stays_usable(CX):
    assert CX._test_peer_wire("silent", 3, 1, 100) == ["timeout:3", "timeout:1", "timeout:2"]


# ---- registration: mccl/_backend.py:30-75, tests/test_smoke.py:12-14 ---------------

def test_backend_is_registered_and_registration_is_idempotent():
    import torch.distributed as dist
    import mccl_amd
    assert mccl_amd.register() is True and mccl_amd.register() is True
    assert "mccl" in dist.Backend.backend_list
    assert dist.Backend.backend_capability["mccl"] == ["cuda"]


def test_factory_fails_loudly_without_a_gpu(CX):
    import torch
    import torch.distributed as dist
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(RuntimeError, match=r"\[MCCL\] no usable GPU"):
        CX._create_process_group_mccl(dist.HashStore(), 0, 1, datetime.timedelta(seconds=5))
    with pytest.raises(RuntimeError, match="rank/size invalid"):
        CX._create_process_group_mccl(dist.HashStore(), 3, 2, datetime.timedelta(seconds=5))


def test_engine_shutdown_under_the_gil_does_not_deadlock_with_a_task_that_needs_it(CX):
    """A process group dropped from Python is destroyed with the GIL held and joins its engine
    thread; the engine's last task may be releasing a tensor Python created, which takes the GIL.
    The join therefore gives the GIL up (regression: rank threads froze when groups were
    created and dropped in a loop)."""
    import threading
    res = []
    t = threading.Thread(target=lambda: res.append(CX._test_progress_shutdown_while_task_needs_gil()), daemon=True)
    t.start()
    t.join(20)
    assert not t.is_alive(), "shutdown dead-locked against a task waiting for the GIL"
    assert res == [1]


def test_logger_levels_and_line_format():
    """DISTRO_LOG_LEVEL as in the reference (csrc/common/Logging.hpp:22-78): default WARN, names in
    any case or digits, lines '[MCCL LEVEL epoch-ms file:line] text' on stderr."""
    import re
    import subprocess
    import sys
    code = ("import mccl_amd; from mccl_amd import _C; "
            "print([int(_C._test_log(l, 'message %d' % l)) for l in range(7)])")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for setting, first in ((None, 3), ("debug", 1), ("TRACE", 0), ("4", 4), ("off", 7), ("nonsense", 3)):
        env = dict(os.environ)
        env.pop("DISTRO_LOG_LEVEL", None)
        if setting is not None:
            env["DISTRO_LOG_LEVEL"] = setting
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=root, env=env, timeout=120)
        assert r.returncode == 0, r.stderr
        enabled = eval(r.stdout.strip().splitlines()[-1])
        assert enabled == [int(first <= l < 6) for l in range(7)], (setting, enabled)
        lines = [l for l in r.stderr.splitlines() if l.startswith("[MCCL ")]
        assert len(lines) == sum(enabled)
        for l in lines:
            assert re.fullmatch(r"\[MCCL (TRACE|DEBUG|INFO |WARN |ERROR|FATAL) \d{13} bindings\.cpp:0\] message \d", l), l
