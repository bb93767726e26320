import os
import sys

import pytest

# libmcclx checks every launch's pointers against their allocations when this is set
os.environ.setdefault("MCCLX_VALIDATE", "1")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _abort_log() -> str:
    """Should the process ever abort, the extension writes the native stack of the thread that
    did it, and the message of an uncaught C++ exception, to this file: file descriptor 2 is
    pytest's capture file while a test runs, and what is written there dies with the process."""
    for d in (os.path.join(ROOT, "gpurun_out"), os.environ.get("TMPDIR") or "/tmp"):
        try:
            os.makedirs(d, exist_ok=True)
            path = os.path.join(d, "mccl_abort_backtrace.txt")
            with open(path, "a"):
                pass
            return path
        except OSError:
            continue
    return "1"


os.environ.setdefault("MCCL_ABORT_BACKTRACE", _abort_log())

for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def _build_if_nothing_is_built():
    """Tests load what is built; only when the native libraries are absent do they build them."""
    from mccl_amd import build as b
    if not os.path.exists(b.LIB_PATH):
        b.build(force=True)
    if not os.path.exists(b.backend_path()):
        b.build_backend()
    from oracle import oracle as orc
    if not os.path.exists(orc.LIB_PATH):
        orc.build()


def pytest_sessionstart(session):
    _build_if_nothing_is_built()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are only meaningful with a device; without one they are skipped
    # (the CPU suite is selected with -m "not gpu").
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
