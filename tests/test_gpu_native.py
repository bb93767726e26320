"""The C ABI from a plain C program on the GPU (tests/native/cabi_gpu.c): no torch and no HIP
headers on the caller's side, results checked in C against the reference's recipe."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_plain_c_client_on_the_gpu():
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "native"))
    import build_native
    exe = build_native.build("cabi_gpu")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "ok", (r.returncode, r.stdout, r.stderr)
