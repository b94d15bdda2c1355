"""Runs the plain-C caller of the library (tests/c_abi/abi_smoke.c, built by linearnexus_amd/build.py):
device memory from hipMalloc, a hand-filled lnx_scan_args, closed-form checks of lnx_chunk_fwd,
lnx_recurrent_fwd and lnx_decode_step, and the error path -- the boundary without Python or torch."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
EXE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "abi_smoke")


def test_plain_c_caller():
    assert os.path.exists(EXE), "run `python -m linearnexus_amd.build` first"
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "lnx_chunk_fwd" in r.stdout and "lnx_decode_step" in r.stdout
