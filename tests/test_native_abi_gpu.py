"""The C ABI from a host written in plain C (tests/native/abi_check.c): no Python, no torch
in the process that calls the library.  The binary is built by `make -C tests/native`
(done by __graft_entry__.build()); here it is only run."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "native", "_build", "abi_check")


def test_plain_c_host_runs_the_scans():
    if not os.path.exists(BINARY):
        pytest.skip("tests/native/_build/abi_check has not been built (make -C tests/native)")
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.startswith("abi_check ok"), done.stdout
