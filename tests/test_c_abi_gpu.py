"""
Runs tests/c_abi/abi_check, a plain-C99 program (no C++, no torch, no Python) that calls every
scan entry point of libscanscam_hip.so on device buffers it allocated itself and checks the results
against sequential host loops. It is built by __graft_entry__.build() (make -C tests/c_abi).
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "abi_check")


def test_plain_c_consumer(gpu):
    assert os.path.exists(BINARY), "tests/c_abi/abi_check is not built: run `make -C tests/c_abi`"
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=120)
    print(done.stdout)
    print(done.stderr)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "abi_check: ok" in done.stdout
