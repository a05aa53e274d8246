"""Runs tests/native/abi_check (a plain HIP program, no Python or torch in the
process) which drives every copy-path entry point of the C ABI and compares
with the C oracle. The binary is built by `tests/native/build_check.py`."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "abi_check")


def test_c_abi_from_a_plain_hip_program(gpu):
    from tests.native.build_check import ensure_native_check
    ensure_native_check()              # builds only if the binary is missing
    assert os.path.exists(BIN)
    proc = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "ABI CHECK PASSED" in proc.stdout
    assert proc.stdout.count("ok: ") == 39
