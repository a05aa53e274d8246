"""Builds tests/native/abi_check: a plain HIP program that drives the C ABI of
libkvcache without Python and checks it against the C oracle (linked in as an
object of its own; the library itself never sees the oracle). Test
infrastructure: `python -m tests.native.build_check`."""
from __future__ import annotations

import os
import subprocess

from lmserve_amd.build import INCLUDE, PKG_DIR, REPO_ROOT, find_hipcc

HERE = os.path.dirname(os.path.abspath(__file__))
NATIVE_CHECK_SRC = os.path.join(HERE, "abi_check.cpp")
NATIVE_CHECK_BIN = os.path.join(HERE, "abi_check")
ORACLE_C = os.path.join(REPO_ROOT, "oracle", "kvc_oracle.c")


def build_native_check(verbose: bool = False) -> str:
    oracle_obj = NATIVE_CHECK_BIN + "_oracle.o"
    main_obj = NATIVE_CHECK_BIN + "_main.o"
    hipcc = find_hipcc()
    steps = [
        ["gcc", "-O2", "-std=c11", "-c", ORACLE_C, "-o", oracle_obj],
        [hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-I", INCLUDE, "-c", NATIVE_CHECK_SRC, "-o", main_obj],
        [hipcc, main_obj, oracle_obj, "-L", PKG_DIR, "-lkvcache",
         "-Wl,-rpath,$ORIGIN/../../lmserve_amd", "-o", NATIVE_CHECK_BIN],
    ]
    for cmd in steps:
        if verbose:
            print(" ".join(cmd), flush=True)
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("native check build failed:\n" + proc.stdout + proc.stderr)
    os.remove(oracle_obj)
    os.remove(main_obj)
    return NATIVE_CHECK_BIN


def ensure_native_check() -> str:
    """Use the built binary; build it if there is none, or if it is older than
    its source and a compiler is at hand."""
    stale = os.path.exists(NATIVE_CHECK_BIN) and \
        os.path.getmtime(NATIVE_CHECK_BIN) < os.path.getmtime(NATIVE_CHECK_SRC)
    if stale:
        try:
            find_hipcc()
        except RuntimeError:
            stale = False
    if stale or not os.path.exists(NATIVE_CHECK_BIN):
        build_native_check(verbose=True)
    return NATIVE_CHECK_BIN


if __name__ == "__main__":
    print(build_native_check(verbose=True))
