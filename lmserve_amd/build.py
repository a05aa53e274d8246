"""Build libkvcache.so (HIP, gfx950) in-tree with hipcc.

`python -m lmserve_amd.build` compiles `csrc/*.hip` into
`lmserve_amd/libkvcache.so`. hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
SOURCES = [os.path.join(PKG_DIR, "csrc", "kvcache.hip"),
           os.path.join(PKG_DIR, "csrc", "rope_cache.hip"),
           os.path.join(PKG_DIR, "csrc", "disk_tier.cpp"),
           os.path.join(PKG_DIR, "csrc", "host_rows.cpp")]
INCLUDE = os.path.join(REPO_ROOT, "include")
LIB_PATH = os.path.join(PKG_DIR, "libkvcache.so")
FAST_SRC = os.path.join(PKG_DIR, "csrc", "fastcall.cpp")
FAST_PATH = os.path.join(PKG_DIR, "_kvc_fast.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def build(verbose: bool = False) -> str:
    """Compile the library; always recompiles. Returns the path of the .so."""
    cmd = [find_hipcc(), *HIPCC_FLAGS, "-I", INCLUDE, *SOURCES, "-o", LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout + proc.stderr)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    try:
        build_fastcall(verbose)
    except Exception as exc:   # the operators then call the same entry points through ctypes
        if os.path.exists(FAST_PATH):
            os.remove(FAST_PATH)   # never leave an extension of another ABI beside the new library
        print(f"warning: _kvc_fast not built ({exc}); per-layer calls go through ctypes",
              file=sys.stderr, flush=True)
    return LIB_PATH


def build_fastcall(verbose: bool = False) -> str:
    """Compile `_kvc_fast`, the CPython entry to the per-layer plan calls (host C++
    against torch's tensor headers; links against libkvcache.so next to it and
    torch's Python library)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise RuntimeError("no C++ compiler for lmserve_amd/csrc/fastcall.cpp")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-I", INCLUDE]
    for inc in cpp_extension.include_paths():
        cmd += ["-isystem", inc]
    rocm = os.path.dirname(os.path.dirname(os.path.realpath(find_hipcc())))
    cmd += ["-I", sysconfig.get_paths()["include"], "-D__HIP_PLATFORM_AMD__", "-isystem",
            os.path.join(rocm, "include"), FAST_SRC, "-L", PKG_DIR, "-lkvcache",
            "-L", torch_lib, "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10",
            "-L", os.path.join(rocm, "lib"), "-lamdhip64",
            f"-Wl,-rpath,$ORIGIN,-rpath,{torch_lib}", "-o", FAST_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building _kvc_fast failed:\n" + proc.stdout + proc.stderr)
    os.replace(FAST_PATH + ".tmp", FAST_PATH)
    return FAST_PATH


HEADERS = [os.path.join(PKG_DIR, "csrc", "common.h"), os.path.join(INCLUDE, "kvcache.h"),
           os.path.join(INCLUDE, "kvcache_experimental.h")]


def is_stale() -> bool:
    """True when a built file is missing or older than one of its sources."""
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    if os.path.exists(FAST_PATH):
        built = min(built, os.path.getmtime(FAST_PATH))
    return any(os.path.exists(f) and os.path.getmtime(f) > built for f in SOURCES + HEADERS + [FAST_SRC])


def ensure_built() -> None:
    """For tests, the smoke check and the benchmark: use what is built; compile
    when the library is missing, or older than its sources and a compiler is at
    hand. The operators themselves never build anything."""
    if not os.path.exists(LIB_PATH):
        build(verbose=True)
    elif is_stale():
        try:
            find_hipcc()
        except RuntimeError:
            print(f"warning: {LIB_PATH} is older than its sources and no hipcc was found",
                  file=sys.stderr, flush=True)
            return
        build(verbose=True)


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
