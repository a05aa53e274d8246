"""Sanitizer builds of the host-only native code (no GPU) under ThreadSanitizer
and under AddressSanitizer + UBSan: the row mover's threads, bounded waits, cancel
and destroy; the disk tier's threaded block I/O, buffered and direct, with aligned
and unaligned pools. Skipped where g++ or its sanitizer runtimes are absent."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


@pytest.mark.parametrize("sanitize", ["thread", "address,undefined"])
@pytest.mark.parametrize("driver,source,needs_hip", [("row_mover_sanitize.cpp", "host_rows.cpp", True),
                                                     ("disk_tier_sanitize.cpp", "disk_tier.cpp", False)])
def test_host_code_under_sanitizers(tmp_path, sanitize, driver, source, needs_hip):
    gxx = shutil.which("g++")
    if gxx is None or (needs_hip and not os.path.isdir(os.path.join(ROCM, "include", "hip"))):
        pytest.skip("needs g++ and the HIP headers")
    exe = tmp_path / "driver"
    cmd = [gxx, "-std=c++17", "-O1", "-g", f"-fsanitize={sanitize}", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(ROCM, "include"), "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "lmserve_amd", "csrc"),
           os.path.join(ROOT, "tests", "native", driver), os.path.join(ROOT, "lmserve_amd", "csrc", source)]
    if needs_hip:
        cmd += ["-L", os.path.join(ROCM, "lib"), "-lamdhip64", f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}"]
    cmd += ["-lpthread", "-o", str(exe)]
    built = subprocess.run(cmd, capture_output=True, text=True)
    if built.returncode != 0:
        pytest.skip(f"sanitizer build not possible here: {built.stderr[-300:]}")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", TSAN_OPTIONS="halt_on_error=1")
    ran = subprocess.run([str(exe), str(tmp_path)], capture_output=True, text=True, timeout=120, env=env)
    assert ran.returncode == 0, ran.stdout[-2000:] + ran.stderr[-4000:]
    assert "bad=0" in ran.stdout
    assert "WARNING: ThreadSanitizer" not in ran.stderr and "ERROR: AddressSanitizer" not in ran.stderr
    assert "runtime error" not in ran.stderr
