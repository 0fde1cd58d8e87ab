"""The library's host-memory routines (tplr_gather_host, tplr_pack12_host, tplr_unpack12_host:
templar_amd/csrc/tplr_host.cpp) built with the host compiler under AddressSanitizer and UndefinedBehaviorSanitizer
and driven over random sizes (tests/host_asan_driver.cpp).  CPU only; skipped when the compiler has no sanitizer
runtime."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_routines_are_clean_under_address_sanitizer(tmp_path):
    cxx = shutil.which("g++") or shutil.which("clang++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "host_asan")
    cmd = [cxx, "-std=c++17", "-g", "-O1", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "templar_amd", "csrc", "tplr_host.cpp"), os.path.join(ROOT, "tests", "host_asan_driver.cpp"),
           "-o", exe, "-pthread"]
    built = subprocess.run(cmd, capture_output=True, text=True)
    if built.returncode != 0 and ("asan" in built.stderr or "ubsan" in built.stderr or "sanitize" in built.stderr):
        pytest.skip("the host compiler has no sanitizer runtime: " + built.stderr.strip().splitlines()[-1])
    assert built.returncode == 0, built.stderr
    # (a library preloaded into every process of this environment comes before the sanitizer's runtime: the
    # runtime is told not to insist on being first)
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1:abort_on_error=0")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.startswith("ok ") and "ERROR: AddressSanitizer" not in run.stderr and "runtime error" not in run.stderr
