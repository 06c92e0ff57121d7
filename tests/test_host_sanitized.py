"""The host allocators under AddressSanitizer and UndefinedBehaviorSanitizer: ``tests/host/alloc_check.cpp``
drives ``csrc/host/cache_alloc.cpp`` through seeded random orders of requests, built as one
program with ``-fsanitize=address,undefined`` (host code only; nothing here touches a GPU)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCES = [os.path.join(ROOT, "tests", "host", "alloc_check.cpp"),
           os.path.join(ROOT, "kv_cache_optimization_for_llm_amd", "csrc", "host", "cache_alloc.cpp")]


def test_allocators_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "alloc_check")
    build = subprocess.run([cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=all", "-static-libasan", *SOURCES, "-o", exe],
                           capture_output=True, text=True, timeout=300)
    if build.returncode != 0 and ("asan" in build.stderr or "ubsan" in build.stderr) and "error:" not in build.stderr:
        pytest.skip(f"this compiler has no sanitizer runtime: {build.stderr[-300:]}")
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0"))
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.startswith("ok ") and int(run.stdout.split()[1]) > 100000
