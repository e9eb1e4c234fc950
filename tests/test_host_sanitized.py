"""The host runtime (cache manager, scheduler) under the address and undefined-behaviour sanitizers: a native driver
is compiled with the library's sources and run over random workloads with small pools.  CPU only."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "prelude_amd", "csrc", "host")


def test_host_runtime_under_sanitizers(tmp_path):
    cxx = shutil.which("g++") or shutil.which("clang++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "host_fuzz")
    sources = [os.path.join(ROOT, "tests", "host_fuzz.cpp")] + [os.path.join(HOST, f) for f in
                                                                ("cache_manager.cpp", "scheduler.cpp", "host_api.cpp")]
    flags = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-I", HOST]
    if cxx.endswith("g++"):
        flags += ["-static-libasan", "-static-libubsan"]       # whatever else is preloaded, the runtime comes first
    build = subprocess.run([cxx, *flags, "-o", exe, *sources], capture_output=True, text=True, timeout=300)
    if build.returncode != 0 and any(w in (build.stderr + build.stdout).lower() for w in ("sanitize", "asan", "ubsan")):
        pytest.skip("this compiler has no sanitizer runtimes: " + build.stderr[-300:])
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([exe, "300"], capture_output=True, text=True, timeout=300,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0"))
    assert run.returncode == 0 and run.stdout.strip().startswith("ok:"), (run.stdout[-1500:], run.stderr[-3000:])
    preemptions = int(run.stdout.split()[-2])
    assert preemptions > 50        # the pools were small enough for the scheduler to have to take requests back
