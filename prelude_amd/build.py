"""Compiles the two native libraries and says where they are.

* ``libprelude_kernels.so`` -- the HIP kernels for gfx950 (``csrc/kernels``), built with hipcc.
* ``libprelude_host.so``    -- cache manager and scheduler (``csrc/host``), built with g++.

Both are built inside the package (``prelude_amd/_lib``) when that folder can
be written, else under the system's temporary folder.  A library is rebuilt
when the text of its sources or the flags changed since it was built.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import List, Sequence

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
GPU_ARCH = "gfx950"

HIPCC_FLAGS = [
    f"--offload-arch={GPU_ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # no packed 32-bit float instructions: some of their forms have been seen to give wrong results on gfx950
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
HOST_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-Wextra"]


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[prelude_amd.build] {msg}", file=sys.stderr, flush=True)


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dir() -> str:
    """Where built libraries live: in the package if possible."""
    env = os.environ.get("PRELUDE_AMD_LIB_DIR")
    if env:
        os.makedirs(env, exist_ok=True)
        return env
    in_tree = os.path.join(PKG_DIR, "_lib")
    if _writable(in_tree):
        return in_tree
    uid = os.getuid() if hasattr(os, "getuid") else 0
    alt = os.path.join(tempfile.gettempdir(), f"prelude_amd_lib_{uid}")
    os.makedirs(alt, exist_ok=True)
    return alt


def _sources(sub: str, exts: Sequence[str]) -> List[str]:
    d = os.path.join(CSRC, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(tuple(exts)))


def _fingerprint(files: Sequence[str], flags: Sequence[str]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(flags).encode())
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _find(tool: str, extra: Sequence[str]) -> str:
    for cand in list(extra) + [shutil.which(tool) or ""]:
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError(f"{tool} not found (looked in {list(extra)} and on PATH)")


def _run(cmd: Sequence[str], what: str) -> None:
    env = dict(os.environ)
    # hipcc and clang want a home for their caches; an empty or unwritable HOME must not stop them
    if not env.get("HOME") or not os.access(env.get("HOME", ""), os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    p = subprocess.run(list(cmd), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if p.returncode != 0:
        raise BuildError(f"{what} failed (exit {p.returncode}):\n$ {' '.join(cmd)}\n{p.stdout}")


class _Ticker:
    """Prints a line every few seconds while a slow build runs."""

    def __init__(self, what: str, every: float = 10.0):
        self.what, self.every = what, every
        self._stop = threading.Event()
        self._t = threading.Thread(target=self._loop, daemon=True)
        self._t0 = time.time()

    def _loop(self):
        while not self._stop.wait(self.every):
            _log(f"still compiling {self.what} ({time.time() - self._t0:.0f} s)")

    def __enter__(self):
        self._t.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()


def kernels_lib_path() -> str:
    return os.path.join(lib_dir(), "libprelude_kernels.so")


def host_lib_path() -> str:
    return os.path.join(lib_dir(), "libprelude_host.so")


def _is_current(lib: str, fp: str) -> bool:
    stamp = lib + ".hash"
    try:
        with open(stamp) as f:
            return os.path.isfile(lib) and f.read().strip() == fp
    except OSError:
        return False


def _finish(lib: str, tmp_lib: str, fp: str) -> None:
    os.replace(tmp_lib, lib)
    with open(lib + ".hash", "w") as f:
        f.write(fp)


def build_kernels(force: bool = False, jobs: int | None = None) -> str:
    srcs = _sources("kernels", (".hip",))
    hdrs = _sources("kernels", (".h",))
    fp = _fingerprint(srcs + hdrs, HIPCC_FLAGS)
    lib = kernels_lib_path()
    if not force and _is_current(lib, fp):
        return lib
    hipcc = _find("hipcc", ["/opt/rocm/bin/hipcc"])
    obj_dir = os.path.join(lib_dir(), "_build", "kernels")
    os.makedirs(obj_dir, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1, len(srcs))
    _log(f"compiling {len(srcs)} HIP sources for {GPU_ARCH} with {jobs} jobs -> {lib}")
    t0 = time.time()

    def one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        _run([hipcc, *HIPCC_FLAGS, "-I", os.path.join(CSRC, "kernels"), "-c", src, "-o", obj],
             f"hipcc {os.path.basename(src)}")
        _log(f"compiled {os.path.basename(src)} ({time.time() - t0:.0f} s)")
        return obj

    with _Ticker("HIP kernels"):
        with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
            objs = list(ex.map(one, srcs))
        tmp = lib + f".tmp{os.getpid()}"
        # hipBLASLt for the products of many rows; a process that has loaded torch holds that library already
        rocm_lib = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(hipcc))), "lib")
        if not os.path.exists(os.path.join(rocm_lib, "libhipblaslt.so")):
            rocm_lib = "/opt/rocm/lib"
        _run([hipcc, f"--offload-arch={GPU_ARCH}", "-shared", "-fPIC", "-o", tmp, *objs,
              f"-L{rocm_lib}", "-lhipblaslt", f"-Wl,-rpath,{rocm_lib}"], "link of the kernel library")
    _finish(lib, tmp, fp)
    _log(f"kernel library ready in {time.time() - t0:.0f} s")
    return lib


def build_host(force: bool = False) -> str:
    srcs = _sources("host", (".cpp",))
    hdrs = _sources("host", (".h",))
    fp = _fingerprint(srcs + hdrs, HOST_FLAGS)
    lib = host_lib_path()
    if not force and _is_current(lib, fp):
        return lib
    cxx = _find("g++", ["/usr/bin/g++"])
    _log(f"compiling the host runtime -> {lib}")
    tmp = lib + f".tmp{os.getpid()}"
    _run([cxx, *HOST_FLAGS, "-shared", "-o", tmp, *srcs], "g++ of the host runtime")
    _finish(lib, tmp, fp)
    return lib


def build_all(force: bool = False) -> None:
    build_host(force)
    build_kernels(force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
    print(kernels_lib_path())
    print(host_lib_path())
