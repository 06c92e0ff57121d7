"""Compiles the HIP kernels (gfx950) and the host allocators into two shared libraries.

``libkva_hip.so``  - every ``csrc/*.hip`` file, compiled with hipcc for gfx950.
``libkva_host.so`` - ``csrc/host/*.cpp``, plain C++ (no GPU runtime needed to load it).

Libraries are kept in ``<package>/_lib`` when that folder can be written, otherwise in a
per-user folder under the system's temporary directory.  A stamp file holds a hash of the
sources and flags, so a library is rebuilt exactly when a source changed.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from concurrent.futures import TimeoutError as FutureTimeout
from typing import List, Tuple

PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG_DIR, "csrc")
GPU_ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={GPU_ARCH}", "-O3", "-fPIC", "-std=c++17",
    # packed fp32 arithmetic is kept off for every kernel of this package
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results go to ordinary vector registers: the kernels work on them at once
    # (softmax, epilogues) and would otherwise copy every value out of the accumulation registers
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-result", "-Wno-unknown-attributes",
]
# the vendor GEMM library (csrc/gemm_vendor.hip); the process has torch's copy of it loaded already
HIP_LINK_LIBS = ["-lhipblaslt"]
HOST_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-shared"]


class BuildError(RuntimeError):
    pass


def _hip_sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _host_sources() -> List[str]:
    d = os.path.join(CSRC, "host")
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".cpp"))


def _headers() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def _digest(paths: List[str], flags: List[str]) -> str:
    h = hashlib.sha256()
    for p in paths:
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(flags).encode())
    return h.hexdigest()


def _lib_dir_candidates() -> List[str]:
    user = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(PKG_DIR, "_lib"),
            os.path.join(tempfile.gettempdir(), f"kva-lib-{user}")]


def _writable_dir() -> str:
    for d in _lib_dir_candidates():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}")
            with open(probe, "w") as f:
                f.write("x")
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the compiled libraries: tried "
                     + ", ".join(_lib_dir_candidates()))


def _find_current(name: str, digest: str):
    for d in _lib_dir_candidates():
        lib, stamp = os.path.join(d, name), os.path.join(d, name + ".stamp")
        try:
            if os.path.isfile(lib) and open(stamp).read().strip() == digest:
                return lib
        except OSError:
            continue
    return None


def _say(msg: str) -> None:
    print(f"[kva build] {msg}", file=sys.stderr, flush=True)


def _run(cmd: List[str], what: str) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise BuildError(f"{what} failed (exit {proc.returncode}):\n{' '.join(cmd)}\n{proc.stdout}")


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); the HIP "
                     "kernels cannot be compiled")


def hip_digest() -> str:
    return _digest(_hip_sources() + _headers(), HIP_FLAGS + HIP_LINK_LIBS)


def host_digest() -> str:
    return _digest(_host_sources(), HOST_FLAGS)


def build_hip(force: bool = False) -> str:
    """Path of an up-to-date ``libkva_hip.so``; compiles it when needed (or when forced)."""
    name, digest = "libkva_hip.so", hip_digest()
    if not force:
        cur = _find_current(name, digest)
        if cur:
            return cur
    out_dir = _writable_dir()
    hipcc = _hipcc()
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = _hip_sources()
    _say(f"compiling {len(srcs)} HIP sources for {GPU_ARCH} into {out_dir}")
    t0 = time.time()

    def compile_one(src: str) -> Tuple[str, float]:
        t = time.time()
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        _run([hipcc, *HIP_FLAGS, "-I", CSRC, "-c", src, "-o", obj], f"compiling {os.path.basename(src)}")
        return obj, time.time() - t

    objs = []
    workers = max(1, min(8, len(srcs), (os.cpu_count() or 2)))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        futures = [pool.submit(compile_one, s) for s in srcs]
        done = 0
        for s, fut in zip(srcs, futures):
            while True:
                try:
                    obj, dt = fut.result(timeout=20)
                    break
                except FutureTimeout:
                    _say(f"still compiling ({done}/{len(srcs)} done, {time.time() - t0:.0f} s)")
            done += 1
            objs.append(obj)
            _say(f"compiled {os.path.basename(s)} ({dt:.0f} s) [{done}/{len(srcs)}]")
    lib = os.path.join(out_dir, name)
    tmp = lib + f".tmp{os.getpid()}"
    rocm_lib = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(hipcc))), "lib")
    _run([hipcc, f"--offload-arch={GPU_ARCH}", "-shared", "-fPIC", *objs, "-L", rocm_lib, *HIP_LINK_LIBS, "-o", tmp],
         "linking " + name)
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(digest + "\n")
    _say(f"built {name} in {time.time() - t0:.0f} s")
    return lib


def build_host(force: bool = False) -> str:
    """Path of an up-to-date ``libkva_host.so`` (the page pool and the buddy allocator)."""
    name, digest = "libkva_host.so", host_digest()
    if not force:
        cur = _find_current(name, digest)
        if cur:
            return cur
    out_dir = _writable_dir()
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if cxx is None:
        try:
            cxx = _hipcc()
        except BuildError:
            raise BuildError("no C++ compiler found for the host allocators") from None
    lib = os.path.join(out_dir, name)
    tmp = lib + f".tmp{os.getpid()}"
    _say(f"compiling host allocators into {out_dir}")
    _run([cxx, *HOST_FLAGS, *_host_sources(), "-o", tmp], "compiling " + name)
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(digest + "\n")
    return lib


def build_all(force: bool = False) -> Tuple[str, str]:
    return build_host(force), build_hip(force)


if __name__ == "__main__":
    h, g = build_all(force="--force" in sys.argv)
    print(h)
    print(g)
