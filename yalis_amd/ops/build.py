"""Compiling and loading the native libraries.

Shared libraries are built from ``yalis_amd/csrc``: the host-side cache manager (C++, g++)
and the HIP kernels for gfx950 (hipcc) in three libraries, each built when first needed: the
kernels of a model step, those that choose tokens, and the benchmark's probes.  All expose a
plain C interface and are loaded with ctypes.  Built files go into ``yalis_amd/csrc/_build`` when that
is writable, else into a per-user folder under the system's temporary directory.
``load_*`` builds on first use when no library matching the sources is there, and
prints a line now and then while the compiler runs.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, List, Sequence

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")

HOST_SOURCES = ["cache_manager.cpp"]
# Libraries of HIP kernels, each built and loaded when first needed: a model step needs
# "kernels" only (so that is all a trace replay compiles), choosing tokens "sampling", the
# benchmark's machine probes "probe".  Every library carries runtime.hip (its error slot).
KERNEL_LIBS = {
    "kernels": ["runtime.hip", "elementwise.hip", "gemm.hip", "gemm_tile.hip", "attention.hip", "library_gemm.hip"],
    "sampling": ["runtime.hip", "sampling.hip"],
    "probe": ["runtime.hip", "probe.hip"],
}
HEADERS = ["common.h", "no_alloc.h"]
# what a library links beside the HIP runtime: the vendor's matrix products for many rows
LINK_LIBS = {"kernels": ["-lhipblaslt"]}

HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

_lock = threading.Lock()
_loaded: Dict[str, ctypes.CDLL] = {}


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[yalis_amd build] {msg}", file=sys.stderr, flush=True)


def build_dir() -> str:
    env = os.environ.get("YALIS_AMD_BUILD_DIR")
    if env:
        os.makedirs(env, exist_ok=True)
        return env
    intree = os.path.join(CSRC, "_build")
    try:
        os.makedirs(intree, exist_ok=True)
        probe = os.path.join(intree, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return intree
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"yalis_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _digest(sources: Sequence[str], flags: Sequence[str]) -> str:
    h = hashlib.sha256()
    for name in list(sources) + HEADERS:
        path = os.path.join(CSRC, name)
        if os.path.isfile(path):
            h.update(name.encode())
            with open(path, "rb") as f:
                h.update(f.read())
    h.update(" ".join(flags).encode())
    return h.hexdigest()[:16]


def _run(cmd: List[str], what: str) -> None:
    start = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            _say(f"still compiling {what} ({int(time.time() - start)} s)")

    t = threading.Thread(target=ticker, daemon=True)
    t.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n$ {' '.join(cmd)}\n{out}")


def _find(tool: str, fallbacks: Sequence[str]) -> str:
    path = shutil.which(tool)
    if path:
        return path
    for f in fallbacks:
        if os.path.isfile(f):
            return f
    raise BuildError(f"{tool} not found (looked on PATH and in {list(fallbacks)})")


def _stamp_path(lib: str) -> str:
    return lib + ".stamp"


def _is_current(lib: str, digest: str) -> bool:
    try:
        with open(_stamp_path(lib)) as f:
            return os.path.isfile(lib) and f.read().strip() == digest
    except OSError:
        return False


def _write_stamp(lib: str, digest: str) -> None:
    with open(_stamp_path(lib), "w") as f:
        f.write(digest)


def build_host(force: bool = False) -> str:
    """The cache manager (host C++)."""
    flags = ["-O2", "-std=c++17", "-fPIC", "-shared"]
    digest = _digest(HOST_SOURCES, flags)
    lib = os.path.join(build_dir(), "libyalis_host.so")
    if not force and _is_current(lib, digest):
        return lib
    cxx = _find("g++", ["/usr/bin/g++", "/opt/rocm/llvm/bin/clang++"])
    _say("compiling the cache manager (host C++)")
    tmp = f"{lib}.{os.getpid()}.tmp"
    _run([cxx, *flags, "-o", tmp, *[os.path.join(CSRC, s) for s in HOST_SOURCES]], "cache manager")
    os.replace(tmp, lib)
    _write_stamp(lib, digest)
    return lib


def build_kernels(name: str = "kernels", force: bool = False) -> str:
    """One library of HIP kernels for gfx950: one object per source, compiled side by side."""
    sources = KERNEL_LIBS[name]
    digest = _digest(sources, HIPCC_FLAGS + LINK_LIBS.get(name, []))
    bdir = build_dir()
    lib = os.path.join(bdir, f"libyalis_{name}.so")
    if not force and _is_current(lib, digest):
        return lib
    hipcc = _find("hipcc", ["/opt/rocm/bin/hipcc"])
    _say(f"compiling {len(sources)} HIP sources for gfx950 (library '{name}'; the largest takes about a minute)")
    objs: List[str] = []
    errors: List[BaseException] = []

    def one(src: str, obj: str) -> None:
        try:
            _run([hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj], src)
            _say(f"compiled {src}")
        except BaseException as e:  # noqa: BLE001 - reported below
            errors.append(e)

    threads = []
    for src in sources:
        obj = os.path.join(bdir, f"{name}_{os.path.splitext(src)[0]}.{os.getpid()}.o")
        objs.append(obj)
        th = threading.Thread(target=one, args=(src, obj))
        th.start()
        threads.append(th)
    for th in threads:
        th.join()
    if errors:
        for o in objs:
            if os.path.exists(o):
                os.remove(o)
        raise errors[0]
    tmp = f"{lib}.{os.getpid()}.tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs, *LINK_LIBS.get(name, [])], "link")
    for o in objs:
        os.remove(o)
    os.replace(tmp, lib)
    _write_stamp(lib, digest)
    _say(f"library '{name}' built")
    return lib


def build_all(force: bool = True) -> None:
    build_host(force=force)
    for name in KERNEL_LIBS:
        build_kernels(name, force=force)


def load_host() -> ctypes.CDLL:
    with _lock:
        if "host" not in _loaded:
            _loaded["host"] = ctypes.CDLL(build_host())
        return _loaded["host"]


def load_kernels(name: str = "kernels") -> ctypes.CDLL:
    with _lock:
        if name not in _loaded:
            _loaded[name] = ctypes.CDLL(build_kernels(name))
        return _loaded[name]
