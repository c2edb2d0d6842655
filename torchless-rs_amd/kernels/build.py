"""Compiling the sources into two shared libraries, and loading them: the HIP
kernels for gfx950 (`libtorchless_hip.so`, hipcc) and the host side of cache
and step (`libtorchless_host.so`, plain C++, no GPU needed).

`build()` always compiles both.  `load()` and `load_host()` load the library
that is there and build only if none is.  The libraries go to `csrc/_build/`
inside the package; if that cannot be written (a read-only checkout), to a
folder of the user's own under the system's temporary directory.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

ARCH = "gfx950"
LIB_NAME = "libtorchless_hip.so"
HOST_LIB_NAME = "libtorchless_host.so"
_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-result"]

_lib: Optional[ctypes.CDLL] = None
_host_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


class ExtensionMissing(RuntimeError):
    """The HIP library could not be built or loaded; nothing runs without it."""


def _say(msg: str) -> None:
    print(f"[torchless-rs_amd build] {msg}", file=sys.stderr, flush=True)


def sources() -> List[str]:
    return sorted(os.path.join(_CSRC, f) for f in os.listdir(_CSRC) if f.endswith(".hip"))


def host_sources() -> List[str]:
    d = os.path.join(_CSRC, "host")
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".cpp"))


def find_cxx() -> str:
    for c in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
              "/opt/rocm/llvm/bin/clang++"):
        if c and (os.path.isfile(c) or shutil.which(c)):
            return c
    raise ExtensionMissing("no C++ compiler found (looked at $CXX, g++, c++, clang++)")


def build_host(verbose: bool = True) -> str:
    """Compile the host library; returns its path."""
    cxx = find_cxx()
    out_dir = next((d for d in build_dirs() if _writable_dir(d)), None)
    if out_dir is None:
        raise ExtensionMissing(f"no writable build folder among {build_dirs()}")
    lib = os.path.join(out_dir, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    t0 = time.time()
    _run_with_progress([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", *host_sources(), "-o", tmp],
                       "the host library")
    os.replace(tmp, lib)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dirs() -> List[str]:
    """Where a built library may be, in the order of preference."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(_CSRC, "_build"),
            os.path.join(tempfile.gettempdir(), f"torchless_rs_amd_build_{uid}")]


def find_hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.isfile(c):
            return c
    raise ExtensionMissing("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _run_with_progress(cmd: List[str], what: str) -> None:
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    done = threading.Event()

    def tick():
        while not done.wait(15.0):
            _say(f"still compiling {what} ({time.time() - t0:.0f} s)")

    th = threading.Thread(target=tick, daemon=True)
    th.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise ExtensionMissing(f"hipcc failed on {what}:\n{out}")
    noise = "is not a recognized feature for this target"
    rest = [l for l in out.splitlines() if l.strip() and noise not in l]
    if rest:
        _say(f"{what}: " + "\n".join(rest))


def build(verbose: bool = True) -> str:
    """Compile every source and link both libraries; returns the path of the kernels'."""
    build_host(verbose)
    hipcc = find_hipcc()
    out_dir = next((d for d in build_dirs() if _writable_dir(d)), None)
    if out_dir is None:
        raise ExtensionMissing(f"no writable build folder among {build_dirs()}")
    srcs = sources()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    objs = [os.path.join(out_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    t0 = time.time()

    def one(i: int) -> None:
        _run_with_progress([hipcc, *HIPCC_FLAGS, "-I", _CSRC, "-c", srcs[i], "-o", objs[i]],
                           os.path.basename(srcs[i]))
        if verbose:
            _say(f"compiled {os.path.basename(srcs[i])} ({time.time() - t0:.0f} s)")

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(one, range(len(srcs))))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    _run_with_progress([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp], "link")
    os.replace(tmp, lib)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def built_library(name: str = LIB_NAME) -> Optional[str]:
    for d in build_dirs():
        p = os.path.join(d, name)
        if os.path.isfile(p):
            return p
    return None


def _warn_if_stale(lib: str, srcs: Optional[List[str]] = None) -> None:
    try:
        srcs = srcs or [os.path.join(_CSRC, f) for f in os.listdir(_CSRC) if f.endswith((".hip", ".hpp"))]
        newest = max(os.path.getmtime(f) for f in srcs)
        if newest > os.path.getmtime(lib) + 1.0:
            _say(f"warning: a source is newer than {lib}; build again to pick it up")
    except OSError:
        pass


def load() -> ctypes.CDLL:
    """The library, built first if there is none."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = built_library()
        if path is None:
            path = build()
        else:
            _warn_if_stale(path)
        try:
            _lib = ctypes.CDLL(path)
        except OSError as e:
            raise ExtensionMissing(f"cannot load {path}: {e}") from None
        return _lib


def load_host() -> ctypes.CDLL:
    """The host library, built first if there is none."""
    global _host_lib
    with _lock:
        if _host_lib is not None:
            return _host_lib
        path = built_library(HOST_LIB_NAME)
        if path is None:
            path = build_host()
        else:
            _warn_if_stale(path, host_sources())
        try:
            _host_lib = ctypes.CDLL(path)
        except OSError as e:
            raise ExtensionMissing(f"cannot load {path}: {e}") from None
        return _host_lib
