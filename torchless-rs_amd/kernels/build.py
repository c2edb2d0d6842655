"""Compiling the sources into shared libraries, and loading them: the HIP
kernels for gfx950 that a model's step needs (`libtorchless_hip.so`, hipcc), the host
side of cache and step (`libtorchless_host.so`, plain C++, no GPU needed) and the
kernels that only measure the machine (`libtorchless_measure.so`, `csrc/measure/`).

`build()` always compiles all three.  `load()`, `load_host()` and `load_measure()` load
the library that is there if it was built from the sources as they are now (a digest of
sources and flags is kept beside each library), and build that library otherwise: a
model's first step compiles the first two, never the third.  The
libraries go to `csrc/_build/` inside the package; if that cannot be written
(a read-only checkout), to a folder of the user's own (mode 0700) under the
system's temporary directory.
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
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

ARCH = "gfx950"
LIB_NAME = "libtorchless_hip.so"
HOST_LIB_NAME = "libtorchless_host.so"
MEASURE_LIB_NAME = "libtorchless_measure.so"
_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-result"]

HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]

_lib: Optional[ctypes.CDLL] = None
_host_lib: Optional[ctypes.CDLL] = None
_measure_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


class ExtensionMissing(RuntimeError):
    """The HIP library could not be built or loaded; nothing runs without it."""


def _say(msg: str) -> None:
    print(f"[torchless-rs_amd build] {msg}", file=sys.stderr, flush=True)


def sources() -> List[str]:
    return sorted(os.path.join(_CSRC, f) for f in os.listdir(_CSRC) if f.endswith(".hip"))


def measure_sources() -> List[str]:
    d = os.path.join(_CSRC, "measure")
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".hip"))


def host_sources() -> List[str]:
    d = os.path.join(_CSRC, "host")
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".cpp"))


def _headers() -> List[str]:
    return sorted(os.path.join(_CSRC, f) for f in os.listdir(_CSRC) if f.endswith((".hpp", ".h")))


def _digest(files: List[str], flags: List[str]) -> str:
    """What a library depends on: the text of its sources and the compiler's flags."""
    h = hashlib.sha256(" ".join(flags).encode())
    for f in files:
        h.update(os.path.basename(f).encode() + b"\0")
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def kernels_digest() -> str:
    return _digest(sources() + _headers(), HIPCC_FLAGS)


def measure_digest() -> str:
    return _digest(measure_sources() + _headers(), HIPCC_FLAGS)


def host_digest() -> str:
    return _digest(host_sources() + [os.path.join(_CSRC, "page.h")], HOST_FLAGS)


def _write_stamp(lib: str, digest: str) -> None:
    with open(lib + ".stamp", "w") as f:
        f.write(digest + "\n")


def _is_current(lib: str, digest: str) -> bool:
    try:
        with open(lib + ".stamp") as f:
            return f.read().strip() == digest
    except OSError:
        return False


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
    digest = host_digest()
    _run_with_progress([cxx, *HOST_FLAGS, *host_sources(), "-o", tmp], "the host library")
    os.replace(tmp, lib)
    _write_stamp(lib, digest)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def _own_private_dir(path: str) -> bool:
    """Is `path` a folder of this user's that nobody else can write to?"""
    try:
        st = os.stat(path)
    except OSError:
        return False
    return (not hasattr(os, "getuid") or st.st_uid == os.getuid()) and not (st.st_mode & 0o022)


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, mode=0o700, exist_ok=True)
        if path.startswith(tempfile.gettempdir() + os.sep) and not _own_private_dir(path):
            return False                     # a folder under /tmp that someone else made, or may write to
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
    """Compile every source and link all libraries; returns the path of the kernels'."""
    lib = build_kernels(verbose)
    build_measure(verbose)
    return lib


def build_measure(verbose: bool = True) -> str:
    """Compile the library of the measuring kernels; returns its path."""
    return _build_hip(measure_sources(), MEASURE_LIB_NAME, measure_digest(), verbose)


def build_kernels(verbose: bool = True) -> str:
    """Compile the host library and the kernels that a step needs; returns the path of the kernels'."""
    build_host(verbose)
    return _build_hip(sources(), LIB_NAME, kernels_digest(), verbose)


def _build_hip(srcs: List[str], name: str, digest: str, verbose: bool) -> str:
    hipcc = find_hipcc()
    out_dir = next((d for d in build_dirs() if _writable_dir(d)), None)
    if out_dir is None:
        raise ExtensionMissing(f"no writable build folder among {build_dirs()}")
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
    lib = os.path.join(out_dir, name)
    tmp = lib + f".tmp{os.getpid()}"
    _run_with_progress([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp], "link")
    os.replace(tmp, lib)
    _write_stamp(lib, digest)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def built_library(name: str = LIB_NAME, digest: Optional[str] = None) -> Optional[str]:
    """The library `name` if one is there: in the package's own folder, or in this user's
    private folder under the temporary directory (never in one that others can write to).
    With `digest`, one that was built from the sources of that digest goes before one that was
    not, wherever it lies: a stale library in a package folder that cannot be written must not
    hide the current one that an earlier process built into the private folder."""
    pkg, tmp = build_dirs()
    found = [p for d in (pkg, tmp) for p in [os.path.join(d, name)]
             if os.path.isfile(p) and (d == pkg or _own_private_dir(d))]
    if digest is not None:
        for p in found:
            if _is_current(p, digest):
                return p
    return found[0] if found else None


def _current_or_rebuilt(path: Optional[str], digest: str, rebuild, what: str) -> str:
    """`path` if it was built from the sources as they are; else a fresh build.  A library that is
    older than its sources is never loaded: a run would then test other kernels than it shows."""
    if path is not None and _is_current(path, digest):
        return path
    if path is not None:
        _say(f"{what} at {path} was not built from the present sources; building again")
    try:
        return rebuild()
    except ExtensionMissing as e:
        if path is None:
            raise
        raise ExtensionMissing(f"{path} is older than its sources and cannot be built again: {e}") from None


def load() -> ctypes.CDLL:
    """The library, built first if there is none."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        digest = kernels_digest()
        path = _current_or_rebuilt(built_library(LIB_NAME, digest), digest, build_kernels, "the kernels' library")
        try:
            _lib = ctypes.CDLL(path)
        except OSError as e:
            raise ExtensionMissing(f"cannot load {path}: {e}") from None
        return _lib


def load_measure() -> ctypes.CDLL:
    """The library of the measuring kernels, built first if there is none."""
    global _measure_lib
    with _lock:
        if _measure_lib is not None:
            return _measure_lib
        digest = measure_digest()
        path = _current_or_rebuilt(built_library(MEASURE_LIB_NAME, digest), digest, build_measure,
                                   "the measuring kernels' library")
        try:
            _measure_lib = ctypes.CDLL(path)
        except OSError as e:
            raise ExtensionMissing(f"cannot load {path}: {e}") from None
        return _measure_lib


def load_host() -> ctypes.CDLL:
    """The host library, built first if there is none."""
    global _host_lib
    with _lock:
        if _host_lib is not None:
            return _host_lib
        digest = host_digest()
        path = _current_or_rebuilt(built_library(HOST_LIB_NAME, digest), digest, build_host, "the host library")
        try:
            _host_lib = ctypes.CDLL(path)
        except OSError as e:
            raise ExtensionMissing(f"cannot load {path}: {e}") from None
        return _host_lib
