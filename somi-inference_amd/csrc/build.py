"""Builds the gfx950 kernel library with hipcc and loads it.

The library is one shared object of ``extern "C"`` entry points over raw
device pointers, so it needs no Python or torch headers and a source compiles
in seconds.  It is built in-tree under ``csrc/_build`` (or, when that folder
cannot be written, under the temporary folder), once per change of the
sources, and loaded with ``ctypes``.  There is no fallback: if hipcc is
missing or a source does not compile, loading raises :class:`KernelBuildError`.
"""

from __future__ import annotations

import concurrent.futures
import ctypes
import hashlib
import os
import shutil
import stat
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libsomi_gfx950.so"
OFFLOAD_ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


class KernelBuildError(RuntimeError):
    """The HIP kernel library could not be built or loaded."""


def sources() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))


def source_digest() -> str:
    digest = hashlib.sha256()
    digest.update(" ".join(HIPCC_FLAGS).encode())
    for name in _headers() + sources():
        digest.update(name.encode())
        with open(os.path.join(CSRC, name), "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _candidate_dirs() -> list[str]:
    dirs = [os.path.join(CSRC, "_build")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"somi_inference_amd_build_{uid}"))
    return dirs


def _own_private(path: str) -> bool:
    """A build folder under the shared temporary folder counts only if it is ours and closed to others."""
    if os.path.dirname(path) == CSRC or not hasattr(os, "getuid"):
        return True
    try:
        info = os.lstat(path)
    except OSError:
        return False
    return stat.S_ISDIR(info.st_mode) and info.st_uid == os.getuid() and not (info.st_mode & 0o022)


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, mode=0o700, exist_ok=True)
        if not _own_private(path):
            return False
        probe = os.path.join(path, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def built_library() -> str | None:
    """Path of an up-to-date library, if one was built before."""
    want = source_digest()
    for folder in _candidate_dirs():
        lib, stamp = os.path.join(folder, LIB_NAME), os.path.join(folder, "digest.txt")
        if _own_private(folder) and os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp, "r", encoding="utf-8") as handle:
                if handle.read().strip() == want:
                    return lib
    return None


def _say(text: str) -> None:
    print(f"[somi_inference_amd] {text}", file=sys.stderr, flush=True)


def build(force: bool = False, verbose: bool = True) -> str:
    """Compile every source for gfx950 and link the library; returns its path."""
    if not force:
        ready = built_library()
        if ready:
            return ready
    hipcc = _hipcc()
    folder = next((d for d in _candidate_dirs() if _writable(d)), None)
    if folder is None:
        raise KernelBuildError(f"no writable build folder among {_candidate_dirs()}")
    names = sources()
    started = time.time()
    if verbose:
        _say(f"compiling {len(names)} HIP sources for {OFFLOAD_ARCH} into {folder}")
    stop = threading.Event()

    def heartbeat() -> None:
        while not stop.wait(20.0):
            _say(f"still compiling ({time.time() - started:.0f} s)")

    beat = threading.Thread(target=heartbeat, daemon=True)
    if verbose:
        beat.start()

    def compile_one(name: str) -> str:
        obj = os.path.join(folder, name[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, name), "-o", obj]
        done = subprocess.run(cmd, capture_output=True, text=True)
        if done.returncode != 0:
            raise KernelBuildError(f"hipcc failed on {name}:\n{done.stderr[-4000:]}")
        if verbose:
            _say(f"compiled {name} ({time.time() - started:.0f} s)")
        return obj

    try:
        workers = max(1, min(len(names), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
        with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
            objects = list(pool.map(compile_one, names))
        lib = os.path.join(folder, LIB_NAME)
        tmp = lib + f".{os.getpid()}.tmp"
        link = subprocess.run([hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", *objects, "-o", tmp],
                              capture_output=True, text=True)
        if link.returncode != 0:
            raise KernelBuildError(f"hipcc failed to link {LIB_NAME}:\n{link.stderr[-4000:]}")
        os.replace(tmp, lib)
        with open(os.path.join(folder, "digest.txt"), "w", encoding="utf-8") as handle:
            handle.write(source_digest() + "\n")
    finally:
        stop.set()
    if verbose:
        _say(f"built {LIB_NAME} in {time.time() - started:.0f} s")
    return lib


_LIB: ctypes.CDLL | None = None


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """The loaded library.  Uses what is built; compiles only when nothing (current) is."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = built_library()
    if path is None:
        if not build_if_missing:
            raise KernelBuildError("the HIP kernel library is not built; run __graft_entry__.build()")
        path = build()
    try:
        _LIB = ctypes.CDLL(path)
    except OSError as err:
        raise KernelBuildError(f"cannot load {path}: {err}") from err
    _LIB.somi_last_error.restype = ctypes.c_char_p
    return _LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
