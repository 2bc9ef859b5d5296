"""Builds and loads ``libmicrollm_hip.so``, the HIP kernels of this package.

The library is compiled in-tree with ``hipcc --offload-arch=gfx950`` from the
``.hip`` files under ``csrc``; nothing of torch is compiled against, so a build
takes seconds. ``load()`` builds only when no library that matches the sources
is there, and fails loudly when it cannot: there is no fallback for the kernels.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIBRARY_NAME = "libmicrollm_hip.so"
ARCH = "gfx950"
# Packed float32 instructions are switched off for every kernel of this library.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]

_library: Optional[ctypes.CDLL] = None


class KernelLibraryError(RuntimeError):
    """The HIP library is missing and cannot be built, or a kernel refused its arguments."""


def _sources() -> List[str]:
    return sorted(os.path.join(CSRC, name) for name in os.listdir(CSRC) if name.endswith(".hip"))


def _source_hash() -> str:
    digest = hashlib.sha256()
    for path in _sources() + sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith(".h")):
        digest.update(os.path.basename(path).encode())
        with open(path, "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(HIPCC_FLAGS).encode())
    return digest.hexdigest()


_fallback_dir: Optional[str] = None


def private_temporary_folder() -> str:
    """A folder under the temporary directory that only this user can write: what is loaded from it runs inside
    this process. The folder with the predictable name is taken only if it is a real folder (no link) that this
    user owns and no one else may write; anyone could have made it beforehand otherwise. Failing that a fresh
    folder with a random name is made, which later processes do not find again: they build again."""
    global _fallback_dir
    if _fallback_dir is not None:
        return _fallback_dir
    named = os.path.join(tempfile.gettempdir(), f"microllm_rocm_amd_{os.getuid()}")
    try:
        os.mkdir(named, 0o700)
    except FileExistsError:
        pass
    except OSError:
        named = None
    if named is not None:
        try:
            status = os.lstat(named)
            import stat
            if stat.S_ISDIR(status.st_mode) and status.st_uid == os.getuid() and not status.st_mode & 0o022:
                _fallback_dir = named
                return named
        except OSError:
            pass
    _fallback_dir = tempfile.mkdtemp(prefix="microllm_rocm_amd_")
    return _fallback_dir


def _candidate_dirs() -> List[str]:
    return [CSRC, private_temporary_folder()]


def _find_built() -> Optional[str]:
    wanted = _source_hash()
    for folder in _candidate_dirs():
        library = os.path.join(folder, LIBRARY_NAME)
        stamp = library + ".stamp"
        if os.path.exists(library) and os.path.exists(stamp):
            with open(stamp, "r", encoding="utf-8") as handle:
                if handle.read().strip() == wanted:
                    return library
    return None


def _hipcc() -> str:
    for candidate in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise KernelLibraryError("hipcc was not found; the HIP kernels cannot be built")


def _say(text: str) -> None:
    print(f"[microllm_rocm_amd] {text}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compile every ``.hip`` file for gfx950 and link the library. Returns its path."""
    hipcc = _hipcc()
    target_dir = None
    for folder in _candidate_dirs():
        try:
            os.makedirs(folder, exist_ok=True)
            probe = os.path.join(folder, f".write_probe_{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            target_dir = folder
            break
        except OSError:
            continue
    if target_dir is None:
        raise KernelLibraryError("no writable folder for the HIP library")
    object_dir = os.path.join(target_dir, "_build")
    os.makedirs(object_dir, exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a home for its caches
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    sources = _sources()
    started = time.time()
    if verbose:
        _say(f"compiling {len(sources)} HIP files for {ARCH} into {target_dir}")

    def compile_one(source: str) -> str:
        obj = os.path.join(object_dir, os.path.basename(source)[:-4] + ".o")
        command = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", source, "-o", obj]
        result = subprocess.run(command, env=env, capture_output=True, text=True)
        if result.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {source}:\n{result.stdout}\n{result.stderr}")
        if verbose:
            _say(f"  compiled {os.path.basename(source)} ({time.time() - started:.0f} s)")
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objects = list(pool.map(compile_one, sources))
    library = os.path.join(target_dir, LIBRARY_NAME)
    temporary = library + f".{os.getpid()}.tmp"
    # -z defs: a kernel whose host side the compiler dropped shows up here, not when the library is loaded
    command = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wl,-z,defs", "-o", temporary, *objects]
    result = subprocess.run(command, env=env, capture_output=True, text=True)
    if result.returncode != 0:
        raise KernelLibraryError(f"linking {library} failed:\n{result.stdout}\n{result.stderr}")
    os.replace(temporary, library)
    with open(library + ".stamp", "w", encoding="utf-8") as handle:
        handle.write(_source_hash() + "\n")
    if verbose:
        _say(f"built {library} in {time.time() - started:.0f} s")
    return library


def load() -> ctypes.CDLL:
    """The loaded library; built first if no build matches the sources."""
    global _library
    if _library is not None:
        return _library
    path = _find_built()
    if path is None:
        try:
            path = build()
        except KernelLibraryError:
            raise
        except Exception as error:  # pragma: no cover - a broken toolchain
            raise KernelLibraryError(f"building the HIP kernels failed: {error}") from error
    try:
        _library = ctypes.CDLL(path)
    except OSError as error:
        raise KernelLibraryError(f"cannot load {path}: {error}") from error
    _library.mll_last_error.restype = ctypes.c_char_p
    _library.mll_sample_workspace.restype = ctypes.c_int64
    return _library


def library_path() -> Optional[str]:
    return _find_built()
