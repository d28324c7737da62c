"""Builds and loads the native libraries of this package: the HIP kernels (gfx950
only) and the host-side bookkeeping of the cache and of a step (`host.cpp`, C++
without GPU code, compiled with the host compiler).

Every `.hip` file here becomes one shared library, compiled with hipcc the
first time something needs it and loaded with ctypes.  A library is rebuilt
when the text of its sources or the flags change (a content hash lies beside
it), so a fresh checkout compiles exactly what the running model touches and a
built tree loads without compiling.  Libraries are written next to the sources
(`csrc/lib/`) so that they travel with the tree; if that folder cannot be
written, a per-user folder under the temporary directory is used instead.
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
from typing import Dict, List

_HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
LIBRARIES: Dict[str, List[str]] = {
    "elementwise": ["elementwise.hip"],
    "norm": ["norm.hip"],
    "rope_kv": ["rope_kv.hip"],
    "attention": ["attention.hip"],
    "gemm": ["gemm.hip"],
    "sampling": ["sampling.hip"],
    "probe": ["probe.hip"],
}
# libraries without GPU code: compiled with the host's C++ compiler
HOST_LIBRARIES: Dict[str, List[str]] = {"host": ["host.cpp"]}
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared"]
HEADERS = ["common.h"]
# headers that only one library includes
OWN_HEADERS: Dict[str, List[str]] = {"sampling": ["sampling.h"]}
# packed 32-bit float instructions are switched off on purpose (device flag); the first kernel
# arguments come preloaded into scalar registers with the dispatch instead of being loaded by the
# kernel's first instructions (every kernel here is short enough for that to count: measured
# 0.3-0.6 % of a decode step at batch 1, 8 and 64; kernels keep the loading prologue for firmware
# that does not preload)
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-mllvm",
    "-amdgpu-kernarg-preload-count=16",
]

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    exe = shutil.which("hipcc")
    if exe:
        return exe
    for cand in ("/opt/rocm/bin/hipcc",):
        if os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels of litellmengine_amd cannot be compiled")


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe.{os.getpid()}")
        with open(probe, "w"):
            pass
        os.unlink(probe)
        return True
    except OSError:
        return False


_lib_dir = None
_lib_dir_lock = threading.Lock()


def lib_dir() -> str:
    global _lib_dir
    with _lib_dir_lock:
        if _lib_dir is None:
            in_tree = os.path.join(_HERE, "lib")
            fallback = os.path.join(tempfile.gettempdir(), f"litellmengine_amd-{os.getuid()}", "lib")
            if _writable_dir(in_tree):
                _lib_dir = in_tree
            elif _writable_dir(fallback):
                _lib_dir = fallback
            else:
                raise BuildError(f"neither {in_tree} nor {fallback} can be written")
        return _lib_dir


def _host_compiler() -> str:
    for cand in ("g++", "c++", "clang++"):
        exe = shutil.which(cand)
        if exe:
            return exe
    return _hipcc()  # compiles plain C++ as well


def _source_hash(name: str) -> str:
    h = hashlib.sha256()
    host = name in HOST_LIBRARIES
    h.update(" ".join(HOST_FLAGS if host else FLAGS).encode())
    for fn in (HOST_LIBRARIES[name] if host else HEADERS + OWN_HEADERS.get(name, []) + LIBRARIES[name]):
        with open(os.path.join(_HERE, fn), "rb") as f:
            h.update(fn.encode())
            h.update(f.read())
    return h.hexdigest()


def _paths(name: str, directory: str):
    return os.path.join(directory, f"liblle_{name}.so"), os.path.join(directory, f"liblle_{name}.hash")


def _find_built(name: str):
    """Path of an up-to-date library, or None."""
    want = _source_hash(name)
    dirs = [os.path.join(_HERE, "lib"), os.path.join(tempfile.gettempdir(), f"litellmengine_amd-{os.getuid()}", "lib")]
    for d in dirs:
        so, hs = _paths(name, d)
        try:
            with open(hs) as f:
                if f.read().strip() == want and os.path.isfile(so):
                    return so
        except OSError:
            continue
    return None


def compile_library(name: str, verbose: bool = True) -> str:
    """Compile one library now (whether or not a built one exists)."""
    if name not in LIBRARIES and name not in HOST_LIBRARIES:
        raise BuildError(f"unknown library {name!r}")
    directory = lib_dir()
    so, hs = _paths(name, directory)
    tmp = f"{so}.{os.getpid()}.{threading.get_ident()}.tmp"
    if name in HOST_LIBRARIES:
        cmd = [_host_compiler()] + HOST_FLAGS + [os.path.join(_HERE, s) for s in HOST_LIBRARIES[name]] + ["-o", tmp]
        what = f"host library '{name}'"
    else:
        cmd = [_hipcc()] + FLAGS + [os.path.join(_HERE, s) for s in LIBRARIES[name]] + ["-o", tmp]
        what = f"kernels '{name}' for {ARCH}"
    if verbose:
        print(f"[litellmengine_amd] compiling {what} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=_HERE, env=env)
    out_chunks: List[str] = []
    reader = threading.Thread(target=lambda: out_chunks.append(proc.stdout.read()), daemon=True)
    reader.start()
    while True:
        try:
            proc.wait(timeout=10)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(
                    f"[litellmengine_amd] still compiling '{name}' ({time.time() - t0:.0f} s)",
                    file=sys.stderr,
                    flush=True,
                )
    reader.join()
    output = "".join(out_chunks)
    if proc.returncode != 0:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise BuildError(f"{cmd[0]} failed for '{name}':\n{output}")
    os.replace(tmp, so)
    with open(hs + ".tmp", "w") as f:
        f.write(_source_hash(name))
    os.replace(hs + ".tmp", hs)
    if verbose:
        print(f"[litellmengine_amd] built {so} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return so


def build_all(verbose: bool = True, jobs: int = 4) -> None:
    """Compile every library, in parallel; always compiles."""
    names = list(LIBRARIES) + list(HOST_LIBRARIES)
    errors: List[BaseException] = []
    sem = threading.Semaphore(jobs)

    def work(n):
        with sem:
            try:
                compile_library(n, verbose)
            except BaseException as e:  # noqa: BLE001
                errors.append(e)

    threads = [threading.Thread(target=work, args=(n,)) for n in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]


def load_library(name: str) -> ctypes.CDLL:
    """The loaded library, compiled first if no up-to-date build exists."""
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        so = _find_built(name) or compile_library(name)
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise BuildError(f"cannot load {so}: {e}") from e
        lib.lle_error_string.restype = ctypes.c_char_p
        lib.lle_error_string.argtypes = [ctypes.c_int]
        _loaded[name] = lib
        return lib
