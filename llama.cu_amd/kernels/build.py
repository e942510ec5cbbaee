"""Building and loading the native libraries.

Each ``.hip`` file under ``csrc/kernels`` becomes one shared library for gfx950, and
``csrc/host`` (the cache manager and the scheduler, plain C++) becomes one more.  A
library is built the first time something asks for it and is kept in ``csrc/_build``
under a name that holds a hash of its sources and flags: a changed source builds
again, an unchanged one is loaded as it is.  There is no fallback: without the
library, and without ``hipcc`` to build it, loading raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, List

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
_KERNEL_DIR = os.path.join(_CSRC, "kernels")
_HOST_DIR = os.path.join(_CSRC, "host")
_REF_DIR = os.path.join(_CSRC, "ref")               # plain C++ references of the kernels, part of the host library
_SHARED_DIR = os.path.join(_CSRC, "shared")       # headers that the host library and kernels both compile

# packed 32-bit float instructions stay off for all device code
HIP_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-shared", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", "-pthread", "-ffp-contract=off"]
# extra flags for experiments (they enter the hash in the libraries' names)
HIP_FLAGS += os.environ.get("LCU_HIP_FLAGS", "").split()

KERNEL_LIBRARIES = ["elementwise", "rope_kv", "attention_generic", "attention_mfma", "gemm_generic", "gemm_skinny",
                    "gemm_mid", "sampling", "random_fill"]
HOST_LIBRARY = "host"

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[llama.cu_amd] {msg}", file=sys.stderr, flush=True)


def _sources(name: str) -> List[str]:
    if name == HOST_LIBRARY:
        return sorted(os.path.join(d, f) for d in (_HOST_DIR, _REF_DIR) for f in os.listdir(d) if f.endswith(".cpp"))
    path = os.path.join(_KERNEL_DIR, name + ".hip")
    if not os.path.isfile(path):
        raise BuildError(f"no kernel source {path}")
    return [path]


_INCLUDE = re.compile(r'^\s*#\s*include\s+"([^"]+)"', re.M)


def _headers(name: str) -> List[str]:
    """The project's own headers that the library's sources include, directly or through one
    another (``#include "..."``, relative to the file that names them): a change of one of them
    builds the library again, a change of any other header does not."""
    seen: Dict[str, None] = {}
    todo = list(_sources(name))
    while todo:
        path = todo.pop()
        with open(path) as f:
            text = f.read()
        for inc in _INCLUDE.findall(text):
            h = os.path.normpath(os.path.join(os.path.dirname(path), inc))
            if h not in seen and os.path.isfile(h):
                seen[h] = None
                todo.append(h)
    return sorted(seen)


def _digest(name: str) -> str:
    h = hashlib.sha256()
    flags = HOST_FLAGS if name == HOST_LIBRARY else HIP_FLAGS
    h.update(" ".join(flags).encode())
    for p in _sources(name) + _headers(name):
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _build_dirs() -> List[str]:
    """Where a built library may lie: in the tree first, else a per-user folder (for a
    tree that this user cannot write)."""
    dirs = [os.path.join(_CSRC, "_build")]
    dirs.append(os.path.join(tempfile.gettempdir(), f"llama_cu_amd_build_{os.getuid()}"))
    return dirs


def library_path(name: str) -> str:
    """The path where the library for the current sources lies or would be built."""
    fname = f"{name}-{_digest(name)}.so"
    for d in _build_dirs():
        p = os.path.join(d, fname)
        if os.path.isfile(p):
            return p
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            if os.access(d, os.W_OK):
                return os.path.join(d, fname)
        except OSError:
            continue
    raise BuildError("no writable folder for built libraries")


def _compiler(name: str) -> str:
    if name == HOST_LIBRARY:
        cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
        if not cxx:
            raise BuildError("no C++ compiler (g++) found to build the host library")
        return cxx
    hipcc = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)
    if not hipcc:
        raise BuildError(f"the kernel library {name!r} is not built and hipcc was not found to build it")
    return hipcc


def build(name: str, force: bool = False) -> str:
    """Compile one library if it is missing (or always with ``force``); returns its path."""
    out = library_path(name)
    if os.path.isfile(out) and not force:
        return out
    cc = _compiler(name)
    flags = HOST_FLAGS if name == HOST_LIBRARY else HIP_FLAGS
    tmp = f"{out}.tmp{os.getpid()}"
    cmd = [cc] + flags + ["-o", tmp] + _sources(name)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())      # hipcc wants a home for its caches
    t0 = time.time()
    _say(f"compiling {name} ...")
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    done = threading.Event()

    def ticker():
        while not done.wait(15):
            _say(f"still compiling {name} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    try:
        log, _ = proc.communicate()
    finally:
        done.set()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"building {name} failed ({' '.join(cmd)}):\n{log}")
    os.replace(tmp, out)
    # older builds of the same library are of no use any more
    for f in os.listdir(os.path.dirname(out)):
        if f.startswith(name + "-") and f.endswith(".so") and f != os.path.basename(out):
            try:
                os.remove(os.path.join(os.path.dirname(out), f))
            except OSError:
                pass
    _say(f"built {name} in {time.time() - t0:.1f} s")
    return out


def build_all(force: bool = True) -> List[str]:
    """Compile every library (what ``__graft_entry__.build()`` calls)."""
    names = [n for n in KERNEL_LIBRARIES if os.path.isfile(os.path.join(_KERNEL_DIR, n + ".hip"))]
    names.append(HOST_LIBRARY)
    paths: Dict[str, str] = {}
    errors: List[str] = []

    def work(n):
        try:
            paths[n] = build(n, force=force)
        except Exception as e:   # collected and raised together below
            errors.append(f"{n}: {e}")
    threads = [threading.Thread(target=work, args=(n,)) for n in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise BuildError("\n".join(errors))
    return [paths[n] for n in names]


def load(name: str) -> ctypes.CDLL:
    """The loaded library ``name``, built first if need be."""
    with _lock:
        lib = _loaded.get(name)
        if lib is None:
            if name != HOST_LIBRARY:
                import torch  # noqa: F401  the HIP runtime that torch loads is the one the kernels must share
            lib = ctypes.CDLL(build(name))
            _loaded[name] = lib
        return lib
