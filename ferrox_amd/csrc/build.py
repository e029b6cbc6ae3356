"""Compiles and loads the native libraries: HIP kernels and the host runtime.

Every `<name>.hip` beside this file becomes one shared object `_lib/<name>.so`,
built with hipcc for gfx950 and loaded through ctypes; `host_runtime.cpp` (cache
book-keeping and step packing, no GPU code) is built with the host compiler.  A library is compiled
when it is first asked for and no object built from the same sources and flags
is there (a hash of both is kept beside the object), so a model compiles what
its parts need and nothing else.  While hipcc runs, a line is printed every few
seconds.  Nothing here falls back to another implementation: without the
library the call that needs it raises.
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

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC"]
HOST_LIBRARIES = ("host_runtime",)
KERNEL_LIBRARIES = ("elementwise", "gemm", "attention", "moe", "sampling")      # what parts of a model may name
# kernels for measurement only (a streaming read, a copy, a loop of MFMA products, a marker): bench.py loads them,
# no model can ask for them; their sources lie in measure/
MEASUREMENT_LIBRARIES = ("probe",)
LIBRARIES = KERNEL_LIBRARIES + MEASUREMENT_LIBRARIES + HOST_LIBRARIES            # what `compile_all` builds
HEADERS = ("common.h",)

_loaded: dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str | None:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _host_compiler() -> str | None:
    for cand in (os.environ.get("CXX"), "g++", "c++", "clang++"):
        path = shutil.which(cand) if cand else None
        if path:
            return path
    return _hipcc()          # hipcc compiles plain C++ for the host as well


def _sources(name: str) -> tuple:
    """The file that is compiled first, then what it includes (all of it goes into the hash)."""
    if name in HOST_LIBRARIES:
        return (name + ".cpp",)
    if name in MEASUREMENT_LIBRARIES:
        return (os.path.join("measure", name + ".hip"),) + HEADERS
    own = (name + ".h",) if os.path.isfile(os.path.join(HERE, name + ".h")) else ()
    return (name + ".hip",) + HEADERS + own


def _source_hash(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(HOST_FLAGS if name in HOST_LIBRARIES else FLAGS).encode())
    for f in _sources(name):
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _lib_dirs() -> list[str]:
    """In-tree first (it travels with the checkout); a per-user temporary folder
    if the tree cannot be written."""
    dirs = [os.path.join(HERE, "_lib")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"ferrox_amd_lib_{uid}"))
    return dirs


def _find_built(name: str, want_hash: str) -> str | None:
    for d in _lib_dirs():
        so, tag = os.path.join(d, name + ".so"), os.path.join(d, name + ".hash")
        if os.path.isfile(so) and os.path.isfile(tag):
            try:
                with open(tag) as f:
                    if f.read().strip() == want_hash:
                        return so
            except OSError:
                pass
    return None


def _writable_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            fd, probe = tempfile.mkstemp(prefix=".probe_", dir=d)      # a name of its own for every caller
            os.close(fd)
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelBuildError("no writable folder for the kernel libraries: tried " + ", ".join(_lib_dirs()))


def compile_library(name: str, verbose: bool = True) -> str:
    """Run hipcc for one library, whatever is already built; returns the path of the object."""
    if name not in LIBRARIES:
        raise KernelBuildError(f"unknown kernel library '{name}'")
    host = name in HOST_LIBRARIES
    compiler = _host_compiler() if host else _hipcc()
    if compiler is None:
        raise KernelBuildError(f"library '{name}' is not built and no {'C++ compiler' if host else 'hipcc'} was found")
    out_dir = _writable_dir()
    so = os.path.join(out_dir, name + ".so")
    tmp = os.path.join(out_dir, f".{name}.{os.getpid()}.{threading.get_ident()}.so")
    cmd = [compiler] + (HOST_FLAGS if host else FLAGS + ["-I", HERE]) + [os.path.join(HERE, _sources(name)[0]), "-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)   # hipcc wants a home for its temporary files
    t0 = time.time()
    if verbose:
        print(f"[ferrox_amd] compiling library '{name}' for {'the host' if host else ARCH} ...", file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=out_dir)
    result: dict = {}

    def pump():
        result["out"] = proc.communicate()[0]

    th = threading.Thread(target=pump, daemon=True)
    th.start()
    while th.is_alive():
        th.join(timeout=10.0)
        if th.is_alive() and verbose:
            print(f"[ferrox_amd] ... still compiling '{name}' ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)
    text = (result.get("out") or b"").decode(errors="replace")
    if proc.returncode != 0:
        try:
            os.remove(tmp)
        except OSError:
            pass
        raise KernelBuildError(f"{os.path.basename(compiler)} failed for '{name}' (exit {proc.returncode}):\n{text}")
    os.replace(tmp, so)
    with open(os.path.join(out_dir, name + ".hash"), "w") as f:
        f.write(_source_hash(name))
    if verbose:
        print(f"[ferrox_amd] built '{name}' in {time.time() - t0:.1f} s -> {so}", file=sys.stderr, flush=True)
    return so


def compile_all(verbose: bool = True) -> None:
    for name in LIBRARIES:
        compile_library(name, verbose)


def ensure_built(names, verbose: bool = True) -> None:
    """Compile those of `names` (libraries that a model's parts name, and the host runtime) that have no current
    object, several at a time."""
    for n in names:
        if n not in KERNEL_LIBRARIES + HOST_LIBRARIES:
            raise KernelBuildError(f"'{n}' is not a kernel library that a part may name (those are: "
                                   f"{', '.join(KERNEL_LIBRARIES)})")
    todo = [n for n in names if _find_built(n, _source_hash(n)) is None]
    if not todo:
        return
    errors = []

    def work(n):
        try:
            compile_library(n, verbose)
        except Exception as e:  # reported below, from the calling thread
            errors.append(e)

    threads = [threading.Thread(target=work, args=(n,)) for n in todo]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]


def load_library(name: str) -> ctypes.CDLL:
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        so = _find_built(name, _source_hash(name))
        if so is None:
            so = compile_library(name)
        lib = ctypes.CDLL(so)
        if name not in HOST_LIBRARIES:
            lib.fx_last_error.restype = ctypes.c_char_p
        _loaded[name] = lib
        return lib
