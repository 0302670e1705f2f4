"""Compiling and loading the native modules: HIP kernels for gfx950 and the C++ host library.

Each module is one shared library built from a few source files with ``hipcc`` (kernels) or
``g++`` (host code).  A library is named after a hash of its sources and flags, so a library
that is present is always the one its sources describe.  A module is compiled the first time
something asks for it; while a compile runs, a line is printed every few seconds.  Libraries go
to ``csrc/_build`` inside the package, or to a per-user folder under the temporary directory when
the package folder cannot be written.
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
from typing import Dict, List, Optional

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")

HIP_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-shared", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC", "-Wall"]

# module name -> (compiler kind, sources relative to csrc, extra dependencies that enter the hash[, extra flags])
MODULES: Dict[str, tuple] = {
    "elementwise": ("hip", ["kernels/elementwise.hip"], ["kernels/common.h"]),
    "gemm_generic": ("hip", ["kernels/gemm_generic.hip"], ["kernels/common.h"]),
    "attn_generic": ("hip", ["kernels/attn_generic.hip"], ["kernels/common.h"]),
    "gemm_bf16": ("hip", ["kernels/gemm_bf16.hip"], ["kernels/common.h", "kernels/pipeline.h", "kernels/no_alloc.h"]),
    "sampling": ("hip", ["kernels/sampling.hip"], ["kernels/common.h"]),
    "host": ("host", ["host/cache_manager.cpp", "host/scheduler.cpp", "host/c_api.cpp"],
             ["host/cache_manager.h", "host/scheduler.h"]),
}

# matrix-core attention: one module per padded head width, compiled when a model of that width runs
for _width in range(32, 257, 32):
    MODULES[f"attn_bf16_hd{_width}"] = ("hip", ["kernels/attn_bf16.hip"], ["kernels/common.h", "kernels/pipeline.h"],
                                         [f"-DHDP={_width}"])

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _module_hash(name: str) -> str:
    kind, sources, deps = MODULES[name][:3]
    digest = hashlib.sha256()
    digest.update(" ".join((HIP_FLAGS if kind == "hip" else HOST_FLAGS) + _extra_flags(name)).encode())
    for rel in list(sources) + list(deps):
        with open(os.path.join(_CSRC, rel), "rb") as handle:
            digest.update(rel.encode())
            digest.update(handle.read())
    return digest.hexdigest()[:12]


def _extra_flags(name: str) -> List[str]:
    entry = MODULES[name]
    return list(entry[3]) if len(entry) > 3 else []


def _build_dirs() -> List[str]:
    dirs = [os.path.join(_CSRC, "_build")]
    dirs.append(os.path.join(tempfile.gettempdir(), f"vipera_rs_amd_build_{os.getuid()}"))
    return dirs


def library_path(name: str, for_writing: bool = False) -> Optional[str]:
    """Path of the built library of ``name``: an existing one, or where a new one goes."""
    filename = f"{name}-{_module_hash(name)}.so"
    for folder in _build_dirs():
        path = os.path.join(folder, filename)
        if os.path.exists(path) and not for_writing:
            return path
    if not for_writing:
        return None
    for folder in _build_dirs():
        try:
            os.makedirs(folder, exist_ok=True)
            handle, probe = tempfile.mkstemp(dir=folder, prefix=".write_test_")
            os.close(handle)
            os.remove(probe)
            return os.path.join(folder, filename)
        except OSError:
            continue
    raise BuildError("no writable folder for built libraries: tried " + ", ".join(_build_dirs()))


def compile_module(name: str, verbose: bool = True) -> str:
    """Compile ``name`` now (even if a library exists) and return the library's path."""
    kind, sources = MODULES[name][:2]
    target = library_path(name, for_writing=True)
    tmp = f"{target}.{os.getpid()}.tmp"
    if kind == "hip":
        command = [_hipcc()] + HIP_FLAGS
    else:
        command = [os.environ.get("CXX") or shutil.which("g++") or "g++"] + HOST_FLAGS
    command += _extra_flags(name) + ["-o", tmp] + [os.path.join(_CSRC, rel) for rel in sources]
    started = time.time()
    if verbose:
        print(f"[vipera build] compiling {name} ({', '.join(sources)})", file=sys.stderr, flush=True)
    process = subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    output: List[str] = []
    reader = threading.Thread(target=lambda: output.append(process.stdout.read()), daemon=True)
    reader.start()
    while True:
        try:
            process.wait(timeout=10)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(f"[vipera build] still compiling {name} ... {time.time() - started:.0f} s",
                      file=sys.stderr, flush=True)
    reader.join()
    text = "\n".join(line for line in "".join(output).splitlines() if "not a recognized feature" not in line)
    if process.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"compiling {name} failed:\n{' '.join(command)}\n{text}")
    os.replace(tmp, target)
    # libraries of older sources of this module are of no use any more
    folder = os.path.dirname(target)
    for entry in os.listdir(folder):
        if entry.startswith(name + "-") and entry.endswith(".so") and os.path.join(folder, entry) != target:
            try:
                os.remove(os.path.join(folder, entry))
            except OSError:
                pass
    if verbose:
        print(f"[vipera build] built {name} in {time.time() - started:.1f} s", file=sys.stderr, flush=True)
    return target


def load_module(name: str) -> ctypes.CDLL:
    """The loaded library of ``name``; compiled first if no built library matches its sources."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        path = library_path(name)
        if path is None:
            path = compile_module(name)
        try:
            library = ctypes.CDLL(path)
        except OSError as err:
            raise BuildError(f"cannot load {path}: {err}") from None
        _loaded[name] = library
        return library


def build_all(verbose: bool = True, jobs: int = 4) -> Dict[str, str]:
    """Compile every module (always), a few at a time; returns module -> library path."""
    results: Dict[str, str] = {}
    errors: List[str] = []
    names = list(MODULES)
    gate = threading.Semaphore(jobs)

    def work(module: str) -> None:
        with gate:
            try:
                results[module] = compile_module(module, verbose)
            except BuildError as err:
                errors.append(str(err))

    threads = [threading.Thread(target=work, args=(module,)) for module in names]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    if errors:
        raise BuildError("\n\n".join(errors))
    return results
