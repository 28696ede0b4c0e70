"""Builds and loads the native libraries.

Each ``csrc/<module>.hip`` becomes one shared library ``_lib/<module>.so`` compiled with
hipcc for gfx950; each ``csrc/host/<module>.cpp`` (host code that never touches a device: the
cache manager's bookkeeping) one compiled with the host's C++ compiler.  A library is built
when it is first needed and its sources have changed (or it is missing); the build prints a
line now and then so that a first call that compiles does not look hung.  When the package
folder cannot be written the libraries go to a per-user folder under the system's temporary
directory.
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
from typing import Dict, Iterable, List, Optional

from ..errors import KernelUnavailable

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
MODULES = ("elementwise", "gemm", "attention", "sampling", "randinit")
HOST_MODULES = ("cache_core",)
HEADERS = ("zf_common.h", "zf_no_alloc.h")
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]
# -packed-fp32-ops off: hipcc must not form packed 32-bit float instructions by itself
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]

_libs: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()
_dir_lock = threading.Lock()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelUnavailable("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                            "the HIP kernels cannot be built")


def _host_compiler() -> str:
    for cand in (os.environ.get("CXX"), "g++", "c++", "clang++"):
        path = shutil.which(cand) if cand else None
        if path:
            return path
    return _hipcc()          # it compiles plain C++ as well


def _source_hash(module: str) -> str:
    h = hashlib.sha256()
    if module in HOST_MODULES:
        with open(os.path.join(CSRC, "host", module + ".cpp"), "rb") as f:
            h.update(f.read())
        h.update(" ".join(HOST_FLAGS).encode())
        return h.hexdigest()
    for name in (module + ".hip",) + HEADERS:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


_lib_dir: Optional[str] = None


def lib_dir() -> str:
    """Where built libraries live: ``zinfer_amd/_lib`` if it can be written, else a per-user
    temporary folder."""
    global _lib_dir
    if _lib_dir is not None:
        return _lib_dir
    with _dir_lock:
        if _lib_dir is not None:
            return _lib_dir
        pkg = os.path.join(os.path.dirname(CSRC), "_lib")
        try:
            os.makedirs(pkg, exist_ok=True)
            fd, probe = tempfile.mkstemp(prefix=".w", dir=pkg)
            os.close(fd)
            os.remove(probe)
            _lib_dir = pkg
        except OSError:
            d = os.path.join(tempfile.gettempdir(), f"zinfer_amd-lib-{os.getuid()}")
            os.makedirs(d, exist_ok=True)
            _lib_dir = d
        return _lib_dir


def _paths(module: str, directory: Optional[str] = None):
    d = directory or lib_dir()
    return os.path.join(d, module + ".so"), os.path.join(d, module + ".hash")


def is_current(module: str) -> bool:
    so, hp = _paths(module)
    if not (os.path.exists(so) and os.path.exists(hp)):
        # a library built elsewhere may sit in the package folder although it is read-only
        so, hp = _paths(module, os.path.join(os.path.dirname(CSRC), "_lib"))
        if not (os.path.exists(so) and os.path.exists(hp)):
            return False
    with open(hp) as f:
        return f.read().strip() == _source_hash(module)


def compile_module(module: str, verbose: bool = True) -> str:
    """Compiles one module (always) and returns the library's path."""
    if module not in MODULES and module not in HOST_MODULES:
        raise KernelUnavailable(f"unknown native module {module!r}")
    so, hp = _paths(module)
    tmp = f"{so}.{os.getpid()}.tmp"
    if module in HOST_MODULES:
        src = os.path.join(CSRC, "host", module + ".cpp")
        cmd = [_host_compiler()] + HOST_FLAGS + [src, "-o", tmp]
    else:
        src = os.path.join(CSRC, module + ".hip")
        cmd = [_hipcc()] + FLAGS + ["-I", CSRC, src, "-o", tmp]
    what = os.path.basename(src)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    if not env["HOME"] or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    t0 = time.time()
    if verbose:
        print(f"[zinfer_amd] compiling {what}" + ("" if module in HOST_MODULES else " for gfx950")
              + " ...", file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env,
                            text=True)
    out_lines: List[str] = []
    reader = threading.Thread(target=lambda: out_lines.extend(proc.stdout.readlines()))
    reader.start()
    while True:
        try:
            proc.wait(timeout=10)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(f"[zinfer_amd] still compiling {what} ({time.time() - t0:.0f} s)",
                      file=sys.stderr, flush=True)
    reader.join()
    if proc.returncode != 0:
        try:
            os.remove(tmp)
        except OSError:
            pass
        text = "".join(l for l in out_lines if "packed-fp32-ops" not in l)
        raise KernelUnavailable(f"{os.path.basename(cmd[0])} failed on {what}:\n{text[-4000:]}")
    os.replace(tmp, so)
    with open(hp, "w") as f:
        f.write(_source_hash(module))
    if verbose:
        print(f"[zinfer_amd] built {os.path.basename(so)} in {time.time() - t0:.1f} s",
              file=sys.stderr, flush=True)
    return so


def build_all(verbose: bool = True) -> None:
    """Compiles every module, whether or not a built library is there."""
    prepare(MODULES + HOST_MODULES, force=True, verbose=verbose)


def prepare(modules: Iterable[str], force: bool = False, verbose: bool = True) -> None:
    """Builds, side by side, those of ``modules`` that are missing or stale."""
    todo = [m for m in dict.fromkeys(modules) if force or not is_current(m)]
    errors: List[BaseException] = []

    def work(m):
        try:
            compile_module(m, verbose)
        except BaseException as e:  # noqa: BLE001 - reported below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(m,)) for m in todo]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]


def load(module: str) -> ctypes.CDLL:
    """The library of ``module``, built first if needed.  Fails loudly if it cannot be had."""
    lib = _libs.get(module)
    if lib is not None:
        return lib
    with _lock:
        lib = _libs.get(module)
        if lib is not None:
            return lib
        if not is_current(module):
            compile_module(module)
        so, _ = _paths(module)
        if not os.path.exists(so):
            so, _ = _paths(module, os.path.join(os.path.dirname(CSRC), "_lib"))
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise KernelUnavailable(f"cannot load {so}: {e}") from None
        _libs[module] = lib
        return lib
