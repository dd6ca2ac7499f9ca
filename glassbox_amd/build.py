"""Compiles the native libraries in-tree and loads them through ctypes.

Two kinds of library live under ``csrc/``: the host runtime (``host/*.cpp``, plain
C++ built with g++: cache manager, scheduler, sampler) and the device kernels
(``hip/*.hip``, built with hipcc for gfx950, one shared object per source file so
that a run compiles only the groups it uses).  Built objects go to
``glassbox_amd/_lib`` with a stamp of the hash of their sources and flags; a
stale or missing object is rebuilt on first use, with a progress line every few
seconds.  If the package folder cannot be written, a per-user folder under the
temporary directory is used instead.
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
from typing import Dict, List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
_ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={_ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
    # the compiler may not form packed fp32 instructions (v_pk_*_f32) from float code: some of their forms have
    # given wrong results on gfx950 hardware, silently
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]

#: name -> (compiler kind, sources relative to csrc, extra dependencies hashed with them)
LIBRARIES: Dict[str, tuple] = {
    "host": ("host", ["host/cache_manager.cpp", "host/scheduler.cpp", "host/c_api.cpp", "host/launch_tape.cpp"],
             ["host/cache_manager.h", "host/scheduler.h", "host/sampler.h"]),
    "elementwise": ("hip", ["hip/elementwise.hip"], ["hip/common.h"]),
    "gemm_f32": ("hip", ["hip/gemm_f32.hip"], ["hip/common.h"]),
    "gemm_bf16": ("hip", ["hip/gemm_bf16.hip"], ["hip/common.h"]),
    "attention_plain": ("hip", ["hip/attention_plain.hip"], ["hip/common.h"]),
    "attention_bf16": ("hip", ["hip/attention_bf16.hip"], ["hip/common.h", "hip/attention_bf16.h"]),
    "sampling": ("hip", ["hip/sampling.hip"], ["hip/common.h"]),
}

_lock = threading.Lock()
_loaded: Dict[str, ctypes.CDLL] = {}


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[glassbox_amd] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the device kernels cannot be built")


_dir_lock = threading.Lock()
_dir: Optional[str] = None


def _lib_dir() -> str:
    """Where built objects live: decided once per process (in-tree if writable)."""
    global _dir
    with _dir_lock:
        if _dir is None:
            d = os.path.join(_HERE, "_lib")
            try:
                os.makedirs(d, exist_ok=True)
                probe = os.path.join(d, f".w{os.getpid()}.{threading.get_ident()}")
                with open(probe, "w"):
                    pass
                os.remove(probe)
            except OSError:
                d = os.path.join(tempfile.gettempdir(), f"glassbox_amd-{os.getuid()}", "_lib")
                os.makedirs(d, exist_ok=True)
            _dir = d
        return _dir


def _digest(name: str) -> str:
    kind, sources, deps = LIBRARIES[name]
    h = hashlib.sha256()
    h.update(" ".join(HIP_FLAGS if kind == "hip" else HOST_FLAGS).encode())
    for rel in list(sources) + list(deps):
        with open(os.path.join(_CSRC, rel), "rb") as fh:
            h.update(rel.encode())
            h.update(fh.read())
    return h.hexdigest()[:16]


def lib_path(name: str) -> str:
    return os.path.join(_lib_dir(), f"libgb_{name}.so")


def _current_at(path: str, name: str) -> bool:
    stamp = path + ".stamp"
    if not (os.path.exists(path) and os.path.exists(stamp)):
        return False
    try:
        with open(stamp) as fh:
            return fh.read().strip() == _digest(name)
    except OSError:
        return False


def find_current(name: str) -> Optional[str]:
    """Path of a built library that matches its sources: the package folder first (also when it
    cannot be written, as in a read-only checkout that ships built objects), then the fallback."""
    for d in (os.path.join(_HERE, "_lib"), _lib_dir()):
        path = os.path.join(d, f"libgb_{name}.so")
        if _current_at(path, name):
            return path
    return None


def is_current(name: str) -> bool:
    return find_current(name) is not None


def compile_library(name: str, quiet: bool = False) -> str:
    """Compile one library now, whatever is there.  Returns the path of the shared object."""
    kind, sources, _ = LIBRARIES[name]
    out = lib_path(name)
    tmp = f"{out}.{os.getpid()}.{threading.get_ident()}.tmp"
    srcs = [os.path.join(_CSRC, s) for s in sources]
    if kind == "hip":
        cmd = [_hipcc()] + HIP_FLAGS + srcs + ["-o", tmp]
    else:
        cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++") or _hipcc()
        cmd = [cxx] + HOST_FLAGS + srcs + ["-o", tmp]
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env.get("HOME", "/"), os.W_OK):
        env["HOME"] = tempfile.gettempdir()  # the compiler driver wants a writable home for its caches
    t0 = time.time()
    if not quiet:
        _say(f"compiling {name} ({', '.join(sources)}) ...")
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=_CSRC)
    done = threading.Event()

    def ticker():
        while not done.wait(10.0):
            _say(f"  still compiling {name}: {time.time() - t0:.0f} s")

    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    log = proc.communicate()[0].decode(errors="replace")
    done.set()
    if proc.returncode != 0:
        try:
            os.remove(tmp)
        except OSError:
            pass
        lines = [l for l in log.splitlines() if "packed-fp32-ops" not in l]
        raise BuildError(f"building {name} failed ({' '.join(cmd)}):\n" + "\n".join(lines[-60:]))
    os.replace(tmp, out)
    with open(out + ".stamp", "w") as fh:
        fh.write(_digest(name))
    if not quiet:
        _say(f"built {name} in {time.time() - t0:.1f} s")
    return out


def build_all(force: bool = True, names: Optional[List[str]] = None, jobs: int = 8) -> None:
    """Compile every library (or ``names``).  With ``force`` also those that are current."""
    todo = [n for n in (names or list(LIBRARIES)) if force or not is_current(n)]
    if todo:
        with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as pool:
            list(pool.map(compile_library, todo))
    if names is None:
        _stamp_version()   # also when nothing had to be compiled: the commit names the Python beside the libraries too


def _git_commit() -> Optional[str]:
    """The checkout's commit (short, with ``+`` if tracked files differ from it), or None where there is no git."""
    root = os.path.dirname(_HERE)
    try:
        r = subprocess.run(["git", "-C", root, "rev-parse", "--short", "HEAD"], capture_output=True, text=True, timeout=10)
        if r.returncode != 0 or not r.stdout.strip():
            return None
        d = subprocess.run(["git", "-C", root, "status", "--porcelain", "--untracked-files=no"], capture_output=True,
                           text=True, timeout=10)
        return r.stdout.strip() + ("+" if d.returncode == 0 and d.stdout.strip() else "")
    except (OSError, subprocess.SubprocessError):
        return None


def _stamp_version() -> None:
    """Notes the commit beside the built libraries, which travel to machines where the sources are no checkout."""
    commit = _git_commit()
    if commit:
        try:
            with open(os.path.join(_lib_dir(), "commit.stamp"), "w") as fh:
                fh.write(commit)
        except OSError:
            pass


def source_version() -> str:
    """What a measurement names as the code it ran: the commit of the checkout; where there is none, ``$GLASSBOX_COMMIT``
    or the commit noted when the libraries were built (``built@...``: the tree may have moved on since); failing
    that, a hash of the native sources (``src-...``)."""
    commit = _git_commit() or os.environ.get("GLASSBOX_COMMIT")
    if commit:
        return commit
    for d in (os.path.join(_HERE, "_lib"), _lib_dir()):
        try:
            with open(os.path.join(d, "commit.stamp")) as fh:
                noted = fh.read().strip()
            if noted:
                return "built@" + noted
        except OSError:
            pass
    h = hashlib.sha256()
    for name in sorted(LIBRARIES):
        h.update(_digest(name).encode())
    return "src-" + h.hexdigest()[:12]


def load(name: str) -> ctypes.CDLL:
    """The library ``name``, compiled first if it is missing or older than its sources."""
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        if name not in LIBRARIES:
            raise BuildError(f"no native library called {name!r}")
        path = find_current(name) or compile_library(name)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"cannot load {path}: {e}") from None
        _loaded[name] = lib
        return lib


def ensure(names: List[str]) -> None:
    """Compile, in parallel, those of ``names`` that are missing or stale (no loading)."""
    build_all(force=False, names=names)
