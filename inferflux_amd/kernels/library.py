"""Builds and loads the native modules: the HIP kernels and the host-side C++ runtime pieces.

Each ``csrc/<name>.hip`` is compiled by hipcc for gfx950 (each ``csrc/<name>.cpp``, which is host code
only, by the C++ compiler) into one shared library
``<name>[-variant].<hash>.so`` and loaded through ctypes.  The hash covers the source, the
shared header, the flags and the variant's defines, so a library on disk always matches the
source beside it: a stale one is simply not found and the module is compiled again.  A module
is compiled when it is first used, which means a run compiles what its model needs and no
more.  Libraries are written next to the sources when that folder is writable (so they travel
with the tree) and to a per-user folder under the temporary directory otherwise.

There is no fallback: if hipcc is missing or a module does not compile, loading raises.
"""
from __future__ import annotations

import ctypes
import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, Iterable, Optional, Sequence, Tuple

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc")
CSRC = os.path.normpath(CSRC)
from .device import ARCH
# -packed-fp32-ops is switched off for device code: some packed float forms have given wrong
# results on this hardware.  The host pass of hipcc does not know the feature and says so.
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]

HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC"]
# INFERFLUX_HOST_SANITIZE=1 builds the host-only modules (the cache's bookkeeping) with the address and
# undefined-behaviour sanitizers, for test runs on the CPU (the process then needs libasan preloaded:
# LD_PRELOAD=$(g++ -print-file-name=libasan.so)).  Device code is never built with a sanitizer.
HOST_SANITIZE = os.environ.get("INFERFLUX_HOST_SANITIZE", "") == "1"
if HOST_SANITIZE:
    HOST_FLAGS = ["-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-std=c++17", "-shared", "-fPIC"]

Variant = Tuple[Tuple[str, int], ...]


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


def _variant_tag(variant: Variant) -> str:
    return "".join(f"-{k.lower()}{v}" for k, v in variant)


def _is_host_module(name: str) -> bool:
    return os.path.isfile(os.path.join(CSRC, f"{name}.cpp"))


def _cxx() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")):
        if cand and (os.path.isfile(cand) or shutil.which(cand)):
            return cand
    return _hipcc()          # hipcc compiles plain C++ too


def _sources(name: str) -> Tuple[str, ...]:
    """The files a module is built from: its source, the header of the same name (its public entry points) where it
    has one, and every header of this folder that the source includes."""
    import re
    if _is_host_module(name):
        return (f"{name}.cpp",)
    files = [f"{name}.hip"]
    with open(os.path.join(CSRC, files[0])) as f:
        included = re.findall(r'^\s*#\s*include\s+"([^"]+)"', f.read(), flags=re.M)
    for fn in ["common.h", f"{name}.h", *included]:
        if fn not in files and os.path.isfile(os.path.join(CSRC, fn)):
            files.append(fn)
    return tuple(files)


def _digest(name: str, variant: Variant) -> str:
    h = hashlib.sha256()
    host = _is_host_module(name)
    for fn in _sources(name):
        with open(os.path.join(CSRC, fn), "rb") as f:
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS if host else FLAGS).encode())
    h.update(repr(variant).encode())
    return h.hexdigest()[:12]


def _fallback_dir(create: bool = False) -> Optional[str]:
    """The per-user folder under the temporary directory that libraries go to when the source folder cannot be
    written.  Libraries are loaded from it, so it must be this user's own and closed to everyone else: a folder
    of that name that somebody else made, or that others may write, is refused.  Without ``create`` a folder
    that does not exist is None."""
    d = os.path.join(tempfile.gettempdir(), f"inferflux_amd-{os.getuid()}")
    if create:
        try:
            os.mkdir(d, 0o700)
        except FileExistsError:
            pass
    try:
        st = os.lstat(d)
    except FileNotFoundError:
        return None
    import stat
    if not stat.S_ISDIR(st.st_mode) or st.st_uid != os.getuid() or st.st_mode & 0o077:
        raise KernelBuildError(f"{d} is not a private folder of this user (owner {st.st_uid}, mode {stat.S_IMODE(st.st_mode):o}): "
                               f"refusing to build into or load libraries from it")
    return d


def _stem(name: str, variant: Variant) -> str:
    """A library's file name up to its hash (a sanitized host build has a name of its own, so that it and the
    ordinary build do not take each other for stale)."""
    san = "-hostsan" if HOST_SANITIZE and _is_host_module(name) else ""
    return f"{name}{san}{_variant_tag(variant)}"


def _lib_filename(name: str, variant: Variant) -> str:
    return f"{_stem(name, variant)}.{_digest(name, variant)}.so"


def find_library(name: str, variant: Variant = ()) -> Optional[str]:
    fn = _lib_filename(name, variant)
    p = os.path.join(CSRC, fn)
    if os.path.isfile(p):
        return p
    # Only a library that is not beside the sources is looked for in the per-user folder, so that a folder of that
    # name which fails the ownership check (anybody can make one) cannot stop a tree that has everything built.
    d = _fallback_dir()
    if d is not None:
        p = os.path.join(d, fn)
        if os.path.isfile(p):
            return p
    return None


def _progress(msg: str) -> None:
    print(f"[inferflux_amd] {msg}", file=sys.stderr, flush=True)


def compile_module(name: str, variant: Variant = (), force: bool = False) -> str:
    """Compile one module (unless an up-to-date library exists) and return the library's path."""
    if not force:
        hit = find_library(name, variant)
        if hit:
            return hit
    host = _is_host_module(name)
    src = os.path.join(CSRC, f"{name}.cpp" if host else f"{name}.hip")
    if not os.path.isfile(src):
        raise KernelBuildError(f"no kernel source {src}")
    out_dir = CSRC if os.access(CSRC, os.W_OK) else _fallback_dir(create=True)
    fn = _lib_filename(name, variant)
    out = os.path.join(out_dir, fn)
    lock_path = os.path.join(out_dir, f".{name}{_variant_tag(variant)}.lock")
    with open(lock_path, "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            if not force and os.path.isfile(out):
                return out
            tmp = f"{out}.{os.getpid()}.tmp"
            defines = [f"-D{k}={v}" for k, v in variant]
            cmd = [_cxx(), *HOST_FLAGS, *defines, src, "-o", tmp] if host else [_hipcc(), *FLAGS, *defines, src, "-o", tmp]
            label = f"{name}{_variant_tag(variant)}"
            _progress(f"compiling {label} for {'the host' if host else ARCH} ...")
            t0 = time.time()
            proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=out_dir)
            done = threading.Event()

            def tick():
                while not done.wait(20.0):
                    _progress(f"still compiling {label} ({time.time() - t0:.0f} s)")

            th = threading.Thread(target=tick, daemon=True)
            th.start()
            log, _ = proc.communicate()
            done.set()
            if proc.returncode != 0 or not os.path.isfile(tmp):
                if os.path.exists(tmp):
                    os.unlink(tmp)
                raise KernelBuildError(f"{os.path.basename(cmd[0])} failed for {label} (exit {proc.returncode}):\n{' '.join(cmd)}\n{log}")
            os.replace(tmp, out)
            # Drop libraries of the same module built from older sources.
            prefix = f"{_stem(name, variant)}."
            for old in os.listdir(out_dir):
                if old.startswith(prefix) and old.endswith(".so") and old != fn:
                    try:
                        os.unlink(os.path.join(out_dir, old))
                    except OSError:
                        pass
            _progress(f"compiled {label} in {time.time() - t0:.1f} s")
            return out
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)


class KernelModule:
    """A loaded library; functions are looked up by name, with their argument types set once."""

    def __init__(self, name: str, variant: Variant, path: str):
        self.name, self.variant, self.path = name, variant, path
        self.lib = ctypes.CDLL(path)
        self.lib.ifx_last_error.restype = ctypes.c_char_p
        self._fns: Dict[str, ctypes._CFuncPtr] = {}

    def fn(self, fname: str, argtypes: Sequence) -> "ctypes._CFuncPtr":
        f = self._fns.get(fname)
        if f is None:
            f = getattr(self.lib, fname)
            f.argtypes = list(argtypes)
            f.restype = ctypes.c_int
            self._fns[fname] = f
        return f

    def last_error(self) -> str:
        return (self.lib.ifx_last_error() or b"").decode(errors="replace")


_MODULES: Dict[Tuple[str, Variant], KernelModule] = {}
_LOCK = threading.Lock()


def load_module(name: str, variant: Variant = ()) -> KernelModule:
    key = (name, variant)
    m = _MODULES.get(key)
    if m is not None:
        return m
    with _LOCK:
        m = _MODULES.get(key)
        if m is None:
            m = KernelModule(name, variant, compile_module(name, variant))
            _MODULES[key] = m
    return m


def all_module_variants() -> Iterable[Tuple[str, Variant]]:
    """Every module and variant the package can ask for: what ``build_all`` compiles."""
    from . import ops
    return ops.module_variants()


def build_all(force: bool = True, jobs: int = 8) -> None:
    todo = list(all_module_variants())
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as ex:
        list(ex.map(lambda nv: compile_module(nv[0], nv[1], force=force), todo))
