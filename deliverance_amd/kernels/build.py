"""Compiling the HIP sources for gfx950 into one shared library, and loading it.

The library is built in-tree (``deliverance_amd/csrc/_build/libdeliverance_hip.so``) with
plain ``hipcc``; when that folder cannot be written, a folder under the system's temporary
directory is used.  ``load()`` builds only when no library is there (or when it is older
than a source); ``build(force=True)`` always compiles.  There is no fallback: without the
library and without ``hipcc`` the engine refuses to run.
"""
from __future__ import annotations

import ctypes
import fcntl
import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))
LIB_NAME = "libdeliverance_hip.so"
ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-result", "-Wno-unknown-warning-option"]
# Per source: kernels that read their matrix-core results back at once (softmax between two
# products) keep them in ordinary vector registers; the default puts them into accumulation
# registers and moves every value out and in again.
EXTRA_FLAGS = {"attn_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}

_lib = None


class KernelLibraryError(RuntimeError):
    pass


def _sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _headers():
    return sorted(glob.glob(os.path.join(CSRC, "*.h")))


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _build_dirs():
    in_tree = os.path.join(CSRC, "_build")
    tag = hashlib.sha1(CSRC.encode()).hexdigest()[:12]
    fallback = os.path.join(tempfile.gettempdir(), f"deliverance_amd_build_{os.getuid()}_{tag}")
    return in_tree, fallback


def _find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


def _stale(lib_path: str) -> bool:
    if not os.path.exists(lib_path):
        return True
    t = os.path.getmtime(lib_path)
    return any(os.path.getmtime(s) > t for s in _sources() + _headers())


def library_path():
    """The newest usable library, or None."""
    for d in _build_dirs():
        p = os.path.join(d, LIB_NAME)
        if os.path.exists(p) and not _stale(p):
            return p
    return None


def build(force: bool = False, verbose: bool = True) -> str:
    """Compile every ``.hip`` source and link the library; returns its path."""
    if not force:
        p = library_path()
        if p:
            return p
    hipcc = _find_hipcc()
    if hipcc is None:
        raise KernelLibraryError(
            "the HIP kernels are not built and hipcc was not found (looked at $HIPCC, PATH and "
            "/opt/rocm/bin/hipcc); this engine has no other compute path")
    in_tree, fallback = _build_dirs()
    out_dir = in_tree if _writable(in_tree) else fallback
    if not _writable(out_dir):
        raise KernelLibraryError(f"cannot write the kernel library to {in_tree} or {fallback}")
    srcs = _sources()
    if not srcs:
        raise KernelLibraryError(f"no HIP sources under {CSRC}")
    # one build at a time per folder: processes that start together in a fresh checkout would
    # otherwise write the same object files; whoever waited finds the library built
    with open(os.path.join(out_dir, ".build.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if not force:
            p = library_path()
            if p:
                return p
        return _build_locked(hipcc, out_dir, srcs, verbose)


def _build_locked(hipcc: str, out_dir: str, srcs, verbose: bool) -> str:
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)       # hipcc wants somewhere to keep its temporary files
    env.setdefault("TMPDIR", tempfile.gettempdir())
    t0 = time.time()

    def say(msg):
        if verbose:
            print(f"[deliverance_amd build] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(src):
        obj = os.path.join(out_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(os.path.basename(src), []), "-I", CSRC, "-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        say(f"  {os.path.basename(src)} done ({time.time() - t0:.0f}s)")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib_tmp = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", lib_tmp],
                       capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise KernelLibraryError(f"linking the kernel library failed:\n{r.stdout}\n{r.stderr}")
    lib_path = os.path.join(out_dir, LIB_NAME)
    os.replace(lib_tmp, lib_path)
    say(f"built {lib_path} in {time.time() - t0:.0f}s")
    return lib_path


def load() -> ctypes.CDLL:
    """The loaded library (built first when missing).  torch is imported before, so that the
    library binds to the HIP runtime that torch has already loaded."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (loads libamdhip64 first)
    path = library_path() or build(force=False)
    try:
        _lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from None
    _lib.da_last_error.restype = ctypes.c_char_p
    return _lib
