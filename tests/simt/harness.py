"""The engine's HIP kernels run on the CPU, thread by thread, with every tensor between protected
pages: a test tool that finds accesses outside a tensor without a GPU.

The kernel sources are compiled for the host against a stand-in for the HIP runtime header
(``include/hip/hip_runtime.h``): GPU threads become fibers, barriers and cross-lane operations keep
their meaning, global memory is host memory.  The resulting library has the same ``da_*`` entry
points as the GPU library, so the engine's own Python (kernel faces, parts, model, step function,
cache manager) drives it unchanged; only the places that talk to the GPU runtime (stream, pinned
memory, the device check) are swapped while ``Sim.patched()`` is active.  An access outside a tensor
ends the process with a message that names kernel, workgroup, thread and tensor; tests therefore run
simulations in a child process (``run_child``).

Nothing here is part of the product: the engine never loads this library and has no CPU path.
"""
from __future__ import annotations

import contextlib
import ctypes
import glob
import hashlib
import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.normpath(os.path.join(HERE, "..", ".."))
CSRC = os.path.join(REPO, "deliverance_amd", "csrc")
CXX_CANDIDATES = ("/opt/rocm/llvm/bin/clang++", "clang++")


def _compiler():
    import shutil
    for c in CXX_CANDIDATES:
        p = c if os.path.isabs(c) else shutil.which(c)
        if p and os.path.exists(p):
            return p
    return None


def available() -> bool:
    return _compiler() is not None and sys.platform.startswith("linux") and os.uname().machine == "x86_64"


def build(verbose: bool = False) -> str:
    """Compile the kernels for the host (once per state of the sources); returns the library's path.
    $DELIVERANCE_SIMT_LIB names a library built by other means (with sanitizers, say)."""
    if os.environ.get("DELIVERANCE_SIMT_LIB"):
        return os.environ["DELIVERANCE_SIMT_LIB"]
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    deps = srcs + sorted(glob.glob(os.path.join(CSRC, "*.h"))) + [
        os.path.join(HERE, "include", "hip", "hip_runtime.h"), os.path.join(HERE, "simt_runtime.cpp")]
    h = hashlib.sha1()
    for p in deps:
        h.update(p.encode())
        with open(p, "rb") as f:
            h.update(f.read())
    out_dir = os.path.join(tempfile.gettempdir(), f"deliverance_amd_simt_{os.getuid()}_{h.hexdigest()[:16]}")
    lib = os.path.join(out_dir, "libdeliverance_simt.so")
    if os.path.exists(lib):
        return lib
    os.makedirs(out_dir, exist_ok=True)
    cxx = _compiler()
    # The kernels are compiled without optimisation: every load and store they spell out is executed
    # (an optimising host compiler drops a load whose value is replaced afterwards, and with it the
    # very access that is out of bounds on the GPU).  The scheduler and the matrix-core arithmetic
    # are compiled with optimisation.
    flags = ["-std=c++17", "-g", "-fPIC", "-Wno-unknown-attributes", "-Wno-unused-result",
             "-I", os.path.join(HERE, "include"), "-I", CSRC]

    def one(src):
        obj = os.path.join(out_dir, os.path.basename(src).rsplit(".", 1)[0] + ".o")
        lang = ["-x", "c++"] if src.endswith(".hip") else []
        opt = ["-O0"] if src.endswith(".hip") else ["-O2"]
        r = subprocess.run([cxx, *lang, *opt, *flags, "-c", src, "-o", obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"host build of {src} failed:\n{r.stderr}")
        if verbose:
            print(f"[simt] {os.path.basename(src)} done", file=sys.stderr, flush=True)
        return obj

    with ThreadPoolExecutor(max_workers=8) as pool:
        objs = list(pool.map(one, srcs + [os.path.join(HERE, "simt_runtime.cpp")]))
    tmp = lib + f".{os.getpid()}"
    r = subprocess.run([cxx, "-shared", "-fPIC", *objs, "-o", tmp], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"linking the host kernel library failed:\n{r.stderr}")
    os.replace(tmp, lib)
    return lib


class _NoStream:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


class Sim:
    """The host kernel library plus guarded tensors."""

    def __init__(self, at_start: bool = False, reverse: bool = False):
        self.lib = ctypes.CDLL(build())
        self.lib.sim_set_order(int(reverse))
        self.lib.da_last_error.restype = ctypes.c_char_p
        self.lib.sim_alloc.restype = ctypes.c_void_p
        self.lib.sim_alloc.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_char_p]
        self.lib.sim_free.argtypes = [ctypes.c_void_p]
        self.lib.sim_launch_count.restype = ctypes.c_long
        self.at_start = at_start

    # ---- memory ---------------------------------------------------------------------------------
    def empty(self, shape, dtype, name="tensor") -> torch.Tensor:
        """A tensor whose memory lies between two protected pages (filled with 0x7f bytes)."""
        shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list, torch.Size)) else (shape,)))
        numel = 1
        for s in shape:
            numel *= s
        nbytes = numel * torch.empty((), dtype=dtype).element_size()
        ptr = self.lib.sim_alloc(nbytes, int(self.at_start), name.encode())
        if not ptr:
            raise MemoryError(f"sim_alloc of {nbytes} bytes failed")
        if numel == 0:
            return torch.empty(shape, dtype=dtype)
        buf = (ctypes.c_char * nbytes).from_address(ptr)
        t = torch.frombuffer(buf, dtype=dtype, count=numel).view(shape)
        t._sim_ptr = ptr
        return t

    def like(self, t: torch.Tensor, name="tensor") -> torch.Tensor:
        out = self.empty(t.shape, t.dtype, name)
        out.copy_(t)
        return out

    def free(self, t: torch.Tensor) -> None:
        ptr = getattr(t, "_sim_ptr", None)
        if ptr:
            self.lib.sim_free(ptr)
            t._sim_ptr = None

    def rehome(self, obj, name="model", _memo=None):
        """Every tensor reachable from ``obj`` (attributes, lists, dicts) moves into guarded memory;
        a tensor that is reached twice stays one tensor."""
        memo = {} if _memo is None else _memo
        if isinstance(obj, torch.Tensor):
            key = (obj.data_ptr(), tuple(obj.shape), tuple(obj.stride()), obj.dtype)
            if key not in memo:
                memo[key] = self.like(obj.contiguous(), name) if obj.is_contiguous() else obj
            return memo[key]
        if isinstance(obj, list):
            for i, v in enumerate(obj):
                obj[i] = self.rehome(v, f"{name}[{i}]", memo)
            return obj
        if isinstance(obj, dict):
            for k, v in list(obj.items()):
                obj[k] = self.rehome(v, f"{name}[{k!r}]", memo)
            return obj
        mod = type(obj).__module__ or ""
        if hasattr(obj, "__dict__") and not isinstance(obj, type) and not mod.startswith(("torch", "numpy", "builtins")):
            if id(obj) in memo:
                return obj
            memo[id(obj)] = obj
            for k, v in list(vars(obj).items()):
                if isinstance(v, (torch.Tensor, list, dict)) or hasattr(v, "__dict__"):
                    new = self.rehome(v, f"{name}.{k}", memo)
                    if new is not v:
                        setattr(obj, k, new)
        return obj

    # ---- the engine's kernel faces on this library -----------------------------------------------
    @contextlib.contextmanager
    def patched(self, auto_guard: bool = False):
        """While active, the engine's kernel faces (``deliverance_amd.kernels.ops``) call this library.
        With ``auto_guard`` every tensor operand of every kernel call is copied into guarded memory of
        exactly the operand's extent for the call and copied back afterwards, so ordinary CPU tensors
        can be passed and still no access outside an operand goes unnoticed."""
        from deliverance_amd.kernels import build as kbuild, ops
        saved = (kbuild._lib, ops._LIB, ops._dev, ops._stream, ops.pinned_stream, ops._ptr, ops._check)
        kbuild._lib, ops._LIB = self.lib, None
        ops._dev = lambda *ts: None
        ops._stream = lambda: None
        ops.pinned_stream = _NoStream
        if auto_guard:
            guard = AutoGuard(self)
            check = ops._check
            ops._ptr = guard.ptr

            def checked(rc):
                guard.finish()
                check(rc)
            ops._check = checked
        try:
            yield self
        finally:
            kbuild._lib, ops._LIB, ops._dev, ops._stream, ops.pinned_stream, ops._ptr, ops._check = saved


class AutoGuard:
    """Guarded stand-ins for the tensor operands of one kernel call."""

    def __init__(self, sim: Sim):
        self.sim = sim
        self.live = []          # (first byte, bytes, flat view of the operand's memory, guarded copy)

    def ptr(self, t):
        if t is None:
            return None
        if t.numel() == 0:
            return t.data_ptr()
        el = t.element_size()
        extent = 1 + sum((n - 1) * st for n, st in zip(t.shape, t.stride()))
        lo, nbytes = t.data_ptr(), extent * el
        for lo0, nb0, _, g0 in self.live:
            if lo0 == lo and nb0 == nbytes:
                return g0._guard_ptr
            if lo < lo0 + nb0 and lo0 < lo + nbytes:
                raise RuntimeError("two operands of one kernel call overlap without being the same view; "
                                   "the guarded copies would not stay coherent")
        who = sys._getframe(1).f_code.co_name
        mis = lo % 16                                   # the stand-in is aligned as the operand is
        g = self.sim.empty((nbytes + mis,), torch.uint8, f"{who}: operand {list(t.shape)} {t.dtype}")
        flat = torch.as_strided(t, (extent,), (1,)).view(torch.uint8)
        g[mis:].copy_(flat)
        g._guard_ptr = g._sim_ptr + mis
        self.live.append((lo, nbytes, flat, g))
        return g._guard_ptr

    def finish(self):
        for lo, nbytes, flat, g in self.live:
            now = g[g.numel() - nbytes:]
            if not torch.equal(flat, now):          # (inputs may lie in read-only memory: a mapped checkpoint)
                flat.copy_(now)
            self.sim.free(g)
        self.live = []


def make_arena(sim: Sim):
    from deliverance_amd.parts.base import Arena

    class SimArena(Arena):
        """Scratch buffers of exactly the size asked for, each between protected pages."""

        def __init__(self):
            super().__init__("cpu")

        def get(self, name, rows, cols, dtype):
            key = (name, cols, dtype)
            t = self._bufs.get(key)
            if t is None or t.shape[0] != rows:
                if t is not None:
                    sim.free(t)
                t = sim.empty((rows, cols), dtype, f"arena:{name}")
                self._bufs[key] = t
            return t

    return SimArena()


def make_runner(model, cache, sim: Sim = None):
    """The engine's step function with the host-to-device copy replaced by a plain copy (into a
    guarded tensor of exactly the step's integers when ``sim`` is given)."""
    from deliverance_amd.engine.step import StepRunner

    class CpuStepRunner(StepRunner):
        def __init__(self):
            super().__init__(model, cache, use_graphs=False)
            if sim is not None:
                self.arena = make_arena(sim)
            self._np = None
            self._dev_t = None

        def _staging_for(self, n):
            import numpy as np
            self._np = np.empty(n, dtype=np.int32)
            return self._np

        def _upload(self, n):
            if sim is None:
                self._dev_t = torch.from_numpy(self._np[:n].copy())
                return self._dev_t
            if self._dev_t is not None:
                sim.free(self._dev_t)
            self._dev_t = sim.empty((n,), torch.int32, "step integers")
            self._dev_t.copy_(torch.from_numpy(self._np[:n]))
            return self._dev_t

    r = CpuStepRunner()
    if sim is not None:
        r.sampled = sim.like(r.sampled, "sampled tokens")
    return r


def SimTraceSession(sim, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16,
                    poison_freed: bool = False, **options):
    """What ``deliverance_amd.trace.TraceSession`` is on the GPU, on the simulated kernels: the same
    class with the step runner's host-to-device copy replaced.  With ``sim`` the model's tensors,
    the cache and the scratch buffers live in guarded memory (use with ``Sim.patched()``); without,
    they are ordinary CPU tensors (use with ``patched(auto_guard=True)``)."""
    from deliverance_amd.trace import TraceSession

    class _Session(TraceSession):
        def _make_runner(self, use_graphs, kernels):
            if sim is not None:
                sim.rehome(self.model, "model")
                for g, t in enumerate(self.cache._group_tensors):
                    new = sim.like(t, f"cache group {g}")
                    self.cache._group_tensors[g] = new
                    for i, slot in enumerate(self.cache.groups[g].slots):
                        self.cache.kv[slot] = new[i]
                for slot, t in list(self.cache.state.items()):
                    self.cache.state[slot] = sim.like(t, f"state {slot}")
            r = make_runner(self.model, self.cache, sim)
            r.kernels = kernels
            return r

        def _drain(self):
            pass

        def run_step(self, rec):
            out = super().run_step(rec)        # on the CPU this is a view of the step's logits buffer
            return None if out is None else out.copy()

    s = _Session(model_dir, dtype, max_tokens, page_size, device="cpu", poison_freed=poison_freed, **options)
    s.sim = sim
    return s


def run_child(args, timeout: int = 900, env_extra=None):
    """Run a fresh Python with ``args`` (tests/ and the repository on its path); returns the
    CompletedProcess.  A fault inside a simulated kernel ends that process with status 97 and a
    message on stderr that names the kernel, the workgroup, the thread and the tensor."""
    env = dict(os.environ)
    env["PYTHONPATH"] = os.pathsep.join([REPO, os.path.join(REPO, "tests"), env.get("PYTHONPATH", "")])
    env.update(env_extra or {})
    return subprocess.run([sys.executable, *args], capture_output=True, text=True, timeout=timeout, env=env, cwd=REPO)
