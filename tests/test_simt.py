"""The engine's HIP kernels on the CPU: the kernel sources compiled for the host and run thread by
thread (tests/simt), every operand of every kernel call between protected pages.  An access outside
an operand ends the child process with a message that names the kernel, the workgroup, the thread
and the operand.  The children run the GPU test files themselves (the same cases, with CPU tensors),
so what the GPU tests cover for results, these runs cover for addresses.

Set DELIVERANCE_SIMT_FULL=1 to run everything the simulated kernels can run (a quarter of an hour
on 8 cores); the default is a selection that takes about a minute.
"""
import os
import subprocess
import sys

import pytest

from simt import harness

pytestmark = pytest.mark.skipif(not harness.available(), reason="needs clang++ on x86-64 Linux")
FULL = os.environ.get("DELIVERANCE_SIMT_FULL") == "1"

# name -> pytest arguments of the child.  The default selection: the cases marked for it in the GPU test files
# (simt_quick, or simt_a and simt_b where two parameter lists cross).
QUICK = "gpu and (simt_quick or (simt_a and simt_b))"
RUNS = {
    # the regression for the block-tile product's loads past K with K below one slab (K = 24, 65 rows and more)
    "tile_product_small_k": ["tests/test_kernels_gpu.py", "-k", "matrix_cores and 50-24", "-n", "2"],
    "kernels": ["tests/test_kernels_gpu.py", "-n", "4"] + ([] if FULL else ["-m", QUICK]),
    "parts": ["tests/test_parts_gpu.py"],
    "replay": ["tests/test_replay_gpu.py", "-n", "4"] if FULL else
              ["tests/test_replay_gpu.py", "-n", "2", "-k", "(mixed and (A or B) and not 32) or want_subset or errors_leave or first_tokens"],
    # inner sizes of 32 in an engine step: qkv and fc of seed 11 (and, in the full run, proj of seed 5)
    "random_configurations": ["tests/test_random_configs_gpu.py", "-n", "4"] if FULL else
                             ["tests/test_random_configs_gpu.py", "-k", "11"],
}
if FULL:
    RUNS["toy_parts"] = ["tests/test_toy_parts_gpu.py", "tests/test_toy_parts2_gpu.py", "-n", "4"]
    RUNS["engine_paths"] = ["tests/test_engine_paths_gpu.py", "-n", "4"]


@pytest.fixture(scope="module")
def children():
    """All children start together (they are independent processes) and are waited for one by one."""
    harness.build()
    env = dict(os.environ)
    env["DELIVERANCE_SIMT"] = "1"
    procs = {}
    for name, args in RUNS.items():
        marks = [] if "-m" in args else ["-m", "gpu"]
        procs[name] = subprocess.Popen([sys.executable, "-m", "pytest", "-x", "-q", *marks, "-p", "no:cacheprovider",
                                        "-s", *args], cwd=harness.REPO, env=env, stdout=subprocess.PIPE,
                                       stderr=subprocess.STDOUT, text=True)
    yield procs
    for p in procs.values():
        if p.poll() is None:
            p.kill()


@pytest.mark.parametrize("name", sorted(RUNS))
def test_simulated_kernels_stay_inside_their_operands(children, name):
    p = children[name]
    out, _ = p.communicate(timeout=3000 if FULL else 900)
    assert p.returncode == 0, f"simulated run '{name}' ended with status {p.returncode}:\n{out[-3000:]}"
    assert " passed" in out and " failed" not in out, out[-2000:]
