"""The command line's host-side commands (no GPU)."""
import json
import os
import subprocess
import sys

import helpers

ROOT = os.path.normpath(os.path.join(os.path.dirname(__file__), ".."))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", "deliverance"), *args], capture_output=True, text=True, timeout=300)


def test_random_then_inspect(tmp_path):
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(helpers.CONFIG_B))
    out = tmp_path / "model"
    p = run("random", "--config", str(cfg), "--seed", "7", "--out", str(out))
    assert p.returncode == 0, p.stderr
    assert (out / "config.json").exists() and (out / "model.safetensors").exists()
    p = run("inspect", str(out))
    assert p.returncode == 0, p.stderr
    assert "architecture GPT2LMHeadModel: 3 layers, width 96, vocabulary 1000, 96 positions" in p.stdout
    assert "h.2.mlp.c_fc.weight" in p.stdout and "[96, 200]" in p.stdout


def test_help_names_the_reference_options():
    p = run("generate", "--help")
    for opt in ("--model", "--working-dtype", "--max-tokens", "--temperature", "--seed", "--warmup-cases", "--max-cases",
                "--kv-context-rows-per-page", "--model-config", "--profile-stages", "--kernels", "--suite-file", "--output", "--jsonl-output"):
        assert opt in p.stdout
    p = run("generate", "--model", "/nonexistent")
    assert p.returncode != 0


def test_bench_measures_one_gpu_only():
    """With more than one GPU asked for, bench.py says so in one line and exits with 2."""
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "--gpus 2" in p.stdout


def test_trace_run_without_a_gpu_says_so(tmp_path):
    """The replay program drives the GPU engine only: without a GPU it ends with a message, not a traceback."""
    import torch
    if torch.cuda.is_available():
        return
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "no GPU is visible" in p.stderr and "Traceback" not in p.stderr
