"""Binding checkpoint tensors to a model by name, with one error for everything wrong.

An architecture declares the tensors it needs as :class:`TensorDecl` records (name, shape
and, for the random-weights mode, how to draw it).  :func:`load_declared` reads them from
a model folder and raises a single :class:`WeightError` that lists every missing tensor,
every unexpected one and every wrong shape.  The reference resolves names one at a time
and fails at the first absent one (safetensors/src/main/java/io/teknek/deliverance/
safetensors/DefaultWeightLoader.java:364-370) and does not check shapes.

Stored dtypes are kept: bfloat16 stays bfloat16, 32-bit floats stay 32-bit, integer
tables become int32; float16 is widened to float32 (lossless), as the reference does when
float32 dominates (safetensors/.../Weights.java:96-146).
"""
from __future__ import annotations

import fnmatch
import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Sequence, Tuple

import torch

from .safetensors_io import WeightSource, write_safetensors


class WeightError(ValueError):
    """The checkpoint does not fit the model; the message lists all faults."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"checkpoint in {folder} does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: expected {list(e)}, found {list(f)}" for n, e, f in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  unusable dtypes ({len(self.wrong_dtype)}): " + "; ".join(
                f"{n}: {d}" for n, d in self.wrong_dtype))
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class TensorDecl:
    name: str
    shape: Tuple[int, ...]
    init: str = "normal"         # "normal" | "ones_plus_normal" | "zeros" | "ones"
    std: float = 0.02
    optional: bool = False       # absent is fine (e.g. an untied head falling back to the table)


_KEPT = {torch.bfloat16: torch.bfloat16, torch.float32: torch.float32,
         torch.float16: torch.float32, torch.float64: torch.float32,
         torch.int32: torch.int32, torch.int64: torch.int32, torch.int16: torch.int32,
         torch.int8: torch.int32, torch.uint8: torch.int32}


def _strip(name: str, prefixes: Sequence[str]) -> str:
    for p in prefixes:
        if name.startswith(p):
            return name[len(p):]
    return name


def load_declared(folder: str, decls: Iterable[TensorDecl], ignore: Sequence[str] = (),
                  strip_prefixes: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """Read exactly the declared tensors.  ``ignore`` holds glob patterns of tensor names a
    checkpoint may carry without the model using them (buffers such as ``h.*.attn.bias``)."""
    source = WeightSource(folder)
    by_name = {}
    for stored in source.names():
        by_name[_strip(stored, strip_prefixes)] = stored
    decls = list(decls)
    declared = {d.name for d in decls}
    missing: List[str] = []
    wrong_shape = []
    wrong_dtype = []
    out: Dict[str, torch.Tensor] = {}
    for d in decls:
        stored = by_name.get(d.name)
        if stored is None:
            if not d.optional:
                missing.append(d.name)
            continue
        dtype, shape = source.info(stored)
        if tuple(shape) != tuple(d.shape):
            wrong_shape.append((d.name, d.shape, shape))
            continue
        t = source.tensor(stored)
        if t.dtype not in _KEPT:
            wrong_dtype.append((d.name, dtype))
            continue
        out[d.name] = t if _KEPT[t.dtype] == t.dtype else t.to(_KEPT[t.dtype])
    unexpected = sorted(n for n in by_name
                        if n not in declared and not any(fnmatch.fnmatchcase(n, p) for p in ignore))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)
    return out


def _generator_for(seed: int, name: str) -> torch.Generator:
    """One generator per (seed, tensor name), so a tensor's values do not depend on the
    order in which tensors are drawn (FNV-1a of the name, mixed with the seed)."""
    h = 0xcbf29ce484222325
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    g = torch.Generator(device="cpu")
    g.manual_seed((h ^ (seed * 0x9E3779B97F4A7C15)) & 0x7FFFFFFFFFFFFFFF)
    return g


def draw_tensor(decl: TensorDecl, seed: int, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    g = _generator_for(seed, decl.name)
    if decl.init == "zeros":
        t = torch.zeros(decl.shape, dtype=torch.float32)
    elif decl.init == "ones":
        t = torch.ones(decl.shape, dtype=torch.float32)
    else:
        t = torch.randn(decl.shape, generator=g, dtype=torch.float32) * decl.std
        if decl.init == "ones_plus_normal":
            t = t + 1.0
        elif decl.init != "normal":
            raise ValueError(f"unknown init {decl.init!r} for tensor {decl.name}")
    return t.to(dtype)


def write_random_model(folder: str, config_dict: dict, decls: Iterable[TensorDecl], seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """The random-weights mode: write ``config.json`` and ``model.safetensors`` so that the
    random model goes through the same loader as a real checkpoint (the reference's tests
    build tiny checkpoints the same way: core/src/test/java/io/teknek/deliverance/model/
    qwen3/Qwen3HfTextModelPortedTest.java:229-272)."""
    os.makedirs(folder, exist_ok=True)
    tensors = {d.name: draw_tensor(d, seed, dtype) for d in decls if not d.optional}
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config_dict, f, indent=1)
    return folder
