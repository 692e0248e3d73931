"""Reading and writing safetensors files, by tensor name.

File layout (safetensors/src/main/java/io/teknek/deliverance/safetensors/
DefaultWeightLoader.java:198-240): an unsigned 64-bit little-endian header length, a JSON
header ``{name: {dtype, shape, data_offsets}, "__metadata__": {...}}`` and the raw bytes,
with offsets counted from the end of the header.  A model folder holds either a
``model.safetensors.index.json`` with a ``weight_map`` or a single ``model.safetensors``
(DefaultWeightLoader.java:108-117).  Each file is mapped once; tensors are views of the
mapping until they are copied to the GPU.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Optional, Tuple

import numpy as np
import torch

MAX_HEADER_BYTES = 1 << 30      # DefaultWeightLoader.java:202-209 rejects larger headers

_ITEMSIZE = {"F64": 8, "F32": 4, "F16": 2, "BF16": 2, "I64": 8, "I32": 4, "I16": 2, "I8": 1,
             "U8": 1, "BOOL": 1}
_TORCH_DTYPE = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16,
                "BF16": torch.bfloat16, "I64": torch.int64, "I32": torch.int32,
                "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool}
_NAME_OF = {v: k for k, v in _TORCH_DTYPE.items()}


class WeightFileError(ValueError):
    """A safetensors file or model folder that cannot be read."""


class SafetensorsFile:
    """One mapped ``.safetensors`` file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise WeightFileError(f"{path}: too short to be a safetensors file ({size} bytes)")
        self._fh = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen <= 0 or hlen > MAX_HEADER_BYTES or 8 + hlen > size:
            raise WeightFileError(f"{path}: header length {hlen} is not plausible for a file of {size} bytes")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not valid JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + hlen
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        data_len = size - self._data_start
        for name, info in header.items():
            try:
                dtype, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                begin, end = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightFileError(f"{path}: malformed header entry for tensor {name!r}") from None
            if dtype not in _ITEMSIZE:
                raise WeightFileError(f"{path}: tensor {name!r} has unsupported dtype {dtype}")
            want = int(np.prod(shape, dtype=np.int64)) * _ITEMSIZE[dtype] if shape else _ITEMSIZE[dtype]
            if begin < 0 or end < begin or end > data_len or end - begin != want:
                raise WeightFileError(
                    f"{path}: tensor {name!r} ({dtype} {list(shape)}) needs {want} bytes but its "
                    f"data_offsets are [{begin}, {end}) in a data section of {data_len} bytes")
            self.entries[name] = (dtype, shape, begin, end)

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def info(self, name: str) -> Tuple[str, Tuple[int, ...]]:
        dtype, shape, _, _ = self.entries[name]
        return dtype, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor in the stored dtype that views the mapping (do not write to it)."""
        dtype, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=_TORCH_DTYPE[dtype])
        buf = memoryview(self._mm)[self._data_start + begin:self._data_start + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")     # the mapping is read-only; tensors are only read
            t = torch.frombuffer(buf, dtype=_TORCH_DTYPE[dtype])
        return t.reshape(shape)


class WeightSource:
    """All tensors of a model folder, whichever file holds them."""

    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.exists(index):
            with open(index) as f:
                weight_map = json.load(f).get("weight_map")
            if not isinstance(weight_map, dict):
                raise WeightFileError(f"{index}: no weight_map")
            for name, fname in weight_map.items():
                if fname not in self._files:
                    self._files[fname] = SafetensorsFile(os.path.join(folder, fname))
                if name not in self._files[fname].entries:
                    raise WeightFileError(f"{index}: tensor {name!r} is not in {fname}")
                self._where[name] = fname
        elif os.path.exists(single):
            self._files["model.safetensors"] = SafetensorsFile(single)
            for name in self._files["model.safetensors"].names():
                self._where[name] = "model.safetensors"
        else:
            raise WeightFileError(
                f"weights not found: {folder} has neither model.safetensors.index.json nor model.safetensors")

    def names(self):
        return list(self._where.keys())

    def info(self, name: str):
        return self._files[self._where[name]].info(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].tensor(name)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor],
                      metadata: Optional[Dict[str, str]] = None) -> None:
    """Write CPU tensors in their own dtypes (the reference's writer:
    safetensors/.../SafeTensorWriter.java:22-80).  Data is aligned to 8 bytes."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors.keys())
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAME_OF:
            raise WeightFileError(f"cannot write tensor {name!r} of dtype {t.dtype}")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAME_OF[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + n]}
        offset += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                        t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
