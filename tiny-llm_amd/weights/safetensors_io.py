"""Reader and writer for the safetensors container, without the library.

Format (as the reference's reader takes it, tiny_llm/weight_managers/safetensors/
src/lib.rs:31-136): 8 bytes little-endian header length, a JSON header
`{name: {dtype, shape, data_offsets:[begin,end]}, "__metadata__": {...}}`, then the
raw little-endian tensor bytes; offsets count from the end of the header.  The
file is memory-mapped and tensors are views into the map: nothing is read until a
tensor is copied to the device.
"""
from __future__ import annotations

import json
import os
import struct
from typing import Dict, Mapping, Tuple

import numpy as np
import torch

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(RuntimeError):
    pass


class SafetensorsFile:
    """A memory-mapped safetensors file: `names()`, `info(name)`, `get(name)`."""

    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
            with open(path, "rb") as f:
                head = f.read(8)
                if len(head) != 8:
                    raise SafetensorsError(f"{path}: shorter than a safetensors header")
                (n,) = struct.unpack("<Q", head)
                if n > size - 8:
                    raise SafetensorsError(f"{path}: header length {n} exceeds the file")
                header = json.loads(f.read(n).decode("utf-8"))
        except OSError as e:
            raise SafetensorsError(f"cannot open {path}: {e}") from e
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries: Dict[str, dict] = header
        self._base = 8 + n
        self._map = np.memmap(path, dtype=np.uint8, mode="c") if size > self._base else None
        for name, e in header.items():
            if e["dtype"] not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unsupported dtype {e['dtype']}")
            b, en = e["data_offsets"]
            count = int(np.prod(e["shape"], dtype=np.int64)) if e["shape"] else 1
            if en - b != count * _DTYPES[e["dtype"]][1] or self._base + en > size:
                raise SafetensorsError(f"{path}: tensor {name} has inconsistent offsets")

    def names(self):
        return list(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        e = self._entries[name]
        return _DTYPES[e["dtype"]][0], tuple(int(s) for s in e["shape"])

    def get(self, name: str) -> torch.Tensor:
        if name not in self._entries:
            raise SafetensorsError(f"tensor {name} cannot be found in {self.path}")
        e = self._entries[name]
        dtype, _ = _DTYPES[e["dtype"]]
        b, en = e["data_offsets"]
        shape = tuple(int(s) for s in e["shape"])
        if en == b:
            return torch.empty(shape, dtype=dtype)
        raw = torch.from_numpy(self._map[self._base + b: self._base + en])
        return raw.view(dtype).reshape(shape)


def open_model_files(folder: str):
    """The safetensors files of a model folder: `model.safetensors`, or the shards
    that `model.safetensors.index.json` names."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.exists(single):
        return [SafetensorsFile(single)]
    if os.path.exists(index):
        with open(index, "r", encoding="utf-8") as f:
            shards = sorted(set(json.load(f)["weight_map"].values()))
        return [SafetensorsFile(os.path.join(folder, s)) for s in shards]
    raise SafetensorsError(f"{folder} holds neither model.safetensors nor model.safetensors.index.json")


def save_file(tensors: Mapping[str, torch.Tensor], path: str, metadata: Mapping[str, str] = None) -> None:
    """Write tensors (CPU, any of the supported dtypes) in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    items = []
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name}: dtype {t.dtype} cannot be stored")
        t = t.detach().cpu().contiguous()
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        items.append(t)
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in items:
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
