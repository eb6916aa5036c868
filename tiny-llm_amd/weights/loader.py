"""Weights by tensor name, from safetensors or from a seed.

The reference copies each graph tensor from the file under its own name, checks
its shape, accepts float32 only and ignores tensors it did not ask for
(tiny_llm/runtime/cuda/cuda_runtime.cpp:346-361,
tiny_llm/weight_managers/safetensors/weight_manager.cpp:16-22, 88-93).  Here every
problem of a checkpoint is collected into ONE error that lists missing tensors,
unexpected tensors and wrong shapes.  Tensors that an architecture's checkpoints
carry without any part needing them are named by the architecture's ModelSpec
(`ignorable_tensors`), not here.

Element types: matrices take the engine's type (bfloat16 for serving, float32 for
the 32-bit path); vectors (norm weights) do too, except that in bfloat16 serving
a vector stored in 32 bits stays in 32 bits; integer tables become int32.

Random weights are a pure function of (seed, tensor name, element index), the same
bits on the host (files for tests) and on the device (`init_random_weights`):
    x = key + (index + 1) * 0x9E3779B97F4A7C15   (mod 2^64), key = sha256("seed/name")[:8]
    x = splitmix64 finaliser of x
    z = NORMAL_TABLE[x >> 44]      (2^20 quantiles of N(0, 1), rounded to float32 once on the host)
    value = std * z                (or 1 + norm_std * z for norm weights), each operation rounded
                                   to float32 by itself
"""
from __future__ import annotations

import fnmatch
import hashlib
import json
import os
from typing import Callable, Dict, Iterable, Mapping, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import WeightSpec
from .safetensors_io import SafetensorsError, open_model_files, save_file

_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


class WeightLoadError(RuntimeError):
    def __init__(self, where: str, missing, unexpected, wrong_shape, wrong_type=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_type = list(wrong_type)
        lines = [f"cannot load weights from {where}:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} expected {list(e)} found {list(f)}" for n, e, f in self.wrong_shape))
        if self.wrong_type:
            lines.append(f"  wrong element types ({len(self.wrong_type)}): " + "; ".join(
                f"{n} is {t}" for n, t in self.wrong_type))
        super().__init__("\n".join(lines))


def target_dtype(spec: WeightSpec, stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if spec.role == "table":
        return torch.int32
    if spec.role == "vector" and engine_dtype == torch.bfloat16 and stored in (torch.float32, torch.float64):
        return torch.float32
    return engine_dtype


def check_against(specs: Sequence[WeightSpec], available: Mapping[str, Tuple[torch.dtype, Tuple[int, ...]]],
                  where: str, ignorable: Iterable[str] = ()) -> Dict[str, str]:
    """Compares what the parts need with what a checkpoint holds.  Returns
    {needed name -> name to read}; raises WeightLoadError listing every problem.
    `ignorable`: glob patterns of tensors that may be present without being needed."""
    missing, wrong_shape, wrong_type = [], [], []
    source: Dict[str, str] = {}
    used = set()
    for s in specs:
        # a tied tensor reads its alias; a copy of it under its own name is tolerated
        if s.alias_of and s.alias_of in available:
            name = s.alias_of
            used.add(s.name)
        elif s.name in available:
            name = s.name
        else:
            missing.append(s.name)
            continue
        used.add(name)
        dt, shape = available[name]
        if tuple(shape) != tuple(s.shape):
            wrong_shape.append((name, tuple(s.shape), tuple(shape)))
        if (s.role == "table") == (dt in _FLOATS):
            wrong_type.append((name, str(dt)))
        source[s.name] = name
    expected_names = {s.name for s in specs}
    ignorable = tuple(ignorable)
    unexpected = sorted(n for n in available if n not in used and n not in expected_names
                        and not any(fnmatch.fnmatch(n, pat) for pat in ignorable))
    if missing or unexpected or wrong_shape or wrong_type:
        raise WeightLoadError(where, missing, unexpected, wrong_shape, wrong_type)
    return source


class WeightSlab:
    """ONE device allocation that holds every resident weight, each at a 256-byte boundary, as the
    reference places all weights in one static arena (tiny_llm/runtime/cuda/cuda_runtime.cpp:139-145).
    Parts make their resident tensors in `bind` (fused, interleaved or as they came); `adopt` moves
    what a part holds into the slab and hands the part views of it."""
    ALIGN = 256

    def __init__(self, nbytes: int, device):
        self.buffer = torch.empty(max(int(nbytes), self.ALIGN), dtype=torch.uint8, device=device)
        self.used = 0
        self.outside = 0        # bytes of part tensors that found no room (a part that makes more than it was given)

    def place(self, t: torch.Tensor) -> torch.Tensor:
        n = t.numel() * t.element_size()
        start = -(-self.used // self.ALIGN) * self.ALIGN
        if n == 0 or start + n > self.buffer.numel():
            self.outside += n
            return t
        view = self.buffer[start:start + n].view(t.dtype).view(t.shape)
        view.copy_(t)
        self.used = start + n
        return view

    def adopt(self, part, shared: Dict[Tuple[int, int], torch.Tensor], alive: Iterable[torch.Tensor]) -> None:
        """Moves the tensors `part` holds on the slab's device into the slab.  `alive`: fetched
        tensors that a later part will receive again (a tied head); what becomes of them is kept in
        `shared`, so that the later part gets the same view and not a second copy."""
        alive_keys = {(t.data_ptr(), t.numel() * t.element_size()) for t in alive}
        here: Dict[Tuple[int, int], torch.Tensor] = {}      # one tensor under two names of this part
        for attr, val in list(vars(part).items()):
            if not (isinstance(val, torch.Tensor) and val.device == self.buffer.device and val.is_contiguous()):
                continue
            key = (val.data_ptr(), val.numel() * val.element_size())
            known = shared.get(key, here.get(key))
            if known is not None and known.dtype == val.dtype:
                setattr(part, attr, known.view(val.shape))
                continue
            view = self.place(val)
            setattr(part, attr, view)
            here[key] = view
            if key in alive_keys:
                shared[key] = view


def _bind_all(decoder, make: Callable[[WeightSpec], torch.Tensor], source_name: Callable[[WeightSpec], str],
              dtype_of: Callable[[WeightSpec], torch.dtype]) -> None:
    """Every part receives the tensors it declared (`make` builds one on the decoder's device, of
    type `dtype_of`; specs with one `source_name` share it) and binds them; what it then holds moves
    into the decoder's weight slab."""
    specs = decoder.weight_specs()
    uses: Dict[str, int] = {}
    sizes: Dict[Tuple[str, torch.dtype], int] = {}
    for s in specs:
        uses[source_name(s)] = uses.get(source_name(s), 0) + 1
        n = 1
        for d in s.shape:
            n *= int(d)
        sizes[(source_name(s), dtype_of(s))] = n * torch.empty((), dtype=dtype_of(s)).element_size()
    parts = decoder.parts()
    total = sum(-(-b // WeightSlab.ALIGN) * WeightSlab.ALIGN for b in sizes.values()) + WeightSlab.ALIGN * len(parts)
    slab = WeightSlab(total, decoder.device)
    cache: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
    shared: Dict[Tuple[int, int], torch.Tensor] = {}
    for part in parts:
        tensors = {}
        for s in part.weights():
            key = (source_name(s), dtype_of(s))
            t = cache.get(key)
            if t is None:
                t = make(s)
                if uses[source_name(s)] > 1:
                    cache[key] = t
            tensors[s.name] = t
        part.bind(tensors)
        slab.adopt(part, shared, cache.values())
    decoder.weight_slab = slab


class Checkpoint:
    """Tensors by name: the safetensors files of a model folder, shadowed by tensors set by hand.

    `set_tensor(name, tensor)` copies the tensor into an in-memory map that is looked at before
    the files, as the reference's weight manager does (tiny_llm/weight_managers/safetensors/
    weight_manager.cpp:74-114): a way to inject or replace single tensors without writing a file."""

    def __init__(self, folder: Optional[str] = None):
        self.folder = folder
        self._files = open_model_files(folder) if folder is not None else []
        self._where = {}
        for f in self._files:
            for n in f.names():
                self._where[n] = f
        self._overlay: Dict[str, torch.Tensor] = {}

    def names(self):
        return list(dict.fromkeys(list(self._overlay) + list(self._where)))

    def __contains__(self, name: str) -> bool:
        return name in self._overlay or name in self._where

    def _missing(self, name: str):
        return SafetensorsError(f"tensor {name} cannot be found in {self.folder or 'the checkpoint'}")

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        if name in self._overlay:
            t = self._overlay[name]
            return t.dtype, tuple(t.shape)
        if name in self._where:
            return self._where[name].info(name)
        raise self._missing(name)

    def get(self, name: str) -> torch.Tensor:
        if name in self._overlay:
            return self._overlay[name]
        if name in self._where:
            return self._where[name].get(name)
        raise self._missing(name)

    def set_tensor(self, name: str, tensor: torch.Tensor) -> None:
        if tensor.numel() == 0:
            raise ValueError(f"tensor {name} is empty")
        self._overlay[name] = tensor.detach().to("cpu", copy=True).contiguous()


def load_weights(decoder, source) -> None:
    """Reads every tensor the decoder's parts declare onto its device.  `source` is a model
    folder or a Checkpoint (a folder's files with tensors set by hand on top)."""
    ckpt = source if isinstance(source, Checkpoint) else Checkpoint(source)
    available = {n: ckpt.info(n) for n in ckpt.names()}
    specs = decoder.weight_specs()
    source_of = check_against(specs, available, ckpt.folder or "the checkpoint",
                              getattr(decoder.spec, "ignorable_tensors", ()))

    def dtype_of(s: WeightSpec) -> torch.dtype:
        return target_dtype(s, available[source_of[s.name]][0], decoder.dtype)

    def make(s: WeightSpec) -> torch.Tensor:
        return ckpt.get(source_of[s.name]).to(device=decoder.device, dtype=dtype_of(s), non_blocking=False).contiguous()

    _bind_all(decoder, make, lambda s: source_of[s.name], dtype_of)


# ------------------------------------------------------------------ random weights
_GOLDEN = 0x9E3779B97F4A7C15
_MASK64 = (1 << 64) - 1
TABLE_BITS = 20
_table_host: Optional[np.ndarray] = None
_table_dev: Dict[str, torch.Tensor] = {}


def normal_table() -> np.ndarray:
    """2^20 quantiles of N(0, 1) at the bucket midpoints, float32.  Made once on the host; the
    device receives a copy, so both sides gather the same bits."""
    global _table_host
    if _table_host is None:
        n = 1 << TABLE_BITS
        u = (torch.arange(n, dtype=torch.float64) + 0.5) / n
        _table_host = (torch.erfinv(2.0 * u - 1.0) * (2.0 ** 0.5)).to(torch.float32).numpy()
    return _table_host


def tensor_key(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}/{name}".encode()).digest()[:8], "little")


def _standard_normal_host(key: int, n: int, chunk: int = 1 << 18) -> np.ndarray:
    table = normal_table()
    out = np.empty(n, dtype=np.float32)
    base = np.arange(1, chunk + 1, dtype=np.uint64) * np.uint64(_GOLDEN)
    for s in range(0, n, chunk):
        m = min(chunk, n - s)
        x = base[:m] + np.uint64((key + s * _GOLDEN) & _MASK64)
        x ^= x >> np.uint64(30)
        x *= np.uint64(0xBF58476D1CE4E5B9)
        x ^= x >> np.uint64(27)
        x *= np.uint64(0x94D049BB133111EB)
        x ^= x >> np.uint64(31)
        x >>= np.uint64(64 - TABLE_BITS)
        out[s:s + m] = table[x]
    return out


def _scale_and_shift(spec: WeightSpec, std: float, norm_std: float) -> Tuple[float, float]:
    """value = shift + scale * z for this tensor."""
    if spec.init in ("ones", "around_one"):
        return float(norm_std), 1.0
    return float(std), 0.0


def random_tensor(spec: WeightSpec, seed: int, std: float, norm_std: float, device="cpu",
                  dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """The tensor that (seed, name) stands for, float32 rounded to `dtype`; independent of load
    order, and the same bits whether it is made on the host or on a GPU."""
    if spec.role == "table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    scale, shift = _scale_and_shift(spec, std, norm_std)
    n = int(np.prod(spec.shape, dtype=np.int64)) if spec.shape else 1
    key = tensor_key(seed, spec.name)
    dev = torch.device(device)
    if dev.type == "cpu":
        if scale == 0.0:
            t = torch.full((n,), shift, dtype=torch.float32)
        else:
            v = _standard_normal_host(key, n) * np.float32(scale)      # rounded to float32
            if shift != 0.0:
                v = v + np.float32(shift)                              # rounded again
            t = torch.from_numpy(v)
        return t.reshape(spec.shape).to(dtype)
    from ..kernels import ops
    tab = _table_dev.get(str(dev))
    if tab is None:
        tab = _table_dev[str(dev)] = torch.from_numpy(normal_table()).to(dev)
    out = torch.empty(spec.shape, dtype=dtype, device=dev)
    return ops.random_normal(out, tab, key, scale, shift)


def init_random_weights(decoder, seed: int = 0, std: float = 0.02, norm_std: float = 0.0) -> None:
    """Fills the decoder with seeded random weights on its device, without a file: the tensors
    `write_random_model` would store for the same seed, rounded to the engine's types."""
    dev = decoder.device

    def source_name(s: WeightSpec) -> str:
        return s.alias_of if s.alias_of else s.name

    def dtype_of(s: WeightSpec) -> torch.dtype:
        return target_dtype(s, torch.float32, decoder.dtype)

    def make(s: WeightSpec) -> torch.Tensor:
        base = WeightSpec(source_name(s), s.shape, s.role, s.init)
        return random_tensor(base, seed, std, norm_std, device=dev, dtype=dtype_of(s))

    _bind_all(decoder, make, source_name, dtype_of)


def write_random_model(folder: str, config: Mapping, seed: int = 0, std: Optional[float] = None,
                       norm_std: float = 0.0, dtype: str = "float32") -> str:
    """Writes `config.json` and `model.safetensors` for `config` (the architecture's own
    config.json keys) with weights drawn from `seed`.  Tied heads are not stored."""
    from ..config.registry import resolve
    from ..models.decoder import Decoder, TORCH_DTYPES

    os.makedirs(folder, exist_ok=True)
    cfg, spec = resolve(config)
    if std is None:
        std = float(config.get("initializer_range", 0.02))
    store = TORCH_DTYPES[{"fp32": "float32", "bf16": "bfloat16"}.get(dtype, dtype)]
    # the decoder is only asked which tensors it needs: sizes the bfloat16 kernels refuse do not
    # matter for a file, so it is built for float32
    dec = Decoder(spec, dtype="float32", device="cpu")
    tensors = {}
    for s in dec.weight_specs():
        if s.alias_of:
            continue
        tensors[s.name] = random_tensor(s, seed, std, norm_std, dtype=torch.int32 if s.role == "table" else store)
    out_cfg = dict(config)
    out_cfg["torch_dtype"] = "float32" if store == torch.float32 else "bfloat16"
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(out_cfg, f, indent=2)
    save_file(tensors, os.path.join(folder, "model.safetensors"), {"format": "pt", "seed": str(seed)})
    return folder
