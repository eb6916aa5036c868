"""Weights by tensor name, from safetensors or from a seed.

The reference copies each graph tensor from the file under its own name, checks
its shape, accepts float32 only and ignores tensors it did not ask for
(tiny_llm/runtime/cuda/cuda_runtime.cpp:346-361,
tiny_llm/weight_managers/safetensors/weight_manager.cpp:16-22, 88-93).  Here every
problem of a checkpoint is collected into ONE error that lists missing tensors,
unexpected tensors and wrong shapes.

Element types: matrices take the engine's type (bfloat16 for serving, float32 for
the 32-bit path); vectors (norm weights) do too, except that in bfloat16 serving
a vector stored in 32 bits stays in 32 bits; integer tables become int32.
"""
from __future__ import annotations

import fnmatch
import hashlib
import json
import os
from typing import Callable, Dict, Iterable, Mapping, Optional, Sequence, Tuple

import torch

from ..parts.base import WeightSpec
from .safetensors_io import open_model_files, save_file

# tensors that checkpoints of this family carry and no part needs
IGNORABLE = ("*.rotary_emb.inv_freq",)

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
                  where: str, ignorable: Iterable[str] = IGNORABLE) -> Dict[str, str]:
    """Compares what the parts need with what a checkpoint holds.  Returns
    {needed name -> name to read}; raises WeightLoadError listing every problem."""
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
    unexpected = sorted(n for n in available if n not in used and n not in expected_names
                        and not any(fnmatch.fnmatch(n, pat) for pat in ignorable))
    if missing or unexpected or wrong_shape or wrong_type:
        raise WeightLoadError(where, missing, unexpected, wrong_shape, wrong_type)
    return source


def _bind_all(decoder, fetch: Callable[[WeightSpec], torch.Tensor]) -> None:
    cache: Dict[str, torch.Tensor] = {}
    for part in decoder.parts():
        tensors = {}
        for s in part.weights():
            tensors[s.name] = fetch(s, cache)
        part.bind(tensors)


def load_weights(decoder, folder: str) -> None:
    """Reads every tensor the decoder's parts declare from `folder` onto its device."""
    files = open_model_files(folder)
    available, where_is = {}, {}
    for f in files:
        for n in f.names():
            available[n] = f.info(n)
            where_is[n] = f
    specs = decoder.weight_specs()
    source = check_against(specs, available, folder)

    def fetch(s: WeightSpec, cache):
        src = source[s.name]
        stored = available[src][0]
        dt = target_dtype(s, stored, decoder.dtype)
        key = (src, dt)
        if key not in cache:
            cache[key] = where_is[src].get(src).to(device=decoder.device, dtype=dt, non_blocking=False).contiguous()
        return cache[key]

    _bind_all(decoder, fetch)


# ------------------------------------------------------------------ random weights
def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}/{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return g


def random_tensor(spec: WeightSpec, seed: int, std: float, norm_std: float, device="cpu") -> torch.Tensor:
    """The float32 tensor that (seed, name) stands for; independent of load order."""
    if spec.role == "table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    g = _generator(seed, spec.name, device)
    if spec.init == "ones" or spec.init == "around_one":
        t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        if norm_std > 0:
            t += norm_std * torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
        return t
    return std * torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)


def init_random_weights(decoder, seed: int = 0, std: float = 0.02, norm_std: float = 0.0) -> None:
    """Fills the decoder with seeded random weights on its device, without a file."""
    dev = decoder.device

    def fetch(s: WeightSpec, cache):
        name = s.alias_of if s.alias_of else s.name
        dt = target_dtype(s, decoder.dtype, decoder.dtype)
        if name not in cache:
            base = WeightSpec(name, s.shape, s.role, s.init)
            cache[name] = random_tensor(base, seed, std, norm_std, device=dev).to(dt).contiguous()
        return cache[name]

    _bind_all(decoder, fetch)


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
    dec = Decoder(spec, dtype="float32", device="cpu")
    tensors = {}
    for s in dec.weight_specs():
        if s.alias_of:
            continue
        t = random_tensor(s, seed, std, norm_std)
        tensors[s.name] = t if s.role == "table" else t.to(store)
    out_cfg = dict(config)
    out_cfg["torch_dtype"] = "float32" if store == torch.float32 else "bfloat16"
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(out_cfg, f, indent=2)
    save_file(tensors, os.path.join(folder, "model.safetensors"), {"format": "pt", "seed": str(seed)})
    return folder
