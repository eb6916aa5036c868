"""One registry from an architecture's name (config.json `architectures[0]`) to
its typed configuration class and its ModelSpec builder.

The reference selects the model with an enum passed by the caller and never
looks at `architectures` (tiny_llm/pipeline/pipeline.hpp:8-10,
tiny_llm/pipeline/pipeline.cpp:30-31); here config.json chooses.
"""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict, Mapping, Tuple

from .spec import ModelSpec

_ARCHITECTURES: Dict[str, Tuple[Callable[[Mapping[str, Any]], Any], Callable[[Any], ModelSpec]]] = {}


class UnknownArchitecture(KeyError):
    pass


def register_architecture(name: str, read_config: Callable[[Mapping[str, Any]], Any],
                          build_spec: Callable[[Any], ModelSpec], *, replace: bool = False) -> None:
    """`read_config(dict) -> typed config`, `build_spec(config) -> ModelSpec`."""
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = (read_config, build_spec)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures():
    return sorted(_ARCHITECTURES)


def architecture_name(raw: Mapping[str, Any]) -> str:
    arch = raw.get("architectures")
    if isinstance(arch, (list, tuple)) and arch:
        return str(arch[0])
    if isinstance(arch, str):
        return arch
    raise UnknownArchitecture(
        "config.json has no `architectures`; known: " + ", ".join(known_architectures()))


def resolve(raw: Mapping[str, Any]):
    """Raw config.json dict -> (typed config, ModelSpec)."""
    name = architecture_name(raw)
    if name not in _ARCHITECTURES:
        raise UnknownArchitecture(
            f"no model registered for architecture {name!r}; known: "
            + ", ".join(known_architectures()))
    read_config, build_spec = _ARCHITECTURES[name]
    cfg = read_config(raw)
    spec = build_spec(cfg)
    spec.validate()
    return cfg, spec


def read_config_json(model_path: str) -> dict:
    path = os.path.join(model_path, "config.json") if os.path.isdir(model_path) else model_path
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def resolve_folder(model_path: str):
    return resolve(read_config_json(model_path))
