from .llama import LlamaConfig, ConfigError
from .engine import EngineConfig
from .spec import PartSpec, LayerSpec, PlanEntry, ModelSpec, pre_norm_layer
from .registry import (register_architecture, unregister_architecture, known_architectures,
                       resolve, resolve_folder, read_config_json, UnknownArchitecture)
