from .llama4 import ConfigError, Llama4TextConfig, RopeScaling
from .registry import (UnknownArchitectureError, architecture_name, get_architecture, known_architectures,
                       load_config, read_config_json, register_architecture)
from .specs import LayerSpec, ModelPlan, OrderEntry, PartSpec, default_order, part

__all__ = [
    "ConfigError", "Llama4TextConfig", "RopeScaling", "UnknownArchitectureError", "architecture_name",
    "get_architecture", "known_architectures", "load_config", "read_config_json", "register_architecture",
    "LayerSpec", "ModelPlan", "OrderEntry", "PartSpec", "default_order", "part",
]
