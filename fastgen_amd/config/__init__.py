from .layout import LayerSpec, ModelLayout, PartSpec, RunEntry
from .model_args import ConfigError, ModelArgs, RopeArgs, architecture_name, read_config_json
from .registry import (
    Architecture,
    get_architecture,
    register_architecture,
    registered_architectures,
    unregister_architecture,
)
from . import llama as _llama  # registers LlamaForCausalLM

__all__ = [
    "Architecture",
    "ConfigError",
    "LayerSpec",
    "ModelArgs",
    "ModelLayout",
    "PartSpec",
    "RopeArgs",
    "RunEntry",
    "architecture_name",
    "get_architecture",
    "read_config_json",
    "register_architecture",
    "registered_architectures",
    "unregister_architecture",
]
