from .llama import ConfigError, LlamaConfig, RopeScaling, llama_model_spec
from .registry import (
    ARCHITECTURES,
    ArchSpec,
    architecture_name,
    architecture_of,
    get_architecture,
    load_config,
    register_architecture,
)
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec, standard_layer

__all__ = [
    "ARCHITECTURES",
    "ArchSpec",
    "ConfigError",
    "LayerRun",
    "LayerSpec",
    "LlamaConfig",
    "ModelSpec",
    "PartSpec",
    "RopeScaling",
    "architecture_name",
    "architecture_of",
    "get_architecture",
    "llama_model_spec",
    "load_config",
    "register_architecture",
    "standard_layer",
]
