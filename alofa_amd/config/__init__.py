from .base import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry
from .registry import (architectures, config_class, config_from_dict, load_config,
                       register_architecture)

__all__ = ["LayerSpec", "ModelConfig", "ModelSpec", "PartSpec", "RunEntry", "architectures",
           "config_class", "config_from_dict", "load_config", "register_architecture"]
