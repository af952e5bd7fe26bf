"""Typed configurations, the description of a model as parts, and the architecture registry."""
from .registry import (ConfigError, config_class_for, config_from_dict, config_from_dir, config_source,
                       preset_dict, preset_names, register_architecture, registered_architectures)
from .spec import LayerCall, ModelSpec, PartSpec, Stored, TensorRef, joined, tensor
from .qwen3 import Qwen3Config

__all__ = ["ConfigError", "config_class_for", "config_from_dict", "config_from_dir", "config_source", "preset_dict",
           "preset_names", "register_architecture",
           "registered_architectures", "LayerCall", "ModelSpec", "PartSpec", "Stored", "TensorRef", "joined", "tensor",
           "Qwen3Config"]
