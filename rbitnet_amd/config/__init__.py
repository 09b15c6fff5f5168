from .spec import PartSpec, LayerSpec, ModelSpec
from .llama import LlamaConfig, RopeScaling
from .registry import (register_architecture, registered_architectures, config_class_for,
                       architecture_of, load_config)

__all__ = ["PartSpec", "LayerSpec", "ModelSpec", "LlamaConfig", "RopeScaling", "register_architecture",
           "registered_architectures", "config_class_for", "architecture_of", "load_config"]
