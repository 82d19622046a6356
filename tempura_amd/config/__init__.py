from .spec import PartSpec, LayerSpec, LayerCall, ModelSpec
from .llama import LlamaConfig, RopeScaling, ConfigError, PRESETS
from .registry import register_architecture, architecture_names, config_class_for, load_config

__all__ = ["PartSpec", "LayerSpec", "LayerCall", "ModelSpec", "LlamaConfig", "RopeScaling",
           "ConfigError", "PRESETS", "register_architecture", "architecture_names",
           "config_class_for", "load_config"]
