from .spec import PartSpec, LayerSpec, LayerCall, ModelSpec
from .llama import LlamaConfig, RopeScaling, ConfigError, PRESETS
from .mifutar import MifutarConfig
from .bomotar import BomotarConfig
from .golavik import GolavikConfig
from .registry import register_architecture, architecture_names, config_class_for, load_config, config_from_file

__all__ = ["PartSpec", "LayerSpec", "LayerCall", "ModelSpec", "LlamaConfig", "MifutarConfig", "BomotarConfig", "GolavikConfig", "RopeScaling",
           "ConfigError", "PRESETS", "register_architecture", "architecture_names",
           "config_class_for", "load_config", "config_from_file"]
