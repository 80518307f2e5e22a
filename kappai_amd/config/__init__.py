from .base import (Architecture, ConfigError, ModelConfig, architecture_name, config_from_dict,
                   known_architectures, load_config, lookup_architecture, register_architecture)
from .lfm2 import Lfm2Config, adjusted_ff_dim
from .shapes import SHAPES, named_shape

__all__ = ["Architecture", "ConfigError", "ModelConfig", "architecture_name", "config_from_dict",
           "known_architectures", "load_config", "lookup_architecture", "register_architecture",
           "Lfm2Config", "adjusted_ff_dim", "SHAPES", "named_shape"]
