from .base import (ArchitectureEntry, ConfigError, ModelConfig, architecture_name,
                   config_from_dict, get_architecture, load_config, register_architecture,
                   registered_architectures, unregister_architecture)
from .mistral import MistralConfig
from .sozetar import SozetarConfig
from .fanitar import FanitarConfig
from .nepisun import NepisunConfig
from .giforax import GiforaxConfig

__all__ = ["ArchitectureEntry", "ConfigError", "ModelConfig", "MistralConfig", "SozetarConfig", "FanitarConfig", "NepisunConfig", "GiforaxConfig", "architecture_name",
           "config_from_dict", "get_architecture", "load_config", "register_architecture",
           "registered_architectures", "unregister_architecture"]
