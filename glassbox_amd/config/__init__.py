from .base import (ConfigError, ModelConfig, architecture_of, config_from_dict, config_from_dir,
                   known_architectures, lookup, register_architecture)
from .llama import LlamaConfig
from .sagalorn import SagalornConfig
from .dekinex import DekinexConfig
from .vumalix import VumalixConfig
from .tekilix import TekilixConfig

__all__ = ["ConfigError", "ModelConfig", "LlamaConfig", "SagalornConfig", "DekinexConfig", "VumalixConfig", "TekilixConfig", "architecture_of", "config_from_dict",
           "config_from_dir", "known_architectures", "lookup", "register_architecture"]
