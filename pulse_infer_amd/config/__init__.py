from .base import ConfigError, JsonReader, ModelConfig
from .registry import (ArchitectureEntry, config_from_dict, load_config, lookup_architecture,
                       register_architecture, registered_architectures, unregister_architecture)
from .qwen3 import Qwen3Config
from .dirozen import DirozenConfig
from .kesovik import KesovikConfig
from .tipidra import TipidraConfig
from .fosupel import FosupelConfig

register_architecture(Qwen3Config.architecture, Qwen3Config, replace=True)
register_architecture(DirozenConfig.architecture, DirozenConfig, replace=True)
register_architecture(KesovikConfig.architecture, KesovikConfig, replace=True)
register_architecture(TipidraConfig.architecture, TipidraConfig, replace=True)
register_architecture(FosupelConfig.architecture, FosupelConfig, replace=True)

__all__ = [
    "ConfigError", "JsonReader", "ModelConfig", "ArchitectureEntry", "config_from_dict", "load_config",
    "lookup_architecture", "register_architecture", "registered_architectures",
    "unregister_architecture", "Qwen3Config", "DirozenConfig", "KesovikConfig", "TipidraConfig", "FosupelConfig",
]
