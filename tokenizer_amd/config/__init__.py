from .base import ConfigError, ModelConfig, read_config_json
from .registry import (Architecture, architecture_name, get_architecture, load_config,
                       register_architecture, registered_architectures)
from .qwen2 import Qwen2Config
from .napadra import NapadraConfig
from .dolidra import DolidraConfig
from .bokulorn import BokulornConfig
from .zomavik import ZomavikConfig

__all__ = ["ConfigError", "ModelConfig", "read_config_json", "Architecture", "architecture_name",
           "get_architecture", "load_config", "register_architecture", "registered_architectures",
           "Qwen2Config", "NapadraConfig", "DolidraConfig", "BokulornConfig", "ZomavikConfig"]
