from .fields import ConfigError
from .gupitar import GupitarConfig
from .qwen2 import Qwen2Config
from .siditar import SiditarConfig
from .zabozen import ZabozenConfig
from .registry import (Architecture, architecture_named, architecture_of, load_config,
                       register_architecture, registered_architectures, unregister_architecture)

__all__ = ["ConfigError", "GupitarConfig", "Qwen2Config", "SiditarConfig", "ZabozenConfig", "Architecture", "architecture_named", "architecture_of",
           "load_config", "register_architecture", "registered_architectures", "unregister_architecture"]
