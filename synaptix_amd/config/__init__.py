from .errors import ConfigError
from .qwen3 import Qwen3Config
from .bizipel import BizipelConfig
from .kamivik import KamivikConfig
from .repolix import RepolixConfig
from .nilepel import NilepelConfig
from .registry import (Architecture, register_architecture, resolve_architecture, known_architectures,
                       load_config, read_config_json)

__all__ = ["ConfigError", "Qwen3Config", "BizipelConfig", "KamivikConfig", "RepolixConfig", "NilepelConfig", "Architecture", "register_architecture", "resolve_architecture",
           "known_architectures", "load_config", "read_config_json"]
