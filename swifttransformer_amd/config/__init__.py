from .hyper_param import OptHyperParam, ConfigError
from .cache_param import CacheParam
from .registry import (register_architecture, resolve_architecture, registered_architectures,
                       hyper_param_from_dir, read_config, Architecture)

from .presets import preset, preset_names

__all__ = ["preset", "preset_names", "OptHyperParam", "ConfigError", "CacheParam", "register_architecture",
           "resolve_architecture", "registered_architectures", "hyper_param_from_dir",
           "read_config", "Architecture"]
