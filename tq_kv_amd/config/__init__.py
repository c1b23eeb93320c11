from .base import ConfigError, KeyReader, read_config_json
from .registry import (architecture_name, config_from_dict, known_architectures, load_config,
                       register_architecture, spec_for)

__all__ = ["ConfigError", "KeyReader", "read_config_json", "architecture_name", "config_from_dict",
           "known_architectures", "load_config", "register_architecture", "spec_for"]
