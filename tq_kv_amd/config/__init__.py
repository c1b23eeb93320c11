from . import catalog
from .base import ConfigError, read_config_json
from .registry import config_from_dict, known_architectures, load_config, spec_for, spec_from_dict

__all__ = ["catalog", "ConfigError", "read_config_json", "config_from_dict", "known_architectures", "load_config", "spec_for",
           "spec_from_dict"]
