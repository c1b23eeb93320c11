"""One registry from an architecture's name to its typed configuration and the function that
turns a configuration into a ModelSpec.

The reference only sniffs `model_type` for the rotary layout and otherwise guesses from tensor
presence (src/models/turbo_generic.rs:2028-2029, :2103-2135).  Here config.json's
`architectures[0]`, or `model_type`, picks the architecture, and an unknown name is an error that
lists the known ones (in the manner of src/hub.rs:317-330).  The registry itself lives in the
engine library (csrc/engine/config.cpp, one file per architecture beside it); this module shows
it to Python.
"""
import json

from .. import native
from ..parts.spec import ModelSpec
from .base import ConfigError, read_config_json

_CONFIG_CLASSES = {}        # architecture name -> Python class that mirrors its typed configuration


def config_class(name):
    """Class decorator: the Python mirror of an architecture's typed configuration."""
    def deco(cls):
        _CONFIG_CLASSES[name] = cls
        return cls
    return deco


def known_architectures():
    return native.parsed(native.library().tqe_known_architectures())


def _text(raw, where):
    if not isinstance(raw, dict):
        raise ConfigError("%s: expected a JSON object at the top level" % where)
    return native.enc(json.dumps(raw))


def config_from_dict(raw, where="config.json"):
    """(architecture name, typed configuration) of a parsed config.json."""
    from .. import architectures  # noqa: F401  (the mirrors register themselves)
    out = native.parsed(native.library().tqe_config_parse(_text(raw, where)))
    name, typed = out["architecture"], out["config"]
    cls = _CONFIG_CLASSES.get(name)
    return name, (cls.from_typed(typed) if cls is not None else typed)


def load_config(model_dir):
    return config_from_dict(read_config_json(model_dir))


def spec_from_dict(raw):
    """The ModelSpec the library builds from a parsed config.json."""
    return ModelSpec.from_json(native.parsed(native.library().tqe_config_spec(_text(raw, "config.json"))))


def spec_for(name, config):
    return spec_from_dict(config.to_dict() if hasattr(config, "to_dict") else config)
