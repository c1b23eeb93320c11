"""One registry from an architecture's name to its configuration class and the
function that turns a configuration into a ModelSpec.

The reference only sniffs `model_type` for the rotary layout and otherwise guesses
from tensor presence (src/models/turbo_generic.rs:2028-2029, :2103-2135).  Here
config.json's `architectures[0]`, or `model_type`, picks the architecture, and an
unknown name is an error that lists the known ones (in the manner of
src/hub.rs:317-330).
"""
from .base import ConfigError, read_config_json

_ARCHITECTURES = {}      # name -> (config class, spec builder)
_ALIASES = {}            # model_type -> name


def register_architecture(name, config_class, spec_builder, model_types=()):
    _ARCHITECTURES[name] = (config_class, spec_builder)
    for mt in model_types:
        _ALIASES[mt] = name


def known_architectures():
    return sorted(_ARCHITECTURES)


def architecture_name(raw):
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs:
        name = archs[0]
        if name in _ARCHITECTURES:
            return name
        raise ConfigError("Unknown architecture '%s'. Known architectures: %s" % (name, ", ".join(known_architectures())))
    mt = raw.get("model_type")
    if mt in _ALIASES:
        return _ALIASES[mt]
    raise ConfigError("config.json names no known architecture (architectures=%r, model_type=%r). "
                      "Known architectures: %s" % (archs, mt, ", ".join(known_architectures())))


def config_from_dict(raw, where="config.json"):
    """(architecture name, typed configuration) of a parsed config.json."""
    if not isinstance(raw, dict):
        raise ConfigError("%s: expected a JSON object at the top level" % where)
    name = architecture_name(raw)
    return name, _ARCHITECTURES[name][0].from_dict(raw, where)


def load_config(model_dir):
    return config_from_dict(read_config_json(model_dir))


def spec_for(name, config):
    return _ARCHITECTURES[name][1](config)
