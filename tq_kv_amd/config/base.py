"""Typed reading of config.json keys.

The reference indexes an untyped JSON value and falls back to defaults
(src/models/turbo_generic.rs:2007-2030).  Here every key is read through a small
typed reader that records which keys were taken, so a configuration class can say
exactly which key is missing or has the wrong type.
"""
import json
import os


class ConfigError(ValueError):
    """A config.json that cannot be used: missing key, wrong type, bad combination."""


_MISSING = object()


class KeyReader:
    """Reads typed values out of a config.json dictionary."""

    def __init__(self, raw, where="config.json"):
        if not isinstance(raw, dict):
            raise ConfigError("%s: expected a JSON object at the top level" % where)
        self.raw = raw
        self.where = where

    def _get(self, key, default):
        value = self.raw.get(key, _MISSING)
        if value is _MISSING or value is None:
            if default is _MISSING:
                raise ConfigError("%s: missing required key '%s'" % (self.where, key))
            return _MISSING
        return value

    def integer(self, key, default=_MISSING, minimum=None):
        value = self._get(key, default)
        if value is _MISSING:
            return default
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value == int(value):
                value = int(value)
            else:
                raise ConfigError("%s: key '%s' must be an integer, got %r" % (self.where, key, value))
        if minimum is not None and value < minimum:
            raise ConfigError("%s: key '%s' must be >= %d, got %d" % (self.where, key, minimum, value))
        return value

    def number(self, key, default=_MISSING, positive=False):
        value = self._get(key, default)
        if value is _MISSING:
            return default
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError("%s: key '%s' must be a number, got %r" % (self.where, key, value))
        value = float(value)
        if positive and not value > 0.0:
            raise ConfigError("%s: key '%s' must be > 0, got %r" % (self.where, key, value))
        return value

    def boolean(self, key, default=_MISSING):
        value = self._get(key, default)
        if value is _MISSING:
            return default
        if not isinstance(value, bool):
            raise ConfigError("%s: key '%s' must be true or false, got %r" % (self.where, key, value))
        return value

    def string(self, key, default=_MISSING):
        value = self._get(key, default)
        if value is _MISSING:
            return default
        if not isinstance(value, str):
            raise ConfigError("%s: key '%s' must be a string, got %r" % (self.where, key, value))
        return value

    def token_ids(self, key):
        """An id or a list of ids (eos_token_id may be either); absent -> []."""
        value = self.raw.get(key)
        if value is None:
            return []
        values = value if isinstance(value, list) else [value]
        for v in values:
            if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                raise ConfigError("%s: key '%s' must hold token ids, got %r" % (self.where, key, value))
        return list(values)


def read_config_json(model_dir):
    """The parsed config.json of a model folder.

    Error texts follow the reference's (src/models/turbo_generic.rs:2008-2011).
    """
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            text = f.read()
    except OSError as e:
        raise ConfigError("Cannot read config.json: %s" % e)
    try:
        return json.loads(text)
    except ValueError as e:
        raise ConfigError("Invalid config.json: %s" % e)
