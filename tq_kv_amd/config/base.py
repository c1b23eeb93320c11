"""Reading config.json.

The reference indexes an untyped JSON value and falls back to defaults
(src/models/turbo_generic.rs:2007-2030).  Here every key is read by the engine library through a
small typed reader (csrc/engine/spec.cpp: KeyReader), so a configuration can say exactly which
key is missing or has the wrong type; this module asks the library.
"""
import json

from .. import native
from ..native import ConfigError

__all__ = ["ConfigError", "read_config_json"]


def read_config_json(model_dir):
    """The parsed config.json of a model folder.

    Error texts follow the reference's (src/models/turbo_generic.rs:2008-2011).
    """
    return json.loads(native.text(native.library().tqe_read_config(native.enc(str(model_dir)))))
