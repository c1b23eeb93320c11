"""Architectures: the Python mirrors of their typed configurations (the architectures themselves
are registered in the engine library, one file each under csrc/engine/)."""
from . import qwen2  # noqa: F401
