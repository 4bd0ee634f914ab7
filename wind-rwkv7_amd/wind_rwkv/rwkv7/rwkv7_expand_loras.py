"""Module path of the reference (rwkv7_expand_loras.py); the implementation lives in loras.py."""
from .loras import expand_loras, ExpandLoras  # noqa: F401
