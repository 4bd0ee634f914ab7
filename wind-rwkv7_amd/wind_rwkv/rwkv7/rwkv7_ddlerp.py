"""Module path of the reference (rwkv7_ddlerp.py); the implementation lives in token_shift.py."""
from .token_shift import ddlerp, DDLerp  # noqa: F401
