"""Module path of the reference (rwkv7_attn_triton.py); the implementation lives in wkv_attn.py."""
from .wkv_attn import attn_triton  # noqa: F401
