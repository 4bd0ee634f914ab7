"""Module path of the reference (rwkv7_attn_triton_bighead.py); the implementation lives in wkv_attn.py."""
from .wkv_attn import attn_triton_bighead  # noqa: F401
