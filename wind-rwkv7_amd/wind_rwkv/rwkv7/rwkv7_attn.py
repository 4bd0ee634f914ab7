"""Module path of the reference (rwkv7_attn.py); the implementation lives in wkv_attn.py."""
from .wkv_attn import attn, load_attn, WindRWKV7, fw_attn, bw_attn  # noqa: F401
