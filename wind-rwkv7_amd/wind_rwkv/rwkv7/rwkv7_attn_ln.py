"""Module path of the reference (rwkv7_attn_ln.py); the implementation lives in wkv_attn_ln.py."""
from .wkv_attn_ln import attn_ln, load_attn_ln, WindRWKV7LN as WindRWKV7, fw_attn_ln, bw_attn_ln  # noqa: F401
