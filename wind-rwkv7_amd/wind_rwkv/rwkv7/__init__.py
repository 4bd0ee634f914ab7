from .wkv_attn import attn, load_attn, WindRWKV7

__version__ = '0.1'
