from .token_shift import ddlerp
from .loras import expand_loras
from .wkv_attn import attn, load_attn, WindRWKV7
from .wkv_attn_ln import attn_ln, load_attn_ln, WindRWKV7LN

__version__ = '0.1'
