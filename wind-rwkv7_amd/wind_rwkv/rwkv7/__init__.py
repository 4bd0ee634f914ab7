from .token_shift import ddlerp
from .loras import expand_loras
from .wkv_attn_ln import attn_ln, attn_ln_step, load_attn_ln, WindRWKV7LN
from .wkv_attn import attn, attn_step, load_attn, attn_triton, attn_triton_bighead, WindRWKV7, WindRWKV7F32
from .wkv_attn import checkpoint_interval, set_checkpoint_interval
from .linear import linear_wgrad, linear_wgrad_group, projection, projection_sets, projections
from .mixer import TimeMixer

__version__ = '0.1'
