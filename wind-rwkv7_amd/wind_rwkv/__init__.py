"""wind_rwkv for MI355X (gfx950): RWKV-7 time-mixer kernels behind the API of johanwind/wind-rwkv7."""
import wind_rwkv.rwkv7

__version__ = '0.1'
