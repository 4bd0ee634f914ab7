"""Module path of the reference (time_mixer.py); the implementation lives in mixer.py."""
from .mixer import TimeMixer, ref_attn  # noqa: F401
