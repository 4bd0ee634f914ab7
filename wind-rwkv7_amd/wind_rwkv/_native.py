"""ctypes binding of the C-ABI library (include/wind_rwkv7.h).

The HIP library is the only implementation: if it is missing, importing the ops fails loudly
instead of falling back to anything slower.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# WIND_RWKV7_LIB names another build of the same library (e.g. one compiled with different options)
LIB_PATH = os.environ.get('WIND_RWKV7_LIB') or os.path.join(_PKG_DIR, 'lib', 'libwind_rwkv7.so')

BF16, F32 = 0, 1  # WIND_RWKV7_BF16 / WIND_RWKV7_F32


class WindRwkv7Error(RuntimeError):
    """A C-ABI entry point returned a non-zero WIND_RWKV7_ERR_* code."""

    def __init__(self, code, message):
        super().__init__(f'wind_rwkv7 error {code}: {message}')
        self.code = code


_vp, _i, _sz, _ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_longlong

# name -> (restype, argtypes); mirrors include/wind_rwkv7.h one to one
SIGNATURES = {
    'wind_rwkv7_abi_version': (_i, []),
    'wind_rwkv7_strerror': (ctypes.c_char_p, [_i]),
    'wind_rwkv7_head_size_supported': (_i, [_i]),
    'wind_rwkv7_attn_head_size_supported': (_i, [_i]),
    'wind_rwkv7_f32_head_size_supported': (_i, [_i]),
    'wind_rwkv7_copy_columns': (_i, [_ll, _i] + [_vp] * 10),
    'wind_rwkv7_cast_to_bf16': (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp]),
    'wind_rwkv7_chunk_len': (_i, []),
    'wind_rwkv7_checkpoint_interval': (_i, []),
    'wind_rwkv7_set_checkpoint_interval': (_i, [_i]),
    'wind_rwkv7_attn_saved_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_fwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_bwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_forward': (_i, [_i] * 6 + [_vp] * 7 + [_vp] * 3 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_prefill': (_i, [_i] * 6 + [_vp] * 7 + [_vp] * 3 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_prefill_static_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_prefill_static': (_i, [_i] * 6 + [_vp] * 7 + [_vp] * 2 + [_vp]),
    'wind_rwkv7_attn_backward': (_i, [_i] * 6 + [_vp] * 6 + [_vp] * 3 + [_vp] * 7 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_ln_saved_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_ln_fwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_ln_bwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_ln_forward': (_i, [_i] * 6 + [_vp] * 9 + [_vp] * 3 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_ln_prefill': (_i, [_i] * 6 + [_vp] * 9 + [_vp] * 3 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_ln_backward': (_i, [_i] * 6 + [_vp] * 8 + [_vp] * 3 + [_vp] * 9 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_decode': (_i, [_i] * 5 + [_vp] * 6 + [_vp, _vp, _vp]),
    'wind_rwkv7_attn_ln_decode': (_i, [_i] * 5 + [_vp] * 8 + [_vp, _vp, _vp]),
    'wind_rwkv7_mixer_decode_workspace_bytes': (_sz, [_i, _i]),
    'wind_rwkv7_mixer_decode': (_i, [_i] * 4 + [_vp] * 6 + [_vp, _sz, _vp]),
    'wind_rwkv7_ddlerp_rank_supported': (_i, [_i]),
    'wind_rwkv7_ddlerp_bwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_ddlerp_forward': (_i, [_i] * 4 + [_vp] * 5 + [_vp] * 3 + [_vp]),
    'wind_rwkv7_ddlerp_backward': (_i, [_i] * 4 + [_vp] * 7 + [_vp] * 4 + [_vp] * 5 + [_vp, _sz, _vp]),
    'wind_rwkv7_ln_epilogue_bwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_ln_epilogue_forward': (_i, [_i] * 4 + [_vp] * 8),
    'wind_rwkv7_ln_epilogue_backward': (_i, [_i] * 4 + [_vp] * 13 + [_vp, _sz, _vp]),
    'wind_rwkv7_expand_loras_rank_supported': (_i, [_i]),
    'wind_rwkv7_expand_loras_bwd_workspace_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_expand_loras_forward': (_i, [_i] * 5 + [_vp] * 14 + [_vp] * 4 + [_vp]),
    'wind_rwkv7_expand_loras_backward': (_i, [_i] * 5 + [_vp] * 14 + [_vp] * 4 + [_vp] * 14 + [_vp, _sz, _vp]),
    'wind_rwkv7_attn_f32_saved_bytes': (_sz, [_i] * 4),
    'wind_rwkv7_attn_f32_forward': (_i, [_i] * 4 + [_vp] * 7 + [_vp] * 3 + [_vp]),
    'wind_rwkv7_attn_f32_prefill': (_i, [_i] * 4 + [_vp] * 7 + [_vp] * 2 + [_vp]),
    'wind_rwkv7_attn_f32_backward': (_i, [_i] * 4 + [_vp] * 6 + [_vp] * 3 + [_vp] * 7 + [_vp]),
    'wind_rwkv7_linear_wgrad_workspace_bytes': (_sz, [_ll, _i, _i]),
    'wind_rwkv7_linear_wgrad': (_i, [_ll, _i, _i, _vp, _ll, _vp, _ll, _vp, _i, _vp, _sz, _vp]),
    'wind_rwkv7_linear_wgrad_group_workspace_bytes': (_sz, [_i, _ll, _vp, _vp]),
    'wind_rwkv7_linear_wgrad_group': (_i, [_i, _ll, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _sz, _vp]),
    'wind_rwkv7_profile_enable': (_i, [_i]),
    'wind_rwkv7_profile_read': (_i, [_i, ctypes.POINTER(ctypes.c_float), _i]),
    'wind_rwkv7_profile_kernel_name': (ctypes.c_char_p, [_i, _i]),
}

# wind_rwkv7_mixer_weights: the time mixer's parameters in the header's order (bf16 device pointers, ln_params fp32)
MIXER_WEIGHT_NAMES = ('time_maa_x', 'time_maa', 'time_maa_w1', 'time_maa_w2', 'Wr', 'Wk', 'Wv', 'Wo',
                      'gate_w1', 'time_decay_w1', 'time_kkk_w1', 'mk_w1', 'time_aaa_w1', 'ma_w1',
                      'gate_w2', 'time_decay_w2', 'time_kkk_w2', 'mk_w2', 'time_aaa_w2', 'ma_w2',
                      'time_decay', 'time_aaaaa', 'time_misc_a', 'time_misc_k', 'ln_params')


class MixerWeights(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in MIXER_WEIGHT_NAMES]


_lib = None


def lib():
    """The loaded library; raises ImportError with build instructions if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f'{LIB_PATH} is missing: build it with `make -C {os.path.dirname(_PKG_DIR)}` '
                '(hipcc, --offload-arch=gfx950). There is no fallback implementation.')
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise WindRwkv7Error(code, lib().wind_rwkv7_strerror(code).decode())
