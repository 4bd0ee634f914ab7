"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, and its
host-side validation rejects bad arguments before touching a GPU (no compute calls here)."""
import ctypes
import os
import re

import pytest

from wind_rwkv import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'wind_rwkv7.h')


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(wind_rwkv7_[a-z0-9_]+)\s*\(', text)))


def test_header_declares_something():
    syms = declared_symbols()
    assert 'wind_rwkv7_attn_forward' in syms and 'wind_rwkv7_attn_backward' in syms


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(_native.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(handle, s)]
    assert not missing, missing


def test_binding_table_covers_header():
    assert sorted(_native.SIGNATURES) == declared_symbols()


def test_version_and_constants():
    lib = _native.lib()
    assert lib.wind_rwkv7_abi_version() == 1
    assert lib.wind_rwkv7_chunk_len() == 16
    assert lib.wind_rwkv7_head_size_supported(64) == 1
    assert lib.wind_rwkv7_head_size_supported(32) == 0
    assert [c for c in range(8, 264, 8) if lib.wind_rwkv7_attn_head_size_supported(c)] == list(range(16, 129, 16))
    assert lib.wind_rwkv7_strerror(4) == b'T must be a multiple of the chunk length (16)'


def test_checkpoint_interval_switch():
    """16 or 32 tokens between kept states; the backward workspace of the one-launch path follows the setting."""
    lib = _native.lib()
    assert lib.wind_rwkv7_checkpoint_interval() == 32
    B, T, H, C = 8, 1024, 12, 64
    nchunks = B * H * T // 16
    try:
        assert lib.wind_rwkv7_set_checkpoint_interval(16) == 0 and lib.wind_rwkv7_checkpoint_interval() == 16
        assert lib.wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C) == nchunks * 20 * 512          # state + dab_u^T per chunk
        for bad in (0, 8, 24, 48, 64, -16):
            assert lib.wind_rwkv7_set_checkpoint_interval(bad) == 2 and lib.wind_rwkv7_checkpoint_interval() == 16
        assert lib.wind_rwkv7_set_checkpoint_interval(32) == 0
        assert lib.wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C) == (nchunks // 2) * 24 * 512   # state per pair, dab_u^T per chunk
    finally:
        lib.wind_rwkv7_set_checkpoint_interval(32)


def test_size_queries():
    lib = _native.lib()
    B, T, H, C = 8, 1024, 12, 64
    nchunks = B * H * T // 16
    # Blocks that prepare and scan in one launch keep, in either direction, a state (16 bf16 fragments of 512 B) per PAIR
    # of chunks and U^T (backward dab_u^T, 4 fragments) per chunk - with an odd number of chunks a state per chunk.
    kept = 20 * 512
    pair = 24 * 512
    # the saved tensor is sized per chunk by its callers, so it has one per-chunk size: that of the larger layout
    assert pair <= 2 * kept
    assert lib.wind_rwkv7_attn_saved_bytes(B, T, H, C) == nchunks * kept
    assert lib.wind_rwkv7_attn_saved_bytes(1, 48, 1, C) == 3 * kept
    assert lib.wind_rwkv7_attn_saved_bytes(1, 16384, 32, C) == 32 * 1024 * kept
    assert lib.wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C) == 256
    # (attn_ln: next to its other buffers - the gradient of the plain WKV7 output, [B,T,H,64] bf16, and per chunk 16
    # floats of bonus-dot gradients and 3 x 64 of parameter partials)
    assert lib.wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C) == (nchunks // 2) * pair
    assert lib.wind_rwkv7_attn_bwd_workspace_bytes(1, 48, 1, C) == 3 * kept    # three chunks: a state per chunk
    assert lib.wind_rwkv7_attn_ln_bwd_workspace_bytes(B, T, H, C) == (nchunks // 2) * pair + B * T * H * 64 * 2 + nchunks * (16 + 3 * 64) * 4
    # (attn_ln keeps the plain output as bf16 plus four fp32 block centres per token and head)
    assert lib.wind_rwkv7_attn_ln_saved_bytes(B, T, H, C) == nchunks * (kept + 16 * 64 * 2 + 16 * 4 * 4)
    # long sequences on few heads run as segments, which takes scratch: three 64x64 fp32 matrices
    # (the segment's affine map N, M and its entering state) per (batch, head, segment); 8 segments at this shape
    seg = 1 * 32 * 8 * 3 * 64 * 64 * 4
    assert lib.wind_rwkv7_attn_fwd_workspace_bytes(1, 16384, 32, C) == seg
    assert lib.wind_rwkv7_attn_bwd_workspace_bytes(1, 16384, 32, C) == 32 * 512 * pair + seg
    assert lib.wind_rwkv7_attn_saved_bytes(B, 1000, H, C) == 0   # T % 16 != 0
    assert lib.wind_rwkv7_attn_saved_bytes(B, T, H, 56) == 0     # head size: no multiple of 16
    assert lib.wind_rwkv7_attn_saved_bytes(B, T, H, 144) == 0    # above the largest
    # attn_ln at another head size: the plain saved tensor followed by the WKV7 output; the backward workspace holds
    # the plain one, the epilogue's records and four sequences
    # (the plain one, the kept WKV7 output and its centres: a float per token, head and block of 16 channels)
    assert lib.wind_rwkv7_attn_ln_saved_bytes(B, T, H, 128) == lib.wind_rwkv7_attn_saved_bytes(B, T, H, 128) + B * T * H * 128 * 2 + B * T * H * 8 * 4
    assert lib.wind_rwkv7_attn_ln_fwd_workspace_bytes(B, T, H, 128) == lib.wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, 128)
    assert lib.wind_rwkv7_attn_ln_bwd_workspace_bytes(B, T, H, 128) >= (
        lib.wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, 128) + lib.wind_rwkv7_ln_epilogue_bwd_workspace_bytes(B, T, H, 128)
        + 4 * B * T * H * 128 * 2)
    assert lib.wind_rwkv7_attn_ln_saved_bytes(B, T, H, 144) == 0
    # other head sizes (C = 16 NB): per chunk the forward keeps NB x NB state fragments and NB of U^T; the prepare
    # kernels' records (6 NB + 2 fragments forward, 5 NB backward, 16 NB floats of decay) are workspace
    for C2, NB in ((32, 2), (96, 6), (128, 8)):
        assert lib.wind_rwkv7_attn_saved_bytes(B, T, H, C2) == nchunks * (NB * NB + NB) * 512
        assert lib.wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C2) == nchunks * ((6 * NB + 2) * 512 + 64 * NB)
        assert lib.wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C2) == nchunks * (5 * NB * 512 + 64 * NB + (NB * NB + NB) * 512)


FWD_OK = dict(B=1, T=16, H=1, C=64, io=0, st=1)


def call_forward(ptr=0x1000, ws=0x1000, ws_bytes=1 << 20, **kw):
    a = dict(FWD_OK, **kw)
    return _native.lib().wind_rwkv7_attn_forward(a['B'], a['T'], a['H'], a['C'], a['io'], a['st'],
                                                 *([ptr] * 10), ws, ws_bytes, None)


@pytest.mark.parametrize('kw,code', [
    (dict(B=0), 2), (dict(T=-16), 2), (dict(C=40), 3), (dict(C=144), 3), (dict(T=24), 4), (dict(io=1), 5), (dict(st=7), 5),
    (dict(ptr=None), 1), (dict(ws=None), 6), (dict(ws_bytes=16), 6), (dict(ws=0x1001), 6),
    (dict(T=1 << 18, H=64), 2),    # a batch element's rows of one tensor reach 2 GiB (32-bit byte offsets inside one)
])
def test_forward_rejects_bad_arguments_on_host(kw, code):
    """Each call must return before anything is enqueued (the pointers are bogus)."""
    assert call_forward(**kw) == code


def test_prefill_rejects_bad_arguments_on_host():
    """The forward that keeps nothing for backward validates like the forward it shares its kernels with."""
    lib = _native.lib()
    ok = [1, 16, 1, 64, 0, 1] + [0x1000] * 10 + [0x1000, 1 << 20, None]
    ok_ln = [1, 16, 1, 64, 0, 1] + [0x1000] * 12 + [0x1000, 1 << 20, None]
    for fn, args in ((lib.wind_rwkv7_attn_prefill, ok), (lib.wind_rwkv7_attn_ln_prefill, ok_ln)):
        # (head sizes: multiples of 16 up to 128 for both)
        for idx, val, code in [(0, 0, 2), (3, 40, 3), (3, 144, 3),
                               (1, 24, 4), (4, 1, 5), (5, 7, 5), (6, None, 1),
                               (len(args) - 5, None, 1), (len(args) - 3, None, 6), (len(args) - 2, 16, 6)]:
            if code is None:
                continue
            bad = list(args)
            bad[idx] = val
            assert fn(*bad) == code, (fn.__name__, idx, val)


def test_f32_prefill_rejects_bad_arguments_on_host():
    lib = _native.lib()
    ok = [2, 32, 3, 64] + [0x1000] * 9 + [None]
    for idx, val, code in [(0, 0, 2), (1, 24, 4), (3, 144, 3), (3, 40, 3), (4, None, 1), (11, None, 1), (12, None, 1)]:
        bad = list(ok)
        bad[idx] = val
        assert lib.wind_rwkv7_attn_f32_prefill(*bad) == code, (idx, val)


def test_backward_rejects_bad_arguments_on_host():
    lib = _native.lib()
    args = [1, 16, 1, 64, 0, 1] + [0x1000] * 16 + [0x1000, 1 << 20, None]
    bad = list(args)
    bad[1] = 17
    assert lib.wind_rwkv7_attn_backward(*bad) == 4
    bad = list(args)
    bad[6 + 14] = None  # db (dsT and ds0 may be NULL - zero gradient of the final state, ds0 not wanted - the rest not)
    assert lib.wind_rwkv7_attn_backward(*bad) == 1
    bad = list(args)
    bad[6 + 7] = None   # s, the tensor saved by the forward
    assert lib.wind_rwkv7_attn_backward(*bad) == 1
    # NULL dsT / ds0 pass the argument checks: with a workspace that is too small the call gets as far as that check
    opt = list(args)
    opt[6 + 8] = None
    opt[6 + 15] = None
    opt[-2] = 0
    assert lib.wind_rwkv7_attn_backward(*opt) == 6
    bad = list(args)
    bad[-2] = 0
    assert lib.wind_rwkv7_attn_backward(*bad) == 6


def test_decode_rejects_bad_arguments_on_host():
    lib = _native.lib()
    ok = [2, 3, 64, 0, 1] + [0x1000] * 8 + [None]
    for idx, val, code in [(0, 0, 2), (1, -1, 2), (2, 40, 3), (2, 144, 3), (3, 1, 5), (4, 9, 5), (5, None, 1), (11, None, 1), (12, None, 1)]:
        bad = list(ok)
        bad[idx] = val
        assert lib.wind_rwkv7_attn_decode(*bad) == code, (idx, val)
    ok_ln = [2, 3, 64, 0, 1] + [0x1000] * 10 + [None]
    for idx, val, code in [(2, 136, 3), (11, None, 1), (12, None, 1), (14, None, 1)]:
        bad = list(ok_ln)
        bad[idx] = val
        assert lib.wind_rwkv7_attn_ln_decode(*bad) == code, (idx, val)


def test_mixer_decode_sizes_and_validation_on_host():
    lib = _native.lib()
    # 13 [Bp, C] bf16 buffers (rows padded to 16) + the LoRA first halves: [Bp,128], [Bp,64], 4 x [Bp,16], each 256-byte aligned
    assert lib.wind_rwkv7_mixer_decode_workspace_bytes(1, 768) == 13 * 16 * 768 * 2 + 16 * 128 * 2 + 16 * 64 * 2 + 4 * 16 * 16 * 2
    assert lib.wind_rwkv7_mixer_decode_workspace_bytes(17, 768) == 2 * lib.wind_rwkv7_mixer_decode_workspace_bytes(1, 768)
    assert lib.wind_rwkv7_mixer_decode_workspace_bytes(1, 100) == 0
    w = _native.MixerWeights(*[256] * len(_native.MIXER_WEIGHT_NAMES))
    ws = lib.wind_rwkv7_mixer_decode_workspace_bytes(1, 768)
    good = dict(B=1, C=768, H=12, sd=_native.F32, w=ctypes.byref(w), x=256, xp=512, st=256, y=256, xc=768, ws=256, wsb=ws, stream=None)
    call = lambda **kw: lib.wind_rwkv7_mixer_decode(*{**good, **kw}.values())
    assert call(B=0) == 2                                    # bad shape
    assert call(H=11) == 3                                   # head size (C must be 64 H)
    assert call(sd=7) == 5                                   # dtype
    assert call(x=None) == 1 and call(w=None) == 1           # null pointer
    assert call(xc=512) == 2                                 # the carried copy of x may not be x_prev itself
    assert call(wsb=ws - 1) == 6 and call(ws=257) == 6       # workspace too small / misaligned
    w.Wo = None
    assert call() == 1


def test_f32_entry_points_validate_on_host():
    lib = _native.lib()
    # the fp32 state every 16 tokens and one float per token and channel
    assert lib.wind_rwkv7_attn_f32_saved_bytes(8, 1024, 12, 64) == (8 * 12 * (1024 // 16) * 64 * 64 + 8 * 1024 * 12 * 64) * 4
    assert lib.wind_rwkv7_attn_f32_saved_bytes(8, 1000, 12, 64) == 0
    # head sizes 16 .. 128 in steps of 16
    assert [c for c in range(8, 264, 8) if lib.wind_rwkv7_f32_head_size_supported(c)] == list(range(16, 129, 16))
    assert lib.wind_rwkv7_attn_f32_saved_bytes(2, 64, 3, 32) == (2 * 3 * (64 // 16) * 32 * 32 + 2 * 64 * 3 * 32) * 4
    assert lib.wind_rwkv7_attn_f32_saved_bytes(2, 64, 3, 96) == (2 * 3 * (64 // 16) * 96 * 96 + 2 * 64 * 3 * 96) * 4
    assert lib.wind_rwkv7_attn_f32_saved_bytes(2, 64, 3, 128) == (2 * 3 * (64 // 16) * 128 * 128 + 2 * 64 * 3 * 128) * 4
    assert lib.wind_rwkv7_attn_f32_saved_bytes(2, 64, 3, 144) == 0
    ok = [2, 32, 3, 64] + [0x1000] * 10 + [None]
    for idx, val, code in [(0, 0, 2), (1, 24, 4), (3, 24, 3), (3, 256, 3), (4, None, 1), (10, None, 1), (13, None, 1)]:
        bad = list(ok)
        bad[idx] = val
        assert lib.wind_rwkv7_attn_f32_forward(*bad) == code, (idx, val)
    ok = [2, 32, 3, 64] + [0x1000] * 16 + [None]
    for idx, val, code in [(2, -1, 2), (1, 8, 4), (3, 136, 3), (10, None, 1), (12, None, 1), (19, None, 1)]:
        bad = list(ok)
        bad[idx] = val
        assert lib.wind_rwkv7_attn_f32_backward(*bad) == code, (idx, val)


def test_linear_wgrad_sizes_and_validation_on_host():
    lib = _native.lib()
    # C x C at 8192 tokens: 16 tiles of 192 x 192 times 16 token ranges = 256 blocks, each leaving a
    # 192 x 192 fp32 partial tile
    assert lib.wind_rwkv7_linear_wgrad_workspace_bytes(8192, 768, 768) == 256 * 192 * 192 * 4
    assert lib.wind_rwkv7_linear_wgrad_workspace_bytes(8192, 768, 128) == lib.wind_rwkv7_linear_wgrad_workspace_bytes(8192, 128, 768)
    assert lib.wind_rwkv7_linear_wgrad_workspace_bytes(8192, 760, 768) == 0      # O % 16 != 0
    assert lib.wind_rwkv7_linear_wgrad_workspace_bytes(0, 768, 768) == 0
    need = lib.wind_rwkv7_linear_wgrad_workspace_bytes(512, 64, 128)   # 256 x 64 tiles
    assert need > 0 and need % 256 == 0
    ok = [512, 64, 128, 0x1000, 64, 0x2000, 128, 0x3000, 1, 0x4000, need, None]
    cases = [(0, 0, 2), (1, 24, 9), (2, 100, 9), (3, None, 1), (5, None, 1), (7, None, 1), (8, 7, 5),
             (4, 60, 2), (4, 68, 2), (6, 120, 2), (3, 0x1008, 2), (9, None, 6), (10, need - 1, 6), (9, 0x4010, 6)]
    for idx, val, code in cases:
        bad = list(ok)
        bad[idx] = val
        assert lib.wind_rwkv7_linear_wgrad(*bad) == code, (idx, val)


def test_linear_wgrad_group_sizes_and_validation_on_host():
    """The grouped weight gradient: workspace of a known case, and every argument error before anything is enqueued."""
    import ctypes
    lib = _native.lib()
    ints = lambda *v: (ctypes.c_int * len(v))(*v)
    longs = lambda *v: (ctypes.c_longlong * len(v))(*v)
    ptrs = lambda *v: (ctypes.c_void_p * len(v))(*v)
    # three C x C problems at 8192 tokens: 48 tiles of 192 x 192 over 256 compute units = 5 token ranges each
    assert lib.wind_rwkv7_linear_wgrad_group_workspace_bytes(3, 8192, ints(768, 768, 768), ints(768, 768, 768)) == 48 * 5 * 192 * 192 * 4
    assert lib.wind_rwkv7_linear_wgrad_group_workspace_bytes(0, 8192, ints(768), ints(768)) == 0
    assert lib.wind_rwkv7_linear_wgrad_group_workspace_bytes(9, 8192, ints(*[64] * 9), ints(*[64] * 9)) == 0
    assert lib.wind_rwkv7_linear_wgrad_group_workspace_bytes(2, 8192, ints(768, 760), ints(768, 768)) == 0    # O % 16
    O, I = ints(768, 64), ints(128, 768)
    need = lib.wind_rwkv7_linear_wgrad_group_workspace_bytes(2, 512, O, I)
    assert need > 0 and need % 256 == 0

    def call(n=2, tokens=512, O=O, I=I, dy=ptrs(0x1000, 0x2000), ld_dy=longs(768, 64), x=ptrs(0x3000, 0x4000),
             ld_x=longs(128, 768), dW=ptrs(0x5000, 0x6000), out=1, ws=0x7000, ws_bytes=need):
        return lib.wind_rwkv7_linear_wgrad_group(n, tokens, O, I, dy, ld_dy, x, ld_x, dW, out, ws, ws_bytes, None)

    assert call(n=0) == 2 and call(n=9) == 2 and call(tokens=0) == 2
    assert call(O=None) == 1 and call(dy=None) == 1 and call(ld_x=None) == 1 and call(dW=None) == 1
    assert call(dy=ptrs(0x1000, None)) == 1 and call(dW=ptrs(None, 0x6000)) == 1
    assert call(O=ints(768, 72)) == 9                       # not a multiple of 16
    assert call(out=7) == 5
    assert call(ld_dy=longs(760, 64)) == 2 and call(ld_x=longs(128, 772)) == 2    # shorter than a row / no multiple of 8
    assert call(x=ptrs(0x3008, 0x4000)) == 2                # 16-byte alignment of the operands
    assert call(ws=None) == 6 and call(ws_bytes=need - 1) == 6 and call(ws=0x7010) == 6


def test_python_wrapper_raises_on_cpu_tensors():
    import torch
    from wind_rwkv.rwkv7 import attn
    x = torch.zeros(1, 16, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        attn(x, x, x, x, x, x, 64)


def test_profile_read_requires_enable():
    buf = (ctypes.c_float * 4)()
    assert _native.lib().wind_rwkv7_profile_read(0, buf, 4) < 0


def test_cast_to_bf16_validates_on_host():
    import ctypes
    lib = _native.lib()
    ptrs = (ctypes.c_void_p * 2)(0x1000, 0x2000)
    dts = (ctypes.c_int * 2)(_native.F32, _native.BF16)
    ns = (ctypes.c_longlong * 2)(16, 16)
    assert lib.wind_rwkv7_cast_to_bf16(0, None, None, None, None, None, None) == 0          # nothing to do
    assert lib.wind_rwkv7_cast_to_bf16(-1, ptrs, dts, ns, None, 0x3000, None) == 2
    assert lib.wind_rwkv7_cast_to_bf16(5000, ptrs, dts, ns, None, 0x3000, None) == 2
    assert lib.wind_rwkv7_cast_to_bf16(2, ptrs, dts, ns, None, None, None) == 1
    assert lib.wind_rwkv7_cast_to_bf16(2, None, dts, ns, None, 0x3000, None) == 1
    bad = (ctypes.c_int * 2)(_native.F32, 7)
    assert lib.wind_rwkv7_cast_to_bf16(2, ptrs, bad, ns, None, 0x3000, None) == 5
    neg = (ctypes.c_longlong * 2)(16, -1)
    assert lib.wind_rwkv7_cast_to_bf16(2, ptrs, dts, neg, None, 0x3000, None) == 2
    assert lib.wind_rwkv7_cast_to_bf16(2, ptrs, dts, ns, neg, 0x3000, None) == 2
    null = (ctypes.c_void_p * 2)(0x1000, None)
    assert lib.wind_rwkv7_cast_to_bf16(2, null, dts, ns, None, 0x3000, None) == 1


def test_copy_columns_validates_on_host():
    import ctypes
    lib = _native.lib()
    vp, ll, ci = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int
    def call(M=64, n=1, src=0x1000, sld=96, sc=64, dst=0x2000, dld=16, dc=0, w=16, op=0, aux=None):
        return lib.wind_rwkv7_copy_columns(M, n, (vp * 1)(src), (ll * 1)(sld), (ci * 1)(sc), (vp * 1)(dst), (ll * 1)(dld),
                                           (ci * 1)(dc), (ci * 1)(w), (ci * 1)(op), None if aux is None else (vp * 1)(aux), None)
    assert call(M=0) == 0 and call(n=0) == 0            # nothing to do
    assert call(M=-1) == 2 and call(n=300) == 2
    assert call(w=12) == 9 and call(w=0) == 9           # widths in 16-byte units
    assert call(op=3) == 2
    assert call(dst=None) == 1
    assert call(op=2) == 1                              # the derivative needs the tanh output
    assert call(sc=60) == 2 and call(sld=72) == 2       # column offset; slice past the row
    assert call(dld=8) == 2 and call(dst=0x2008) == 2


def test_operators_fail_loudly_without_the_library(monkeypatch, tmp_path):
    """No fallback: with the shared library absent every operator raises, naming the file and how to build it."""
    import torch
    from wind_rwkv.rwkv7 import attn, ddlerp
    monkeypatch.setattr(_native, '_lib', None)
    monkeypatch.setattr(_native, 'LIB_PATH', str(tmp_path / 'libwind_rwkv7.so'))
    with pytest.raises(ImportError, match='is missing: build it'):
        _native.lib()
    x = torch.zeros(1, 16, 64, dtype=torch.bfloat16)
    with pytest.raises((ImportError, RuntimeError)):
        attn(x, x, x, x, x, x, 64)
    with pytest.raises((ImportError, RuntimeError)):
        ddlerp(x, torch.zeros(64), torch.zeros(128, 64), torch.zeros(4, 64, 32), torch.zeros(4, 1, 1, 64))
