"""CPU-side checks of the TimeMixer module: parameter names and shapes (state-dict compatibility with the
reference, time_mixer.py:42-104), the closed-form initial values, and the wiring of the block, which is
run through its plain-PyTorch switches in fp64 and compared with the oracle's composition of the spec
functions (oracle/seq_ref.py:time_mixer_seq)."""
from collections import namedtuple

import torch

from oracle import seq_ref
from wind_rwkv.rwkv7 import TimeMixer

Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])

EXPECTED = {  # name -> shape at C = 768 (time_mixer.py:42-104)
    'time_maa_x': (768,), 'time_maa': (4, 1, 1, 768), 'time_decay': (768,), 'time_faaaa': (768,),
    'time_aaaaa': (768,), 'time_maa_w1': (128, 768), 'time_maa_w2': (4, 768, 32), 'time_decay_w1': (64, 768),
    'time_decay_w2': (768, 64), 'time_aaa_w1': (16, 768), 'time_aaa_w2': (768, 16), 'time_kkk_w1': (16, 768),
    'time_kkk_w2': (768, 16), 'gate_w1': (128, 768), 'gate_w2': (768, 128), 'ma_w1': (16, 768), 'ma_w2': (768, 16),
    'time_misc_a': (768,), 'mk_w1': (16, 768), 'mk_w2': (768, 16), 'time_misc_k': (768,), 'Wr': (768, 768),
    'Wk': (768, 768), 'Wv': (768, 768), 'Wo': (768, 768), 'ln_x.weight': (768,), 'ln_x.bias': (768,),
}


def make(C=768, H=12, layer=6, **kw):
    return TimeMixer(Config(12, H, C), layer, **kw)


def test_parameter_names_and_shapes():
    m = make(use_triton_ddlerp=False, use_triton_loras=False, attn_impl='ref')
    got = {n: tuple(p.shape) for n, p in m.named_parameters()}
    assert got == EXPECTED


def test_closed_form_initial_values():
    C, layer, n_layer = 768, 6, 12
    m = make(C=C, layer=layer, use_triton_ddlerp=False, use_triton_loras=False, attn_impl='ref')
    r0 = layer / (n_layer - 1)
    r1 = 1 - layer / n_layer
    ddd = torch.arange(C) / C
    assert torch.allclose(m.time_maa_x, 1 - ddd ** (0.6 * r1 ** 0.9))
    assert torch.allclose(m.time_maa[2, 0, 0], 1 - (ddd ** (0.9 * r1) + 0.4 * r0))
    assert torch.allclose(m.time_maa[3, 0, 0], 1 - (ddd ** (0.4 * r1) + 0.6 * r0))
    n = torch.arange(C, dtype=torch.float32)
    assert torch.allclose(m.time_decay, -7 + 5 * (n / (C - 1)) ** (0.85 + r0 ** 0.5) + 0.5, atol=1e-6)
    assert float(m.Wo.abs().max()) == 0.0 and float(m.time_maa_w1.abs().max()) == 0.0
    # orthogonal second halves: columns of the [rank, C] factor are orthonormal up to the 0.1 scale
    w = m.time_decay_w2.detach()          # [C, 64]
    assert torch.allclose(w.T @ w, 0.01 * torch.eye(64), atol=1e-5)
    g = m.gate_w1.detach()                # [128, C]
    assert torch.allclose(g @ g.T, 0.01 * torch.eye(128), atol=1e-5)
    bound = 0.5 / 768 ** 0.5
    assert float(m.Wr.abs().max()) <= bound and float(m.Wr.abs().max()) > 0.9 * bound


def test_wiring_matches_oracle_composition():
    torch.manual_seed(0)
    C, H, B, T = 128, 2, 2, 12
    m = make(C=C, H=H, layer=3, use_triton_ddlerp=False, use_triton_loras=False, attn_impl='ref').double()
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(std=0.1)            # as the reference's block test does (tests/test_time_mixer.py:75)
    x = torch.randn(B, T, C, dtype=torch.float64)
    params = {n: p.detach() for n, p in m.named_parameters()}
    ref = seq_ref.time_mixer_seq(params, x, H)
    out = m(x)
    assert out.dtype == torch.float64
    assert seq_ref.rel_err(out.detach(), ref) < 1e-12


def test_block_oracle_with_the_c_recurrence_matches_autograd_over_the_token_loop(c_oracle):
    """The full-size block parity test runs the block oracle with the C restatement of the recurrence (hand-derived
    adjoint) in place of autograd over the Python token loop: same output and same gradients."""
    torch.manual_seed(1)
    C, H, B, T = 128, 2, 2, 24
    m = make(C=C, H=H, layer=3, use_triton_ddlerp=False, use_triton_loras=False, attn_impl='ref').double()
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(std=0.1)
    x = torch.randn(B, T, C, dtype=torch.float64)
    dy = torch.randn(B, T, C, dtype=torch.float64)
    grads = []
    for wkv7 in (None, c_oracle.wkv7):
        params = {n: p.detach().clone().requires_grad_() for n, p in m.named_parameters()}
        xi = x.clone().requires_grad_()
        y = seq_ref.time_mixer_seq(params, xi, H, stage=seq_ref.bf16_boundary, weight=seq_ref.bf16_ste, wkv7=wkv7)
        grads.append([y.detach()] + list(torch.autograd.grad(y, [xi] + list(params.values()), dy)))
    for a, b in zip(*grads):
        assert seq_ref.rel_err(b, a) < 1e-10


def test_decode_cache_survives_copy_and_pickle():
    """The working copies `step` keeps (bf16 parameters, per-batch workspaces) are tensors only and are left out of
    pickling and deep copies; a copy remakes its own; `invalidate_decode_cache` drops them after a write through
    `p.data`, which the cache key (storage address, version counter) cannot see."""
    import copy
    import io
    import pickle

    m = make(C=128, H=2, use_triton_ddlerp=False, use_triton_loras=False, attn_impl='ref')
    cache = m._decode_weights()
    assert m._decode_weights() is cache                       # unchanged parameters: the same copies
    assert all(isinstance(t, torch.Tensor) for t in cache[1]) and isinstance(cache[2], torch.Tensor)
    m2 = copy.deepcopy(m)
    assert '_decode_cache' not in m2.__dict__ and '_decode_cache' in m.__dict__
    m3 = pickle.loads(pickle.dumps(m))
    assert '_decode_cache' not in m3.__dict__
    buf = io.BytesIO()
    torch.save(m, buf)
    assert torch.equal(m2._decode_weights()[1][4], cache[1][4])   # Wr as bf16, remade by the copy
    with torch.no_grad():
        m.Wr.mul_(2.0)                                        # an in-place write bumps the version: remade
    assert m._decode_weights() is not cache
    cache = m._decode_weights()
    m.Wr.data.mul_(0.5)                                       # invisible to the key ...
    assert m._decode_weights() is cache
    m.invalidate_decode_cache()                               # ... so the caller says so
    assert torch.equal(m._decode_weights()[1][4], m.Wr.detach().bfloat16())
