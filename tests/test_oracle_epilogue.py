"""Pins oracle/seq_ref.py:attn_ln_epilogue against torch's library group_norm and special cases."""
import torch

from oracle import inputs, seq_ref

F = torch.nn.functional
D = torch.float64


def data(B=2, T=6, H=3, C=8, seed=1):
    d = inputs.attn_ln_inputs(B, T, H, C, seed)
    y = torch.randn(B, T, H, C, generator=torch.Generator().manual_seed(seed + 5), dtype=D)
    return {k: (v.to(D) if torch.is_tensor(v) else v) for k, v in d.items()}, y


def test_against_library_group_norm_and_closed_form():
    d, y = data()
    B, T, H, C = y.shape
    out = seq_ref.attn_ln_epilogue(y, d['q'], d['k'], d['v'], d['g'], d['params'])
    gn = F.group_norm(y.reshape(B * T, H * C), H, d['params'][0], d['params'][1], eps=64e-5).view(B, T, H, C)
    bonus = (d['q'] * d['k'] * d['params'][2].view(H, C)).sum(-1, keepdim=True) * d['v']
    assert torch.allclose(out, (gn + bonus) * d['g'], atol=1e-12)


def test_identity_parameters_reduce_to_plain_group_norm():
    d, y = data(seed=2)
    B, T, H, C = y.shape
    params = torch.stack([torch.ones(H * C, dtype=D), torch.zeros(H * C, dtype=D), torch.zeros(H * C, dtype=D)])
    out = seq_ref.attn_ln_epilogue(y, d['q'], d['k'], d['v'], torch.ones_like(y), params)
    gn = F.group_norm(y.reshape(B * T, H * C), H, eps=64e-5).view(B, T, H, C)
    assert torch.allclose(out, gn, atol=1e-12)
    # biased variance: each normalised head has mean 0 and second moment var/(var+eps) < 1
    assert torch.allclose(out.mean(-1), torch.zeros(B, T, H, dtype=D), atol=1e-12)
    var = y.var(-1, unbiased=False)
    assert torch.allclose((out ** 2).mean(-1), var / (var + 64e-5), atol=1e-12)


def test_bonus_term_only():
    """ln_w = ln_b = 0 leaves exactly (sum_c q k bonus) * v * g."""
    d, y = data(seed=3)
    B, T, H, C = y.shape
    params = d['params'].clone()
    params[0] = 0
    params[1] = 0
    out = seq_ref.attn_ln_epilogue(y, d['q'], d['k'], d['v'], d['g'], params)
    exp = torch.einsum('bthc,bthc,hc->bth', d['q'], d['k'], params[2].view(H, C))[..., None] * d['v'] * d['g']
    assert torch.allclose(out, exp, atol=1e-12)


def test_epilogue_gradcheck():
    d, y = data(B=1, T=2, H=2, C=4, seed=4)
    xs = [t.clone().requires_grad_() for t in (y, d['q'], d['k'], d['v'], d['g'], d['params'])]
    assert torch.autograd.gradcheck(seq_ref.attn_ln_epilogue, xs, eps=1e-6, atol=1e-6)
