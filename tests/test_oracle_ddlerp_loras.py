"""Pins oracle/seq_ref.py:ddlerp_seq and expand_loras_seq (the reference holds no vectors for them):
explicit per-token loops, special cases that collapse the formulas, library routines, invariants."""
import torch

from oracle import inputs, seq_ref

F = torch.nn.functional
D64 = torch.float64


def dd(B=2, T=5, C=8, D=4, seed=1):
    d = inputs.ddlerp_inputs(B, T, C, D, seed)
    return {k: (v.to(D64) if torch.is_tensor(v) else [t.to(D64) for t in v]) for k, v in d.items()}


def test_ddlerp_explicit_token_loop():
    d = dd()
    y = seq_ref.ddlerp_seq(d['x'], d['alpha'], d['L'], d['R'], d['beta'])
    B, T, C = d['x'].shape
    Dr = d['R'].shape[2]
    for b in range(B):
        for t in range(T):
            x = d['x'][b, t]
            prev = d['x'][b, t - 1] if t > 0 else torch.zeros(C, dtype=D64)
            xx = prev - x
            mid = torch.tanh(d['L'] @ (x + xx * d['alpha']))
            for k in range(4):
                c = d['R'][k] @ mid[k * Dr:(k + 1) * Dr] + d['beta'][k, 0, 0]
                assert torch.allclose(y[k, b, t], x + xx * c, atol=1e-12)


def test_ddlerp_zero_lora_gives_plain_lerp():
    """R = 0 or L = 0: y_k = x + xx*beta_k (tanh(0) = 0)."""
    d = dd(seed=2)
    xx = seq_ref.token_shift(d['x']) - d['x']
    exp = d['x'][None] + xx[None] * d['beta']
    assert torch.allclose(seq_ref.ddlerp_seq(d['x'], d['alpha'], d['L'], torch.zeros_like(d['R']), d['beta']), exp)
    assert torch.allclose(seq_ref.ddlerp_seq(d['x'], d['alpha'], torch.zeros_like(d['L']), d['R'], d['beta']), exp)


def test_ddlerp_first_token_and_batch_independence():
    """At t = 0 the shifted row is zero (xx = -x) for every batch element, not the previous batch's last row."""
    d = dd(seed=3)
    y = seq_ref.ddlerp_seq(d['x'], d['alpha'], d['L'], d['R'], d['beta'])
    y1 = seq_ref.ddlerp_seq(d['x'][1:], d['alpha'], d['L'], d['R'], d['beta'])
    assert torch.allclose(y[:, 1:], y1, atol=1e-13)
    # beta = 1, no LoRA: y = x + (0 - x)*1 = 0 at t = 0
    y0 = seq_ref.ddlerp_seq(d['x'], d['alpha'], d['L'], torch.zeros_like(d['R']), torch.ones_like(d['beta']))
    assert torch.allclose(y0[:, :, 0], torch.zeros_like(y0[:, :, 0]), atol=1e-13)


def test_ddlerp_gradcheck():
    d = dd(B=1, T=3, C=4, D=2, seed=4)
    xs = [d[n].clone().requires_grad_() for n in ('x', 'alpha', 'L', 'R', 'beta')]
    assert torch.autograd.gradcheck(seq_ref.ddlerp_seq, xs, eps=1e-6, atol=1e-6)


def el(B=2, T=4, C=16, D=4, seed=1):
    d = inputs.expand_loras_inputs(B, T, C, D, seed)
    return {k: (v.to(D64) if torch.is_tensor(v) else [t.to(D64) for t in v]) for k, v in d.items()}


NAMES = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']


def test_expand_loras_invariants():
    d = el()
    H = 8
    w, k, kk, b = seq_ref.expand_loras_seq(*[d[n] for n in NAMES], H)
    B, T, C = w.shape
    # kk is unit-norm per head; b = -kk*a with a = sigmoid(...) in (0,1)
    assert torch.allclose(kk.view(B, T, C // H, H).norm(dim=-1), torch.ones(B, T, C // H, dtype=D64), atol=1e-12)
    a = torch.sigmoid(d['a_bias'] + d['a_in'] @ d['Wa'].t())
    assert torch.allclose(b, -kk * a, atol=1e-13)
    # w = -softplus(-(bias+w_in)) - 0.5 <= -0.5, and equals log(sigmoid(.)) - 0.5
    assert (w <= -0.5).all()
    assert torch.allclose(w, F.logsigmoid(d['w_bias'] + d['w_in']) - 0.5, atol=1e-12)
    # library normalize agrees
    z = d['k_in'] + torch.tanh(d['z_in']) @ d['Wz'].t()
    assert torch.allclose(kk, F.normalize(z.view(B, T, C // H, H), dim=-1).view(B, T, C), atol=1e-12)


def test_expand_loras_zero_lora_inputs():
    """Zero LoRA activations: a, ma, mk reduce to sigmoid(bias); k_out = k_in*(ma + a - ma*a)*exp(w*mk)."""
    d = el(seed=2)
    for n in ('z_in', 'a_in', 'ma_in', 'mk_in'):
        d[n] = torch.zeros_like(d[n])
    w, k, kk, b = seq_ref.expand_loras_seq(*[d[n] for n in NAMES], 8)
    a, ma, mk = (torch.sigmoid(d[n]) for n in ('a_bias', 'ma_bias', 'mk_bias'))
    assert torch.allclose(k, d['k_in'] * (ma + a - ma * a) * torch.exp(w * mk), atol=1e-12)
    B, T, C = w.shape
    assert torch.allclose(kk, F.normalize(d['k_in'].view(B, T, C // 8, 8), dim=-1).view(B, T, C), atol=1e-12)


def test_expand_loras_gradcheck():
    d = el(B=1, T=2, C=8, D=2, seed=3)
    xs = [d[n].clone().requires_grad_() for n in NAMES]
    assert torch.autograd.gradcheck(lambda *z: seq_ref.expand_loras_seq(*z, 4), xs, eps=1e-6, atol=1e-6)
