"""Writes the golden vectors under tests/golden/ from the fp64 oracle.

The reference holds no fixtures of its own (its scripts draw unseeded data and compare two live
implementations, tests/test_attn.py:34-48), so these are this repository's: small seeded cases per operator -
inputs rounded to bf16 and stored as their bit patterns, expected outputs and gradients from the fp64 oracle
stored as float32.  They anchor two things that live code cannot: the oracle itself (tests/test_golden.py
recomputes them, so a later edit of oracle/ that changes a result fails), and the HIP path against numbers that
no run of today's code can move (tests/test_gpu_golden.py).

    python tests/golden/make_fixtures.py        # from the repository root; overwrites the .npz files
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import inputs, seq_ref  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
LORA_NAMES = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']


def bits(t):
    """bf16 tensor -> uint16 bit patterns"""
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def f32(t):
    return t.detach().to(torch.float32).numpy()


def wkv7_case(with_ln):
    B, T, H, C = 1, 32, 2, 64
    d = inputs.attn_ln_inputs(B, T, H, C, seed=2024, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(2025)
    s0 = 0.3 * torch.randn(B, H, C, C, generator=gen)
    dsT = torch.randn(B, H, C, C, generator=gen)
    names = list('qwkvab') + (['g'] if with_ln else [])
    leaves = [d[n].double().requires_grad_() for n in names]
    s64 = s0.double().requires_grad_()
    out = {'in_' + n: bits(d[n]) for n in names}
    out.update(in_s0=f32(s0), in_dy=bits(d['dy']), in_dsT=f32(dsT))
    if with_ln:
        p64 = d['params'].double().requires_grad_()
        y, sT = seq_ref.attn_ln_seq(*leaves, p64, s64)
        out['in_params'] = f32(d['params'])
    else:
        y, sT = seq_ref.wkv7_seq(*leaves, s64)
    torch.autograd.backward([y, sT], [d['dy'].double(), dsT.double()])
    out.update(y=f32(y), sT=f32(sT), ds0=f32(s64.grad))
    for n, x in zip(names, leaves):
        out['d' + n] = f32(x.grad)
    if with_ln:
        out['dparams'] = f32(p64.grad)
    return out


def ddlerp_case():
    B, T, C, D = 1, 32, 64, 32
    d = inputs.ddlerp_inputs(B, T, C, D, seed=2026, dtype=torch.bfloat16)
    pn = ('alpha', 'L', 'R', 'beta')
    pr = {n: d[n].bfloat16() for n in pn}
    x = d['x'].double().requires_grad_()
    p = {n: pr[n].double().requires_grad_() for n in pn}
    y = seq_ref.ddlerp_seq(x, p['alpha'], p['L'], p['R'], p['beta'])
    g = torch.autograd.grad(y, [x] + [p[n] for n in pn], torch.stack([t.double() for t in d['dy']]))
    out = {'in_x': bits(d['x']), 'in_dy': np.stack([bits(t) for t in d['dy']]), 'y': f32(y), 'dx': f32(g[0])}
    for i, n in enumerate(pn):
        out['in_' + n] = bits(pr[n])
        out['d' + n] = f32(g[1 + i])
    return out


def expand_loras_case():
    B, T, C, D = 1, 32, 64, 16
    d = inputs.expand_loras_inputs(B, T, C, D, seed=2027, dtype=torch.bfloat16)
    for n in LORA_NAMES[2:10]:
        d[n] = (d[n].float() * 0.5).bfloat16()
    xs = [d[n].double().requires_grad_() for n in LORA_NAMES]
    ys = seq_ref.expand_loras_seq(*xs, 64)
    gs = torch.autograd.grad(ys, xs, [t.double() for t in d['dy']])
    out = {'in_' + n: bits(d[n]) for n in LORA_NAMES}
    out['in_dy'] = np.stack([bits(t) for t in d['dy']])
    for n, y in zip(['w', 'k', 'kk', 'b'], ys):
        out[n] = f32(y)
    for n, g in zip(LORA_NAMES, gs):
        out['d' + n] = f32(g)
    return out


CASES = {'wkv7_b1_t32_h2.npz': lambda: wkv7_case(False), 'attn_ln_b1_t32_h2.npz': lambda: wkv7_case(True),
         'ddlerp_t32_c64_d32.npz': ddlerp_case, 'expand_loras_t32_c64_d16.npz': expand_loras_case}

if __name__ == '__main__':
    for name, make in CASES.items():
        arrays = make()
        np.savez(os.path.join(HERE, name), **arrays)
        print(name, sum(a.nbytes for a in arrays.values()) // 1024, 'KiB')
