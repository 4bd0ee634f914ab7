"""The whole TimeMixer block at the benchmark configuration as it is stated: B=8, T=1024, d=768, 12 heads of 64, bf16;
x ~ N(0,1); token-shift mix parameters ~ U(0,1); every LoRA weight ~ 0.02 N(0,1); Wr, Wk, Wv, Wo ~ N(0, 1/768); the
remaining vectors (decay and gate biases, bonus, GroupNorm) as TimeMixer's own deterministic initialisation; upstream
gradient ~ N(0,1); seed 4.

Oracle: the fp64 block (oracle/seq_ref.py:time_mixer_seq, following tests/test_time_mixer.py:26-55) that rounds to bf16
exactly where the pipeline's interfaces round, with the C restatement of the recurrence so that the full size fits.
Metric and protocol: tests/utils.py:18-56 (normalised L2 error of the output and of the gradient of x and of every
parameter, gate 1e-2).
"""
from collections import namedtuple

import pytest
import torch

from oracle import seq_ref

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = 1e-2
Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
B, T, C, H = 8, 1024, 768, 12
MIX = ('time_maa_x', 'time_maa')
PROJ = ('Wr', 'Wk', 'Wv', 'Wo')


def build(seed=4):
    from wind_rwkv.rwkv7 import TimeMixer
    gen = torch.Generator().manual_seed(seed)
    model = TimeMixer(Config(12, H, C), 6)
    with torch.no_grad():
        for n, p in model.named_parameters():
            if n in MIX:
                p.copy_(torch.rand(p.shape, generator=gen))
            elif n in PROJ:
                p.copy_(torch.randn(p.shape, generator=gen) * C ** -0.5)
            elif n.endswith('_w1') or n.endswith('_w2'):
                p.copy_(torch.randn(p.shape, generator=gen) * 0.02)
    x = torch.randn(B, T, C, generator=gen).bfloat16()
    dy = torch.randn(B, T, C, generator=gen).bfloat16()
    return model, x, dy


def test_block_parity_at_the_benchmark_configuration(c_oracle):
    model, x, dy = build()
    names = [n for n, _ in model.named_parameters()]
    po = {n: p.detach().double().requires_grad_() for n, p in model.named_parameters()}
    xo = x.double().requires_grad_()
    yo = seq_ref.time_mixer_seq(po, xo, H, stage=seq_ref.bf16_boundary, weight=seq_ref.bf16_ste, wkv7=c_oracle.wkv7)
    go = torch.autograd.grad(yo, [xo] + [po[n] for n in names], dy.double())
    model = model.to(DEV)
    xd = x.to(DEV).requires_grad_()
    yd = model(xd)
    yd.backward(dy.to(DEV))
    torch.cuda.synchronize()
    errs = {'y': seq_ref.rel_err(yd.detach().float().cpu(), yo.detach()), 'dx': seq_ref.rel_err(xd.grad.float().cpu(), go[0])}
    for i, (n, p) in enumerate(model.named_parameters()):
        errs['d' + n] = seq_ref.rel_err(p.grad.float().cpu(), go[1 + i])
    print('cfg4 block errors vs stage-rounded oracle:', {k: f'{v:.2e}' for k, v in errs.items()})
    bad = {k: e for k, e in errs.items() if not e <= TOL}
    assert not bad, f'over {TOL}: {bad}'
