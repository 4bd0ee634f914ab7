"""The calling pattern of the reference's own scripts, run against this package.

tests/utils.py:18-56 (`grad_check`): parameters are cloned leaves, `f(*params, *aux)`, outputs normalised to a
tuple, `torch.autograd.backward(y, dy, retain_graph=True)`, gradients read from `.grad` (missing ones count as
zeros).  tests/test_time_mixer.py:62-85: the block is called through `torch.func.functional_call` with every
parameter replaced by such a clone, redrawn N(0, 0.1^2), and a float32 input.  The modules are imported under
the reference's paths (wind_rwkv/rwkv7/rwkv7_attn_ln.py, time_mixer.py, ...).
"""
from collections import namedtuple

import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _protocol(f, params, aux=()):
    params = [p.clone().requires_grad_() for p in params]
    y = f(*params, *aux)
    if type(y) != tuple:
        y = (y,)
    gen = torch.Generator(device=DEV).manual_seed(3)
    dy = tuple(torch.randn(o.shape, generator=gen, device=DEV).to(o.dtype) for o in y)
    torch.autograd.backward(y, dy, retain_graph=True)
    grads = [torch.zeros_like(p) if p.grad is None else p.grad.clone() for p in params]
    return y, dy, grads


def test_operators_through_the_reference_module_paths():
    from wind_rwkv.rwkv7.rwkv7_attn import attn, load_attn
    from wind_rwkv.rwkv7.rwkv7_attn_ln import attn_ln, load_attn_ln
    from wind_rwkv.rwkv7.rwkv7_ddlerp import ddlerp
    from wind_rwkv.rwkv7.rwkv7_expand_loras import expand_loras
    B, T, H, C = 2, 64, 12, 64
    load_attn(C)
    load_attn_ln(C)
    d = inputs.attn_ln_inputs(B, T, H, C, 31, dtype=torch.bfloat16)
    seqs = [d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab']
    # attn: y and the six gradients against the fp64 recurrence on the same upstream gradient
    y, dy, grads = _protocol(attn, seqs, aux=(C,))
    ref_in = [d[n].double().requires_grad_() for n in 'qwkvab']
    y_ref, _ = seq_ref.wkv7_seq(*ref_in)
    y_ref.backward(dy[0].view(B, T, H, C).double().cpu())
    assert seq_ref.rel_err(y[0].detach().view(B, T, H, C).float().cpu(), y_ref.detach()) <= 1e-2
    for g, r in zip(grads, ref_in):
        assert seq_ref.rel_err(g.view(B, T, H, C).float().cpu(), r.grad) <= 1e-2
    # attn_ln, ddlerp, expand_loras: the protocol runs, outputs are tuples where the reference's are, every
    # parameter receives a finite gradient of its own dtype
    y, _, grads = _protocol(attn_ln, seqs + [d['g'].reshape(B, T, H * C).to(DEV), d['params'].to(DEV)], aux=(C,))
    assert len(y) == 1 and grads[-1].dtype == torch.float32 and all(torch.isfinite(g).all() for g in grads)
    dd = inputs.ddlerp_inputs(B, T, 768, 32, 6, dtype=torch.bfloat16)
    y, _, grads = _protocol(ddlerp, [dd[n].to(DEV) for n in ('x', 'alpha', 'L', 'R', 'beta')])
    assert len(y) == 4 and all(torch.isfinite(g).all() and g.abs().sum() > 0 for g in grads)
    el = inputs.expand_loras_inputs(B, T, 768, 16, 7, dtype=torch.bfloat16)
    names = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']
    y, _, grads = _protocol(expand_loras, [el[n].to(DEV) for n in names], aux=(64,))
    assert len(y) == 4 and all(torch.isfinite(g).all() and g.abs().sum() > 0 for g in grads)


def test_block_through_functional_call():
    """tests/test_time_mixer.py:62-85: module built with the reference's keyword flags, parameters swapped in with
    torch.func.functional_call, float32 input.  Gradients must reach the swapped-in tensors and equal those of
    the module called with the same values as its own parameters."""
    from wind_rwkv.rwkv7.time_mixer import TimeMixer
    Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
    model = TimeMixer(Config(12, 12, 768), 6, use_triton_ddlerp=True, use_triton_loras=True, attn_impl='cuda').to(DEV)
    keys = list(dict(model.named_parameters()).keys())
    gen = torch.Generator(device=DEV).manual_seed(9)
    values = [torch.randn(p.shape, generator=gen, device=DEV) * 0.1 for p in model.parameters()]
    x = torch.randn(2, 64, 768, generator=gen, device=DEV)

    def f(*args):
        return torch.func.functional_call(model, dict(zip(keys, args[:-1])), (args[-1],))

    y, dy, grads = _protocol(f, values + [x])
    assert y[0].dtype == torch.bfloat16 and all(torch.isfinite(g).all() for g in grads)
    assert all(g.abs().sum() > 0 for g in grads), 'a swapped-in parameter received no gradient'
    with torch.no_grad():
        for p, v in zip(model.parameters(), values):
            p.copy_(v)
    xl = x.clone().requires_grad_()
    y2 = model(xl)
    y2.backward(dy[0])
    assert torch.equal(y2, y[0]) and torch.equal(xl.grad, grads[-1])
    for p, g in zip(model.parameters(), grads[:-1]):
        assert torch.equal(p.grad, g)
