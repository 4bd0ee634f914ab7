"""The HIP path against the committed golden vectors (tests/golden/*.npz, written once from the fp64 oracle by
tests/golden/make_fixtures.py): outputs, final state and every gradient within the 1e-2 gate for bf16 I/O."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = 1e-2
HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def _bf(z, key):
    return torch.from_numpy(z[key].view(np.int16).copy()).view(torch.bfloat16)


def _err(got, ref):
    ref = torch.from_numpy(np.asarray(ref)).double()
    return float((got.detach().double().cpu().reshape(ref.shape) - ref).norm() / max(float(ref.norm()), 1e-30))


@pytest.mark.parametrize('with_ln', [False, True])
def test_wkv7_and_attn_ln(with_ln):
    from wind_rwkv.rwkv7 import WindRWKV7, WindRWKV7LN
    z = np.load(os.path.join(HERE, 'attn_ln_b1_t32_h2.npz' if with_ln else 'wkv7_b1_t32_h2.npz'))
    names = list('wqkvab') + (['g'] if with_ln else [])
    xs = [_bf(z, 'in_' + n).to(DEV).requires_grad_() for n in names]
    s0 = torch.from_numpy(z['in_s0']).to(DEV).requires_grad_()
    if with_ln:
        params = torch.from_numpy(z['in_params']).to(DEV).requires_grad_()
        y, sT, _ = WindRWKV7LN.apply(*xs, params, s0)
    else:
        y, sT, _ = WindRWKV7.apply(*xs, s0)
    torch.autograd.backward([y, sT], [_bf(z, 'in_dy').to(DEV), torch.from_numpy(z['in_dsT']).to(DEV)])
    errs = {'y': _err(y, z['y']), 'sT': _err(sT, z['sT']), 'ds0': _err(s0.grad, z['ds0'])}
    errs.update({'d' + n: _err(x.grad, z['d' + n]) for n, x in zip(names, xs)})
    if with_ln:
        errs['dparams'] = _err(params.grad, z['dparams'])
    assert all(e <= TOL for e in errs.values()), errs


def test_ddlerp():
    from wind_rwkv.rwkv7 import ddlerp
    z = np.load(os.path.join(HERE, 'ddlerp_t32_c64_d32.npz'))
    pn = ('alpha', 'L', 'R', 'beta')
    x = _bf(z, 'in_x').to(DEV).requires_grad_()
    ps = [_bf(z, 'in_' + n).float().to(DEV).requires_grad_() for n in pn]
    ys = ddlerp(x, *ps)
    dy = torch.from_numpy(z['in_dy'].view(np.int16).copy()).view(torch.bfloat16).to(DEV)
    torch.autograd.backward(list(ys), list(dy.unbind(0)))
    errs = {'y': _err(torch.stack(ys), z['y']), 'dx': _err(x.grad, z['dx'])}
    errs.update({'d' + n: _err(p.grad, z['d' + n]) for n, p in zip(pn, ps)})
    assert all(e <= TOL for e in errs.values()), errs


def test_expand_loras():
    from wind_rwkv.rwkv7 import expand_loras
    names = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']
    z = np.load(os.path.join(HERE, 'expand_loras_t32_c64_d16.npz'))
    xs = [(_bf(z, 'in_' + n).float() if i >= 6 else _bf(z, 'in_' + n)).to(DEV).requires_grad_() for i, n in enumerate(names)]
    ys = expand_loras(*xs, 64)
    dy = torch.from_numpy(z['in_dy'].view(np.int16).copy()).view(torch.bfloat16).to(DEV)
    torch.autograd.backward(list(ys), list(dy.unbind(0)))
    errs = {n: _err(y, z[n]) for n, y in zip(['w', 'k', 'kk', 'b'], ys)}
    errs.update({'d' + n: _err(x.grad, z['d' + n]) for n, x in zip(names, xs)})
    assert all(e <= TOL for e in errs.values()), errs
