"""GPU parity of ddlerp against the fp64 oracle (forward: four streams; backward: dx and the four
parameter gradients).  Gate 1e-2 as in the reference's script (tests/test_ddlerp.py:40, tests/utils.py:18);
the oracle sees the same bf16-rounded x and parameters the kernels see."""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
TOL = 1e-2
DEV = 'cuda'
PNAMES = ('alpha', 'L', 'R', 'beta')


def run_both(B, T, C, D, seed):
    from wind_rwkv.rwkv7 import ddlerp
    d = inputs.ddlerp_inputs(B, T, C, D, seed, dtype=torch.bfloat16)
    pr = {n: d[n].bfloat16() for n in PNAMES}                       # what the kernels see
    # oracle
    xo = d['x'].double().requires_grad_()
    po = {n: pr[n].double().requires_grad_() for n in PNAMES}
    yo = seq_ref.ddlerp_seq(xo, po['alpha'], po['L'], po['R'], po['beta'])
    dyo = torch.stack([g.double() for g in d['dy']])
    go = torch.autograd.grad(yo, [xo] + [po[n] for n in PNAMES], dyo)
    # device (fp32 parameters, as the module holds them)
    xd = d['x'].to(DEV).requires_grad_()
    pd = {n: pr[n].float().to(DEV).requires_grad_() for n in PNAMES}
    ys = ddlerp(xd, pd['alpha'], pd['L'], pd['R'], pd['beta'])
    torch.autograd.backward(list(ys), [g.to(DEV) for g in d['dy']])
    torch.cuda.synchronize()
    got = {'y': torch.stack([y.detach().float().cpu() for y in ys]), 'dx': xd.grad.float().cpu()}
    ref = {'y': yo.detach(), 'dx': go[0]}
    for i, n in enumerate(PNAMES):
        got['d' + n] = pd[n].grad.float().cpu()
        ref['d' + n] = go[1 + i]
    return got, ref


def check(got, ref):
    errs = {k: seq_ref.rel_err(got[k], ref[k]) for k in ref}
    bad = {k: e for k, e in errs.items() if not e <= TOL}
    assert not bad, f'over tolerance: {bad} (all: {errs})'
    return errs


# the last three: 32 channel blocks; 1037 token tiles (the four-tiles-per-block kernels with a spare wavefront);
# 514 tiles (two per block)
@pytest.mark.parametrize('B,T,C', [(1, 16, 64), (2, 48, 128), (3, 64, 768), (2, 1024, 256), (2, 64, 2048), (17, 976, 256),
                                   (2, 4112, 128)])
def test_ddlerp_parity(B, T, C):
    check(*run_both(B, T, C, 32, seed=300 + T + C))


# rank 64 (two 32-wide contractions per interpolation; the second backward pass keeps its weight fragments in
# registers): a single tile, a ragged count of tiles, the two- and four-tiles-per-block kernels, 64 channel blocks
@pytest.mark.parametrize('B,T,C', [(1, 16, 64), (2, 48, 128), (3, 64, 768), (8, 1024, 768), (17, 976, 256), (2, 4112, 128),
                                   (1, 256, 4096)])
def test_ddlerp_parity_rank_64(B, T, C):
    errs = check(*run_both(B, T, C, 64, seed=700 + T + C))
    print('ddlerp rank 64 errors', {k: f'{v:.2e}' for k, v in errs.items()})


def test_ddlerp_parity_cfg4_shape():
    """x [8,1024,768], D = 32: the time-mixer block's shape."""
    errs = check(*run_both(8, 1024, 768, 32, seed=4))
    print('ddlerp cfg4 errors', {k: f'{v:.2e}' for k, v in errs.items()})


def test_ddlerp_outputs_are_views_of_one_buffer_and_bf16():
    from wind_rwkv.rwkv7 import ddlerp
    d = inputs.ddlerp_inputs(1, 16, 64, 32, 1, dtype=torch.bfloat16)
    ys = ddlerp(d['x'].to(DEV), *[d[n].to(DEV) for n in PNAMES])
    assert len(ys) == 4 and all(y.dtype == torch.bfloat16 and y.shape == (1, 16, 64) for y in ys)


def test_ddlerp_zero_lora_reduces_to_plain_lerp():
    from wind_rwkv.rwkv7 import ddlerp
    d = inputs.ddlerp_inputs(2, 32, 128, 32, 2, dtype=torch.bfloat16)
    x = d['x'].to(DEV)
    beta = d['beta'].bfloat16().to(DEV)
    ys = ddlerp(x, d['alpha'].to(DEV), d['L'].to(DEV), torch.zeros_like(d['R']).to(DEV), beta)
    xf = x.float()
    xx = torch.cat([torch.zeros_like(xf[:, :1]), xf[:, :-1]], 1) - xf
    for k in range(4):
        exp = (xf + xx * beta[k, 0, 0].float()).bfloat16()
        assert seq_ref.rel_err(ys[k].float().cpu(), exp.float().cpu()) < 1e-3


# ranks the kernels do not have run at the next one that they have, zero-padded (the reference takes the rank from the
# shapes, rwkv7_ddlerp.py:311)
@pytest.mark.parametrize('D', [8, 16, 40, 48])
def test_ddlerp_parity_other_ranks(D):
    got, ref = run_both(2, 64, 256, D, seed=900 + D)
    assert got['dL'].shape == ref['dL'].shape == (4 * D, 256) and got['dR'].shape == (4, 256, D)
    check(got, ref)


# ranks above 64 run as pieces of at most 64 whose outputs are added
@pytest.mark.parametrize('D', [96, 128, 160])
def test_ddlerp_parity_ranks_above_64(D):
    got, ref = run_both(2, 64, 256, D, seed=950 + D)
    assert got['dL'].shape == (4 * D, 256) and got['dR'].shape == (4, 256, D)
    check(got, ref)


def test_ddlerp_rejects_unsupported_shapes():
    from wind_rwkv import _native
    lib = _native.lib()
    assert lib.wind_rwkv7_ddlerp_forward(1, 16, 100, 32, *([0x1000] * 8), None) == 9
    assert lib.wind_rwkv7_ddlerp_forward(1, 10, 64, 32, *([0x1000] * 8), None) == 4
    for rank in (8, 16, 48, 96, 128):
        assert lib.wind_rwkv7_ddlerp_forward(1, 16, 64, rank, *([0x1000] * 8), None) == 8
