"""GPU parity of expand_loras against the fp64 oracle: the four outputs and all fourteen gradients.
Gate 1e-2 (tests/test_expand_loras.py:58, tests/utils.py:18); the oracle sees the bf16-rounded inputs."""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
TOL = 1e-2
DEV = 'cuda'
NAMES = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']
OUT = ['w', 'k', 'kk', 'b']


def run_both(B, T, C, D, seed, scale=1.0, head_size=64):
    from wind_rwkv.rwkv7 import expand_loras
    d = inputs.expand_loras_inputs(B, T, C, D, seed, dtype=torch.bfloat16)
    for n in NAMES[2:10]:
        d[n] = (d[n].float() * scale).bfloat16()
    xo = [d[n].double().requires_grad_() for n in NAMES]
    yo = seq_ref.expand_loras_seq(*xo, head_size)
    go = torch.autograd.grad(yo, xo, [g.double() for g in d['dy']])
    xd = [(d[n].float() if i >= 6 else d[n]).to(DEV).requires_grad_() for i, n in enumerate(NAMES)]
    yd = expand_loras(*xd, head_size)
    torch.autograd.backward(list(yd), [g.to(DEV) for g in d['dy']])
    torch.cuda.synchronize()
    got = {n: y.detach().float().cpu() for n, y in zip(OUT, yd)}
    ref = {n: y.detach() for n, y in zip(OUT, yo)}
    for n, x, g in zip(NAMES, xd, go):
        got['d' + n] = x.grad.float().cpu()
        ref['d' + n] = g
    return got, ref


def check(got, ref):
    errs = {k: seq_ref.rel_err(got[k], ref[k]) for k in ref}
    bad = {k: e for k, e in errs.items() if not e <= TOL}
    assert not bad, f'over tolerance: {bad} (all: {errs})'
    return errs


# the last two: 32 heads; 1037 token tiles over 4 heads
@pytest.mark.parametrize('B,T,C,D', [(1, 16, 64, 16), (2, 48, 128, 16), (2, 64, 768, 16), (2, 64, 256, 32), (1, 32, 128, 64),
                                     (2, 64, 2048, 16), (17, 976, 256, 16)])
def test_expand_loras_parity(B, T, C, D):
    check(*run_both(B, T, C, D, seed=400 + T + D, scale=0.5))


# Head sizes other than 64: the forward walks each head on its own, the backward takes the norm and the projection
# of every (token, head) from a first kernel.  All three ranks; heads smaller than, straddling (48, 96: a block of 64
# channels holds pieces of two heads) and larger than the 64-channel blocks; one head over all channels; 1037 tiles.
@pytest.mark.parametrize('B,T,C,D,N', [(1, 16, 64, 16, 16), (2, 48, 128, 16, 32), (2, 64, 192, 16, 48), (2, 64, 192, 32, 96),
                                       (2, 64, 768, 16, 128), (1, 32, 256, 64, 128), (2, 64, 256, 32, 256),
                                       (2, 64, 2048, 16, 32), (17, 976, 256, 16, 128), (8, 1024, 768, 16, 128)])
def test_expand_loras_parity_other_head_sizes(B, T, C, D, N):
    errs = check(*run_both(B, T, C, D, seed=900 + T + D + N, scale=0.5, head_size=N))
    print(f'expand_loras head size {N} worst', max(errs.items(), key=lambda kv: kv[1]))


def test_expand_loras_parity_cfg4_shape():
    """[8,1024,768] with rank 16: the time-mixer block's shape; inputs ~ N(0,1) as in the reference's script."""
    errs = check(*run_both(8, 1024, 768, 16, seed=4))
    print('expand_loras cfg4 errors', {k: f'{v:.2e}' for k, v in errs.items()})


def test_expand_loras_output_invariants():
    from wind_rwkv.rwkv7 import expand_loras
    d = inputs.expand_loras_inputs(2, 32, 128, 16, 5, dtype=torch.bfloat16)
    w, k, kk, b = expand_loras(*[d[n].to(DEV) for n in NAMES], 64)
    assert all(t.dtype == torch.bfloat16 and t.shape == (2, 32, 128) for t in (w, k, kk, b))
    assert (w.float() <= -0.5 + 1e-2).all()
    norms = kk.float().view(2, 32, 2, 64).norm(dim=-1)
    assert torch.allclose(norms, torch.ones_like(norms), atol=2e-2)


def test_expand_loras_rejects_unsupported():
    from wind_rwkv import _native
    lib = _native.lib()
    p = [0x1000] * 18
    for head_size in (8, 24, 40, 0, -16):          # head sizes are multiples of 16
        assert lib.wind_rwkv7_expand_loras_forward(1, 16, 64, 16, head_size, *p, None) == 3
    assert lib.wind_rwkv7_expand_loras_forward(1, 16, 96, 16, 48, *p, None) == 9    # channels in blocks of 64
    assert lib.wind_rwkv7_expand_loras_forward(1, 16, 128, 16, 96, *p, None) == 9   # heads that do not tile the channels
    assert lib.wind_rwkv7_expand_loras_forward(1, 16, 64, 8, 64, *p, None) == 8
    assert lib.wind_rwkv7_expand_loras_forward(1, 16, 96, 16, 64, *p, None) == 9
