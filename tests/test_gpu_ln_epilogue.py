"""The attn_ln epilogue as an operator of its own (GroupNorm over each head + bonus + gate; the reference computes it
inside its attn_ln kernels, attn_ln.cu:11-37 forward and :40-104 backward, spec tests/test_attn_ln.py:18-21) against
the same expression in float64 with autograd, on the bf16-rounded inputs the kernels see.  Every stage is elementwise
or a per-token sum, so the error is that of the bf16 outputs: gate 5e-3 on every tensor."""
import pytest
import torch

from oracle import seq_ref

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = 5e-3


def reference(y, q, k, v, g, params, H):
    B, T, HC = y.shape
    C = HC // H
    yh = y.view(B, T, H, C)
    xhat = (yh - yh.mean(-1, keepdim=True)) * torch.rsqrt(yh.var(-1, unbiased=False, keepdim=True) + 64e-5)
    x1 = xhat.view(B, T, HC) * params[0] + params[1]
    dot = (q * k * params[2]).view(B, T, H, C).sum(-1, keepdim=True)
    return (x1 + (dot * v.view(B, T, H, C)).view(B, T, HC)) * g


def run_both(B, T, H, C, seed, offset=0.0):
    from wind_rwkv.rwkv7.wkv_attn_ln import LnEpilogue
    gen = torch.Generator().manual_seed(seed)
    seqs = [(torch.randn(B, T, H * C, generator=gen) + (offset if i == 0 else 0.0)).bfloat16() for i in range(5)]
    params = torch.randn(3, H * C, generator=gen)
    dout = torch.randn(B, T, H * C, generator=gen).bfloat16()
    ref_in = [t.double().requires_grad_() for t in seqs] + [params.double().requires_grad_()]
    out_ref = reference(*ref_in, H)
    out_ref.backward(dout.double())
    dev_in = [t.to(DEV).requires_grad_() for t in seqs] + [params.to(DEV).requires_grad_()]
    out = LnEpilogue.apply(*dev_in, H)
    assert out.dtype == torch.bfloat16
    out.backward(dout.to(DEV))
    torch.cuda.synchronize()
    errs = {'out': seq_ref.rel_err(out.detach().float().cpu(), out_ref.detach())}
    for n, x, xr in zip(('dy', 'dq', 'dk', 'dv', 'dg', 'dparams'), dev_in, ref_in):
        errs[n] = seq_ref.rel_err(x.grad.float().cpu(), xr.grad)
    return errs


# every head size; one tile; a tile count that is no multiple of the four wavefronts of a block; more ranges than tiles
# allow (one head); 1037 tiles
@pytest.mark.parametrize('C', [16, 32, 48, 64, 80, 96, 112, 128])
@pytest.mark.parametrize('B,T,H', [(1, 16, 1), (2, 48, 3), (3, 1040, 5), (17, 976, 2)])
def test_ln_epilogue_parity(B, T, H, C):
    errs = run_both(B, T, H, C, seed=1000 + C + T)
    assert all(e <= TOL for e in errs.values()), errs


def test_ln_epilogue_parity_block_shape():
    """[8,1024,768] as 6 heads of 128: the shape of the time-mixer block."""
    errs = run_both(8, 1024, 6, 128, seed=4)
    print('ln_epilogue [8,1024,6x128] errors', {k: f'{v:.2e}' for k, v in errs.items()})
    assert all(e <= TOL for e in errs.values()), errs


def test_ln_epilogue_large_mean():
    """A WKV7 output whose mean is twenty times its spread: the variance is taken about the mean, not as a
    difference of second moments."""
    errs = run_both(2, 64, 4, 128, seed=5, offset=20.0)
    assert errs['out'] <= TOL and errs['dg'] <= TOL, errs


def test_ln_epilogue_reproducible():
    from wind_rwkv.rwkv7.wkv_attn_ln import LnEpilogue
    gen = torch.Generator().manual_seed(6)
    base = [torch.randn(3, 1040, 5 * 96, generator=gen).bfloat16().to(DEV) for _ in range(5)] + [torch.randn(3, 5 * 96, generator=gen).to(DEV)]
    dout = torch.randn(3, 1040, 5 * 96, generator=gen).bfloat16().to(DEV)
    runs = []
    for _ in range(2):
        xs = [t.clone().requires_grad_() for t in base]
        LnEpilogue.apply(*xs, 5).backward(dout)
        runs.append([x.grad.clone() for x in xs])
    assert all(torch.equal(a, b) for a, b in zip(*runs))


def test_ln_epilogue_rejects_unsupported():
    from wind_rwkv import _native
    lib = _native.lib()
    p = [0x1000] * 7
    assert lib.wind_rwkv7_ln_epilogue_forward(1, 16, 2, 144, *p, None) == 3
    assert lib.wind_rwkv7_ln_epilogue_forward(1, 16, 2, 24, *p, None) == 3
    assert lib.wind_rwkv7_ln_epilogue_forward(1, 10, 2, 64, *p, None) == 4
    assert lib.wind_rwkv7_ln_epilogue_bwd_workspace_bytes(1, 10, 2, 64) == 0
    assert lib.wind_rwkv7_ln_epilogue_bwd_workspace_bytes(8, 1024, 6, 128) > 0


@pytest.mark.parametrize('C,with_state', [(32, False), (128, True), (96, True)])
def test_attn_ln_entry_points_at_other_head_sizes(C, with_state):
    """wind_rwkv7_attn_ln_forward / _backward at a head size other than 64 (the C-level composition of the plain
    entry points, the epilogue kernels and the sum of the two parts of dq, dk, dv) against the operator-level
    composition that attn_ln() makes of the same kernels: bit for bit."""
    from oracle import inputs
    from wind_rwkv.rwkv7 import attn_ln
    from wind_rwkv.rwkv7.wkv_attn import no_state
    from wind_rwkv.rwkv7.wkv_attn_ln import bw_attn_ln, fw_attn_ln
    B, T, H = 2, 80, 3
    d = inputs.attn_ln_inputs(B, T, H, C, 17, dtype=torch.bfloat16)
    names = list('wqkvab') + ['g']
    gen = torch.Generator().manual_seed(18)
    s0 = (0.2 * torch.randn(B, H, C, C, generator=gen)).to(DEV) if with_state else None
    dy = d['dy'].reshape(B, T, H * C).to(DEV)
    params = d['params'].to(DEV)
    # operator level
    xs = {n: d[n].reshape(B, T, H * C).to(DEV).requires_grad_() for n in names}
    pr = params.clone().requires_grad_()
    out, sT = attn_ln(xs['q'], xs['w'], xs['k'], xs['v'], xs['a'], xs['b'], xs['g'], pr, C, s0=s0, return_state=True)
    out.backward(dy)
    # C level
    raw = [d[n].to(DEV).contiguous() for n in names]
    st = s0 if with_state else no_state(torch.bfloat16, DEV)   # (what attn() passes for an absent state)
    y, sT2, saved = fw_attn_ln(*raw, params, st)
    grads = bw_attn_ln(*raw, params, saved, dy.view(B, T, H, C), no_state(torch.float32, DEV), want_ds0=False)
    torch.cuda.synchronize()
    assert torch.equal(y.view(B, T, H * C), out.detach()) and torch.equal(sT2, sT)
    for n, gr in zip(names, grads[:7]):
        assert torch.equal(gr.view(B, T, H * C), xs[n].grad), n
    assert torch.equal(grads[7], pr.grad)
    # the forward that keeps nothing
    y3, sT3, _ = fw_attn_ln(*raw, params, st, save=False)
    assert torch.equal(y3, y) and torch.equal(sT3, sT2)
