"""The operators under ``torch.compile(fullgraph=True)``.

The reference's own scripts wrap its operators this way before checking and timing them
(tests/test_attn_ln.py:52 with mode='reduce-overhead', tests/test_ddlerp.py:37, tests/test_expand_loras.py:56;
tests/test_time_mixer.py:67 for the block), so a drop-in has to trace without a graph break: every kernel
launch is a ``torch.library`` operator, size queries are constants for the tracer, and nothing reads a data
pointer outside an operator.  Compiled results must equal the eager ones bit for bit (same kernels).
"""
from collections import namedtuple

import pytest
import torch

from oracle import inputs

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _leaves(args):
    return [a.detach().clone().requires_grad_() for a in args]


def _check(fn, args, tol=0.0, **compile_kw):
    """tol = 0: bit for bit (everything is this package's kernels); tol > 0: normalised error, where the compiler
    fuses PyTorch expressions of its own and rounds differently from the eager run."""
    torch._dynamo.reset()
    compiled = torch.compile(fn, fullgraph=True, **compile_kw)
    results = []
    for f in (fn, compiled, compiled):           # the second compiled call replays what the first one built
        leaves = _leaves(args)
        out = f(*leaves)
        outs = list(out) if isinstance(out, (tuple, list)) else [out]
        torch.autograd.backward(outs, [torch.ones_like(o) for o in outs])
        torch.cuda.synchronize()
        results.append([o.detach().clone() for o in outs] + [x.grad.clone() for x in leaves])
    for got in results[1:]:
        for i, (a, b) in enumerate(zip(got, results[0])):
            if tol:
                err = float((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30))
                assert err <= tol, f'compiled result {i}: {err}'
                continue
            assert torch.equal(a, b), f'compiled result {i} differs from the eager one'


def _seqs(B=2, T=64, H=12, C=64, seed=5):
    d = inputs.attn_ln_inputs(B, T, H, C, seed, dtype=torch.bfloat16)
    return d, [d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab']


@pytest.mark.parametrize('C', [64, 128])
def test_attn_compiles(C):
    """Head size 64 and, with the kernels of the other head sizes, 128."""
    from wind_rwkv.rwkv7 import attn
    _, seqs = _seqs(H=768 // C, C=C)
    _check(lambda *a: attn(*a, C), seqs)


def test_attn_ln_compiles_at_another_head_size():
    """attn_ln at head size 128 with dot_prec='bf16': the plain operator's kernels and the epilogue operator trace
    as one graph (two registered operators each way)."""
    from wind_rwkv.rwkv7 import attn_ln
    d, seqs = _seqs(H=6, C=128)
    args = seqs + [d['g'].reshape(2, 64, 768).to(DEV), d['params'].to(DEV)]
    _check(lambda *a: attn_ln(*a, 128), args)


@pytest.mark.parametrize('mode', [None, 'reduce-overhead'])
def test_attn_ln_compiles(mode):
    from wind_rwkv.rwkv7 import attn_ln
    d, seqs = _seqs()
    args = seqs + [d['g'].reshape(2, 64, 768).to(DEV), d['params'].to(DEV)]
    _check(lambda *a: attn_ln(*a, 64), args, **({'mode': mode} if mode else {}))


def test_ddlerp_compiles():
    from wind_rwkv.rwkv7 import ddlerp
    d = inputs.ddlerp_inputs(2, 64, 768, 32, 6, dtype=torch.bfloat16)
    _check(ddlerp, [d[n].to(DEV) for n in ('x', 'alpha', 'L', 'R', 'beta')])


def test_expand_loras_compiles():
    from wind_rwkv.rwkv7 import expand_loras
    d = inputs.expand_loras_inputs(2, 64, 768, 16, 7, dtype=torch.bfloat16)
    names = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']
    _check(lambda *a: expand_loras(*a, 64), [d[n].to(DEV) for n in names])


@pytest.mark.parametrize('H', [12, 6])
def test_time_mixer_compiles(H):
    """12 heads of 64: the fused kernels; 6 heads of 128: that head size's WKV7 kernels, the epilogue operator and the
    LoRA expansion with per-head statistics, all registered operators too."""
    from wind_rwkv.rwkv7 import TimeMixer
    Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
    gen = torch.Generator().manual_seed(8)
    model = TimeMixer(Config(12, H, 768), 6)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    model = model.to(DEV)
    x = torch.randn(2, 64, 768, generator=gen).to(DEV)
    torch._dynamo.reset()
    compiled = torch.compile(model, fullgraph=True)
    results = []
    for f in (model, compiled, compiled):
        xl = x.clone().requires_grad_()
        y = f(xl)
        y.backward(torch.ones_like(y))
        torch.cuda.synchronize()
        results.append([y.detach().clone(), xl.grad.clone()] + [p.grad.clone() for p in model.parameters()])
        model.zero_grad(set_to_none=True)
    for got in results[1:]:
        for i, (a, b) in enumerate(zip(got, results[0])):
            assert torch.equal(a, b), f'compiled result {i} differs from the eager one'


def test_compiled_operators_follow_a_changing_shape():
    """The reference's scripts call one compiled function at two batch sizes (tests/test_attn_ln.py:54-60: B=2 for
    the check, B=64 for the timing); the second shape makes the tracer recompile with symbolic sizes, which
    must not reach the library's size queries."""
    from wind_rwkv.rwkv7 import attn_ln, ddlerp, expand_loras
    torch._dynamo.reset()
    f = torch.compile(lambda *a: attn_ln(*a, 64), fullgraph=True)
    g = torch.compile(ddlerp, fullgraph=True)
    h = torch.compile(lambda *a: expand_loras(*a, 64), fullgraph=True)
    names = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']
    for B, T in [(2, 64), (3, 128), (1, 48)]:
        d = inputs.attn_ln_inputs(B, T, 12, 64, 5, dtype=torch.bfloat16)
        args = [d[n].reshape(B, T, 768).to(DEV) for n in 'qwkvab'] + [d['g'].reshape(B, T, 768).to(DEV), d['params'].to(DEV)]
        dd = inputs.ddlerp_inputs(B, T, 768, 32, 6, dtype=torch.bfloat16)
        el = inputs.expand_loras_inputs(B, T, 768, 16, 7, dtype=torch.bfloat16)
        for fn, eager, a in ((f, lambda *x: attn_ln(*x, 64), args), (g, ddlerp, [dd[n].to(DEV) for n in ('x', 'alpha', 'L', 'R', 'beta')]),
                             (h, lambda *x: expand_loras(*x, 64), [el[n].to(DEV) for n in names])):
            res = []
            for call in (eager, fn):
                leaves = _leaves(a)
                out = call(*leaves)
                outs = list(out) if isinstance(out, (tuple, list)) else [out]
                torch.autograd.backward(outs, [torch.ones_like(o) for o in outs])
                res.append([o.detach() for o in outs] + [x.grad for x in leaves])
            for i, (x, y) in enumerate(zip(*res)):
                assert torch.equal(x, y), f'B={B} T={T}: compiled result {i} differs'
