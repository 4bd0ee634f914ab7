"""WKV7 with float32 sequences (the fp32 kernels) against the fp64 sequential recurrence.

Gate: normalised L2 error <= 1e-4 on the output, the final state and every gradient, for float32 inputs and
outputs.  The reference's counterpart is its Triton kernel with dot_prec='fp32' (rwkv7_attn_triton.py:159-198);
the spec is the token loop of tests/test_attn.py:6-18, restated in oracle/seq_ref.py:wkv7_seq and, with its
hand-derived adjoint in fp64 C, in oracle/wkv7_oracle.c.
"""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
TOL = 1e-4
DEV = 'cuda'
NAMES = 'wqkvab'


def _run(d, B, T, H, C, with_state):
    from wind_rwkv.rwkv7 import WindRWKV7F32
    xs = [d[n].float().to(DEV).requires_grad_() for n in NAMES]
    s0 = (d['s0'].float() if with_state else torch.zeros(B, H, C, C)).to(DEV).requires_grad_()
    y, sT, _ = WindRWKV7F32.apply(*xs, s0)
    dsT = d['dsT'].float().to(DEV) if with_state else None
    torch.autograd.backward([y, sT] if with_state else [y], [d['dy'].float().to(DEV), dsT] if with_state else [d['dy'].float().to(DEV)])
    return y, sT, [x.grad for x in xs], s0.grad


# (1, 256, 4) and (8, 1024, 12): the reference's CPU-runnable configuration and the headline shape
@pytest.mark.parametrize('B,T,H,with_state', [(1, 16, 1, False), (2, 48, 3, True), (2, 1024, 2, True), (1, 256, 4, False),
                                              (8, 1024, 12, False), (1, 2048, 3, True), (130, 16, 1, False)])
def test_f32_parity(c_oracle, B, T, H, with_state):
    C = 64
    d = inputs.wkv7_inputs(B, T, H, C, seed=100 + T, dtype=torch.float32, s0_scale=0.3 if with_state else 0.0,
                           dsT_scale=1.0 if with_state else 0.0)
    args = [d[n] for n in 'qwkvab']
    y_ref, sT_ref = c_oracle.forward(*args, d['s0'])
    g_ref = c_oracle.backward(*args, d['s0'], d['dy'], d['dsT'])     # dq, dw, dk, dv, da, db, ds0
    ref = dict(zip(['dq', 'dw', 'dk', 'dv', 'da', 'db', 'ds0'], g_ref))
    y, sT, grads, ds0 = _run(d, B, T, H, C, with_state)
    assert y.dtype == torch.float32
    assert seq_ref.rel_err(y.detach().cpu(), y_ref) <= TOL
    assert seq_ref.rel_err(sT.detach().cpu(), sT_ref) <= TOL
    for n, g in zip(NAMES, grads):
        assert seq_ref.rel_err(g.cpu(), ref['d' + n]) <= TOL, n
    if with_state:
        assert seq_ref.rel_err(ds0.cpu(), ref['ds0']) <= TOL


@pytest.mark.parametrize('C', [16, 32, 48, 80, 96, 112, 128])
def test_f32_head_sizes(c_oracle, C):
    """Head sizes other than 64 (the reference: one CUDA build per head size, rwkv7_attn.py:46-51, and the
    large-head Triton kernels, rwkv7_attn_triton_bighead.py:31-322): every multiple of 16 up to 128 against the
    fp64 oracle, with an initial state and a gradient on the final state.  Up to 48 the kernels work at a width of 64
    channels and leave the rest empty, 80 .. 112 at 128 channels (32 lanes per state row)."""
    B, T, H = 2, 48, 3
    d = inputs.wkv7_inputs(B, T, H, C, seed=200 + C, dtype=torch.float32, s0_scale=0.3, dsT_scale=1.0)
    args = [d[n] for n in 'qwkvab']
    y_ref, sT_ref = c_oracle.forward(*args, d['s0'])
    ref = dict(zip(['dq', 'dw', 'dk', 'dv', 'da', 'db', 'ds0'], c_oracle.backward(*args, d['s0'], d['dy'], d['dsT'])))
    y, sT, grads, ds0 = _run(d, B, T, H, C, True)
    assert seq_ref.rel_err(y.detach().cpu(), y_ref) <= TOL
    assert seq_ref.rel_err(sT.detach().cpu(), sT_ref) <= TOL
    for n, g in zip(NAMES, grads):
        assert seq_ref.rel_err(g.cpu(), ref['d' + n]) <= TOL, n
    assert seq_ref.rel_err(ds0.cpu(), ref['ds0']) <= TOL


@pytest.mark.parametrize('C', [64, 128])
def test_f32_many_heads(c_oracle, C):
    """More (batch, head) pairs than half the compute units: the forward runs one block per head with all its rows."""
    B, T, H = 34, 32, 4
    d = inputs.wkv7_inputs(B, T, H, C, seed=260 + C, dtype=torch.float32, s0_scale=0.3, dsT_scale=1.0)
    args = [d[n] for n in 'qwkvab']
    y_ref, sT_ref = c_oracle.forward(*args, d['s0'])
    ref = dict(zip(['dq', 'dw', 'dk', 'dv', 'da', 'db', 'ds0'], c_oracle.backward(*args, d['s0'], d['dy'], d['dsT'])))
    y, sT, grads, ds0 = _run(d, B, T, H, C, True)
    assert seq_ref.rel_err(y.detach().cpu(), y_ref) <= TOL and seq_ref.rel_err(sT.detach().cpu(), sT_ref) <= TOL
    for n, g in zip(NAMES, grads):
        assert seq_ref.rel_err(g.cpu(), ref['d' + n]) <= TOL, n
    assert seq_ref.rel_err(ds0.cpu(), ref['ds0']) <= TOL


def test_f32_large_head_long_sequence(c_oracle):
    """C = 128 at T = 1024: 64 chunks of 16 tokens per block, four windows each in the backward."""
    B, T, H, C = 1, 1024, 2, 128
    d = inputs.wkv7_inputs(B, T, H, C, seed=321, dtype=torch.float32)
    args = [d[n] for n in 'qwkvab']
    y_ref, _ = c_oracle.forward(*args, d['s0'])
    ref = dict(zip(['dq', 'dw', 'dk', 'dv', 'da', 'db', 'ds0'], c_oracle.backward(*args, d['s0'], d['dy'], d['dsT'])))
    y, _, grads, _ = _run(d, B, T, H, C, False)
    assert seq_ref.rel_err(y.detach().cpu(), y_ref) <= TOL
    for n, g in zip(NAMES, grads):
        assert seq_ref.rel_err(g.cpu(), ref['d' + n]) <= TOL, n


def test_other_head_sizes_through_the_public_names():
    """attn, attn_triton and attn_triton_bighead on bf16 tensors with head sizes other than 64: attn and
    dot_prec='bf16' run the bf16 matrix-core kernels for those head sizes (1e-2 gate), the default dot_prec='fp32'
    the fp32 kernels on the upcast inputs, y back in bf16 (one rounding of the output)."""
    from wind_rwkv.rwkv7 import attn, attn_triton, attn_triton_bighead, load_attn
    from wind_rwkv import _native
    for C, fn, tol in [(32, attn, 1e-2), (128, attn_triton_bighead, 4e-3), (96, lambda *x: attn_triton(*x, dot_prec='bf16'), 1e-2),
                       (128, lambda *x: attn_triton_bighead(*x, dot_prec='bf16'), 1e-2)]:
        B, T, H = 2, 32, 2
        load_attn(C)
        d = inputs.wkv7_inputs(B, T, H, C, seed=40 + C, dtype=torch.bfloat16)
        y_ref, _ = seq_ref.wkv7_seq(*[d[n].double() for n in 'qwkvab'])
        flat = [d[n].reshape(B, T, H * C).to(DEV).requires_grad_() for n in 'qwkvab']
        y = fn(*flat, C)
        assert y.dtype == torch.bfloat16 and y.shape == (B, T, H * C)
        assert seq_ref.rel_err(y.detach().view(B, T, H, C).float().cpu(), y_ref) <= tol    # 4e-3: bf16 rounding of y only
        y.float().sum().backward()
        assert all(x.grad is not None and x.grad.dtype == torch.bfloat16 and torch.isfinite(x.grad).all() for x in flat)
    with pytest.raises(_native.WindRwkv7Error):
        load_attn(256)
    with pytest.raises(_native.WindRwkv7Error):
        load_attn(24)


def test_f32_public_wrapper_and_dot_prec():
    """attn() on float32 tensors and attn_triton(dot_prec='fp32') on bf16 tensors both run the fp32 kernels."""
    from wind_rwkv.rwkv7 import attn, attn_triton
    B, T, H, C = 2, 64, 3, 64
    d = inputs.wkv7_inputs(B, T, H, C, seed=9, dtype=torch.bfloat16)
    y_ref, sT_ref = seq_ref.wkv7_seq(*[d[n].double() for n in 'qwkvab'])
    flat32 = {n: d[n].float().reshape(B, T, H * C).to(DEV) for n in 'qwkvab'}
    y, sT = attn(*[flat32[n] for n in 'qwkvab'], C, return_state=True)
    assert y.dtype == torch.float32 and sT.dtype == torch.float32
    assert seq_ref.rel_err(y.view(B, T, H, C).cpu(), y_ref) <= TOL
    assert seq_ref.rel_err(sT.cpu(), sT_ref) <= TOL
    flat16 = {n: d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab'}
    y16 = attn_triton(*[flat16[n] for n in 'qwkvab'], C, dot_prec='fp32')
    assert y16.dtype == torch.bfloat16
    assert torch.equal(y16, y.bfloat16())        # same kernels, one rounding of the output
    y_fast = attn_triton(*[flat16[n] for n in 'qwkvab'], C, dot_prec='bf16')
    assert seq_ref.rel_err(y_fast.view(B, T, H, C).float().cpu(), y_ref) <= 1e-2


@pytest.mark.parametrize('B,T,H,C', [(8, 256, 12, 64), (2, 128, 3, 128), (2, 64, 5, 48)])
def test_f32_backward_is_reproducible(B, T, H, C):
    """dq, dk, da, db, dw are sums of two blocks' parts added by atomics onto zeros: two addends, so the order in
    which they arrive does not show in the result."""
    d = inputs.wkv7_inputs(B, T, H, C, seed=77, dtype=torch.float32, s0_scale=0.3, dsT_scale=1.0)
    first = _run(d, B, T, H, C, True)
    for _ in range(3):
        again = _run(d, B, T, H, C, True)
        assert torch.equal(first[0], again[0]) and torch.equal(first[1], again[1]) and torch.equal(first[3], again[3])
        assert all(torch.equal(g0, g1) for g0, g1 in zip(first[2], again[2]))


@pytest.mark.parametrize('T,cut,H,C', [(96, 32, 2, 64), (8192, 2048, 3, 64), (2048, 512, 2, 128), (512, 256, 70, 32)])
def test_f32_is_reproducible_and_carries_state(T, cut, H, C):
    from wind_rwkv.rwkv7 import attn
    B = 1
    d = inputs.wkv7_inputs(B, T, H, C, seed=13, dtype=torch.float32)
    flat = {n: d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab'}
    args = lambda sl: [flat[n][:, sl].contiguous() for n in 'qwkvab']
    y_all, s_all = attn(*args(slice(0, T)), C, return_state=True)
    y_again, _ = attn(*args(slice(0, T)), C, return_state=True)
    assert torch.equal(y_all, y_again)
    y1, s1 = attn(*args(slice(0, cut)), C, return_state=True)
    y2, s2 = attn(*args(slice(cut, T)), C, s0=s1, return_state=True)
    # the token recurrence is the same arithmetic whether or not the sequence is cut
    assert torch.equal(torch.cat([y1, y2], dim=1), y_all) and torch.equal(s2, s_all)


@pytest.mark.parametrize('rows', [128, 256, 4096])
def test_group_norm_heads_matches_fp64_library_routine(rows):
    """The per-head normalisation of the PyTorch-composed epilogues against the framework's group_norm evaluated in
    fp64 on the CPU: forward and ALL gradients.  (The framework's GPU backward in this build returns wrong weight and
    bias gradients from 256 rows on, which is why the package does not call it; asserted here so that the reason
    stays visible - if that assertion fails the framework has been fixed and the helper may go.)"""
    from wind_rwkv.rwkv7.wkv_attn_ln import group_norm_heads
    H, HC = 12, 768
    g = torch.Generator().manual_seed(rows)
    y, dy = torch.randn(rows, HC, generator=g), torch.randn(rows, HC, generator=g)
    w, b = torch.randn(HC, generator=g), torch.randn(HC, generator=g)
    ref_in = [t.double().requires_grad_() for t in (y, w, b)]
    torch.nn.functional.group_norm(ref_in[0], H, ref_in[1], ref_in[2], eps=64e-5).backward(dy.double())
    dev_in = [t.to(DEV).requires_grad_() for t in (y, w, b)]
    out = group_norm_heads(*dev_in[:1], H, *dev_in[1:])
    out.backward(dy.to(DEV))
    ref_out = torch.nn.functional.group_norm(y.double(), H, w.double(), b.double(), eps=64e-5)
    assert seq_ref.rel_err(out.detach().cpu(), ref_out) <= 1e-6
    for x, r in zip(dev_in, ref_in):
        assert seq_ref.rel_err(x.grad.cpu(), r.grad) <= 1e-5
    if rows >= 256:
        lib_in = [t.to(DEV).requires_grad_() for t in (y, w, b)]
        torch.nn.functional.group_norm(*lib_in[:1], H, *lib_in[1:], eps=64e-5).backward(dy.to(DEV))
        assert seq_ref.rel_err(lib_in[1].grad.cpu(), ref_in[1].grad) > 0.1, 'the framework routine is right again'


@pytest.mark.parametrize('B,T', [(2, 64), (2, 256)])
def test_attn_ln_f32_matches_oracle(B, T):
    """attn_ln on float32 tensors (fp32 WKV7 kernels + the epilogue in PyTorch): output, final state and all
    gradients within 1e-4 of the fp64 oracle, from a non-zero initial state (a zero state makes the normalised
    first token ill-conditioned in any precision).  512 rows as well as 128: the parameter gradients of the
    normalisation depend on the row count in the framework's own routine (see above)."""
    from wind_rwkv.rwkv7 import attn_ln
    H, C = 3, 64
    d = inputs.attn_ln_inputs(B, T, H, C, 77, dtype=torch.float32)
    gen = torch.Generator().manual_seed(78)
    s0 = 0.3 * torch.randn(B, H, C, C, generator=gen)
    names = list('qwkvab') + ['g']
    ref_in = [d[n].double().requires_grad_() for n in names]
    p64 = d['params'].double().requires_grad_()
    s64 = s0.double().requires_grad_()
    out_ref, sT_ref = seq_ref.attn_ln_seq(*ref_in, p64, s64)
    dy = torch.randn(B, T, H, C, generator=gen)
    out_ref.backward(dy.double())
    dev_in = [d[n].reshape(B, T, H * C).to(DEV).requires_grad_() for n in names]
    pd = d['params'].to(DEV).requires_grad_()
    sd = s0.to(DEV).requires_grad_()
    out, sT = attn_ln(*dev_in, pd, C, s0=sd, return_state=True)
    out.backward(dy.reshape(B, T, H * C).to(DEV))
    assert out.dtype == torch.float32
    assert seq_ref.rel_err(out.detach().view(B, T, H, C).cpu(), out_ref.detach()) <= TOL
    assert seq_ref.rel_err(sT.detach().cpu(), sT_ref.detach()) <= TOL
    for n, x, r in zip(names, dev_in, ref_in):
        assert seq_ref.rel_err(x.grad.view(B, T, H, C).cpu(), r.grad) <= TOL, n
    assert seq_ref.rel_err(pd.grad.cpu(), p64.grad) <= TOL
    assert seq_ref.rel_err(sd.grad.cpu(), s64.grad) <= TOL


def test_attn_ln_other_head_size():
    """attn_ln(dot_prec='fp32') with HEAD_SIZE 32 on bf16 tensors: fp32 WKV7 kernels + epilogue in PyTorch, bf16 out;
    against the fp64 oracle on the same rounded inputs (the error is the rounding of the output)."""
    from wind_rwkv.rwkv7 import attn_ln, load_attn_ln
    B, T, H, C = 2, 32, 4, 32
    load_attn_ln(C)
    d = inputs.attn_ln_inputs(B, T, H, C, 91, dtype=torch.bfloat16)
    names = list('qwkvab') + ['g']
    gen = torch.Generator().manual_seed(92)
    s0 = 0.3 * torch.randn(B, H, C, C, generator=gen)
    out_ref, _ = seq_ref.attn_ln_seq(*[d[n].double() for n in names], d['params'].double(), s0.double())
    dev_in = [d[n].reshape(B, T, H * C).to(DEV).requires_grad_() for n in names]
    pd = d['params'].to(DEV).requires_grad_()
    out = attn_ln(*dev_in, pd, C, s0=s0.to(DEV), dot_prec='fp32')
    assert out.dtype == torch.bfloat16
    assert seq_ref.rel_err(out.detach().view(B, T, H, C).float().cpu(), out_ref) <= 4e-3
    out.float().sum().backward()
    assert all(x.grad is not None and torch.isfinite(x.grad).all() for x in dev_in) and torch.isfinite(pd.grad).all()


@pytest.mark.parametrize('C,with_state', [(32, False), (128, False), (32, True), (128, True)])
def test_attn_ln_other_head_size_bf16_kernels(C, with_state):
    """attn_ln at head sizes 32 and 128 on bf16 tensors (the default route, the same as dot_prec='bf16'): the plain operator's bf16 matrix-core
    kernels for that head size followed by the epilogue kernels, bf16 out; output and every gradient against the fp64 oracle (autograd
    through the token loop) on the same rounded inputs, at the bf16 gate of 1e-2 (measured: <= 7.4e-3).  T = 256:
    on sequences of a few dozen tokens from a random state the loss is dominated by the first tokens, whose small
    WKV7 output the normalisation divides by, and dq, dk then miss the gate at EVERY head size, the fused kernels of
    head size 64 included (1.0e-2 ... 1.3e-2 there at T = 64, the same inputs through this composition within 1e-4
    of them) - a property of bf16 operands on such inputs, not of a head size."""
    from wind_rwkv.rwkv7 import attn_ln, load_attn_ln
    B, T, H = 2, 256, 4
    load_attn_ln(C)
    d = inputs.attn_ln_inputs(B, T, H, C, 91, dtype=torch.bfloat16)
    names = list('qwkvab') + ['g']
    gen = torch.Generator().manual_seed(92)
    s0 = 0.1 * torch.randn(B, H, C, C, generator=gen) if with_state else None
    ref_in = [d[n].double().requires_grad_() for n in names]
    ref_p = d['params'].double().requires_grad_()
    out_ref, _ = seq_ref.attn_ln_seq(*ref_in, ref_p, s0.double() if with_state else None)
    out_ref.backward(d['dy'].double())
    dev_in = [d[n].reshape(B, T, H * C).to(DEV).requires_grad_() for n in names]
    pd = d['params'].to(DEV).requires_grad_()
    out = attn_ln(*dev_in, pd, C, s0=s0.to(DEV) if with_state else None)
    assert out.dtype == torch.bfloat16
    out.backward(d['dy'].reshape(B, T, H * C).to(DEV))
    errs = {n: seq_ref.rel_err(x.grad.view(B, T, H, C).float().cpu(), xr.grad) for n, x, xr in zip(names, dev_in, ref_in)}
    errs['params'] = seq_ref.rel_err(pd.grad.cpu(), ref_p.grad)
    errs['out'] = seq_ref.rel_err(out.detach().view(B, T, H, C).float().cpu(), out_ref.detach())
    assert all(e <= 1e-2 for e in errs.values()), errs
    # dot_prec='bf16' names the same route; dot_prec='fp32' and float32 tensors run the fp32 kernels
    with torch.no_grad():
        out_b = attn_ln(*[x.detach() for x in dev_in], pd.detach(), C, s0=s0.to(DEV) if with_state else None, dot_prec='bf16')
        assert torch.equal(out_b, out.detach())
        out_d = attn_ln(*[x.detach() for x in dev_in], pd.detach(), C, s0=s0.to(DEV) if with_state else None,
                        dot_prec='fp32')
        out32 = attn_ln(*[x.detach().float() for x in dev_in], pd.detach(), C, s0=s0.to(DEV) if with_state else None,
                        dot_prec='bf16')
    assert out32.dtype == torch.float32 and torch.equal(out32.bfloat16(), out_d)
    assert seq_ref.rel_err(out32.view(B, T, H, C).cpu(), out_ref.detach()) <= 1e-4
