"""GPU parity of attn_ln (WKV7 + per-head GroupNorm + bonus + gate) against the fp64 oracle.

The oracle composes the C restatement of the recurrence with the fp64 epilogue of oracle/seq_ref.py,
differentiated by autograd; inputs are the bf16-rounded ones.  Gate: normalised error <= 1e-2 on the
output, the final state, the seven sequence gradients, dparams and ds0.

Conditioning note.  GroupNorm is scale-invariant, so its gradient at a token grows like 1/std(y_t).  With a
ZERO initial state the first token is y_0 = (k_0.q_0) v_0, whose normalised value flips sign where the
64-term dot product k_0.q_0 crosses zero: near that set no bf16-operand arithmetic (this one or the
reference's) can reproduce the gradient to 1e-2, and ds0, which only sees the first few tokens, is
dominated by it.  The small cases therefore start from a generic state (entries ~ N(0,1)), where every
tensor including ds0 meets the gate; the zero-state benchmark configuration gates everything the public
wrapper exposes (it creates s0 itself and drops ds0, rwkv7_attn_ln.py:61-62) and holds ds0 to a looser bound (0.25).
"""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
TOL = 1e-2
DEV = 'cuda'
SEQ = ('w', 'q', 'k', 'v', 'a', 'b', 'g')


def oracle(c_oracle, d, state_dtype):
    s0 = d['s0'].to(state_dtype).double()
    dsT = d['dsT'].to(state_dtype).double()
    args = [d[n].double() for n in 'qwkvab']
    y, sT = c_oracle.forward(*args, s0)
    y = y.clone().requires_grad_()
    leaf = {n: d[n].double().clone().requires_grad_() for n in ('q', 'k', 'v', 'g')}
    params = d['params'].double().clone().requires_grad_()
    out = seq_ref.attn_ln_epilogue(y, leaf['q'], leaf['k'], leaf['v'], leaf['g'], params)
    gy, gq, gk, gv, gg, gp = torch.autograd.grad(out, [y, leaf['q'], leaf['k'], leaf['v'], leaf['g'], params],
                                                d['dy'].double())
    dq, dw, dk, dv, da, db, ds0 = c_oracle.backward(*args, s0, gy, dsT)
    return dict(y=out.detach(), sT=sT, dw=dw, dq=dq + gq, dk=dk + gk, dv=dv + gv, da=da, db=db, dg=gg, dparams=gp,
                ds0=ds0)


def device(d, state_dtype):
    from wind_rwkv.rwkv7.wkv_attn_ln import WindRWKV7LN
    xs = {n: d[n].to(DEV).requires_grad_() for n in SEQ}
    params = d['params'].to(DEV).requires_grad_()
    s0 = d['s0'].to(state_dtype).to(DEV).requires_grad_()
    y, sT, _ = WindRWKV7LN.apply(*[xs[n] for n in SEQ], params, s0)
    torch.autograd.backward([y, sT], [d['dy'].to(DEV), d['dsT'].to(state_dtype).to(DEV)])
    torch.cuda.synchronize()
    out = dict(y=y, sT=sT, dparams=params.grad, ds0=s0.grad, **{'d' + n: xs[n].grad for n in SEQ})
    return {k: v.detach().float().cpu() for k, v in out.items()}


def check(got, ref, skip=()):
    errs = {k: seq_ref.rel_err(got[k], ref[k]) for k in ref}
    bad = {k: e for k, e in errs.items() if not e <= TOL and k not in skip}
    assert not bad, f'over tolerance: {bad} (all: {errs})'
    return errs


@pytest.mark.parametrize('B,T,H,state_dtype,s0s', [
    (1, 16, 1, torch.float32, 1.0),
    (2, 64, 3, torch.float32, 1.0),
    (2, 64, 3, torch.bfloat16, 1.0),
    (2, 272, 2, torch.float32, 1.0),
    (20, 32, 12, torch.float32, 1.0),     # 240 (batch, head) pairs: one block per head, the epilogue inside the forward kernel
    (5, 48, 20, torch.bfloat16, 1.0),     # 100 pairs: two blocks per head, the epilogue as a kernel of its own
])
def test_attn_ln_parity_small(c_oracle, B, T, H, state_dtype, s0s):
    d = inputs.attn_ln_inputs(B, T, H, 64, seed=200 + T, dtype=torch.bfloat16)
    d['s0'] = torch.randn(B, H, 64, 64, generator=torch.Generator().manual_seed(7)) * s0s
    d['dsT'] = torch.randn(B, H, 64, 64, generator=torch.Generator().manual_seed(8)) * s0s
    check(device(d, state_dtype), oracle(c_oracle, d, state_dtype))


@pytest.mark.parametrize('interval', [16, 32])
def test_attn_ln_parity_at_either_checkpoint_interval(c_oracle, interval):
    """A state per 16-token chunk (the reference's layout) or per pair of chunks (the default) in both directions."""
    from wind_rwkv.rwkv7 import set_checkpoint_interval
    d = inputs.attn_ln_inputs(3, 160, 4, 64, seed=260, dtype=torch.bfloat16)
    d['s0'] = torch.randn(3, 4, 64, 64, generator=torch.Generator().manual_seed(7))
    d['dsT'] = torch.randn(3, 4, 64, 64, generator=torch.Generator().manual_seed(8))
    set_checkpoint_interval(interval)
    try:
        got = device(d, torch.float32)
    finally:
        set_checkpoint_interval(32)
    check(got, oracle(c_oracle, d, torch.float32))


def _offset_inputs(B, T, H, offset, seed, C=64):
    """attn_ln inputs whose value vectors carry a common offset: the WKV7 output of a token is then a multiple of
    (offset + noise) per channel, i.e. its mean over the head is about `offset` times its spread."""
    d = inputs.attn_ln_inputs(B, T, H, C, seed=seed, dtype=torch.bfloat16)
    d['v'] = (d['v'].float() + offset).bfloat16()
    # (a generic initial state: from a zero state the first token's normalised output is ill-conditioned, see above)
    d['s0'] = torch.randn(B, H, C, C, generator=torch.Generator().manual_seed(seed + 1))
    d['dsT'] = torch.zeros(B, H, C, C)
    return d


def test_large_mean_both_forward_forms(c_oracle):
    """GroupNorm divides by the spread of a token's WKV7 output over the head, so what is handed to it must be accurate
    relative to that spread, not to the output's size.  The one-kernel forward normalises the fp32 accumulators (as the
    reference does, attn_ln.cu:192); the forward that runs the epilogue as a kernel of its own (few (batch, head)
    pairs) hands the output over in bf16, centred per block of 16 channels so that the rounding is relative to the
    spread; the backward epilogue reads the same kept tensor in either case.  With a mean of ~20 spreads, through
    either form (12 pairs: two kernels; the same 12 replicated to 144 pairs: one kernel): the output and every
    gradient that the epilogue feeds directly meet the usual gate against the fp64 oracle.  Uncentred bf16 would be
    off by 20 * 2^-9 = 4 % of the normalised output.  dw, da and db are a different matter: with such value vectors
    the recurrence's own bf16 matrix operands limit them (7e-2 against the oracle, in both forms alike, and with any
    epilogue); they are only held to agree between the forms as they do against the oracle."""
    H, T = 12, 128
    base = _offset_inputs(1, T, H, 20.0, seed=271)
    wide = {k: (v.repeat(12, *[1] * (v.dim() - 1)) if k != 'params' else v) for k, v in base.items()}   # (s0 included)
    few, many = device(base, torch.float32), device(wide, torch.float32)
    ref = oracle(c_oracle, base, torch.float32)
    for name in ('y', 'dq', 'dk', 'dv', 'dg'):
        for form, got in (('two kernels', few), ('one kernel', many)):
            err = seq_ref.rel_err(got[name][0], ref[name][0])
            assert err < TOL, (name, form, err)
        assert seq_ref.rel_err(few[name][0], many[name][0]) < 5e-3, name
    for name in ('dw', 'da', 'db'):
        e_few, e_many = seq_ref.rel_err(few[name][0], ref[name][0]), seq_ref.rel_err(many[name][0], ref[name][0])
        assert e_few < 0.1 and e_many < 0.1 and abs(e_few - e_many) < 0.3 * max(e_few, e_many), (name, e_few, e_many)


def test_large_mean_long_sequence_on_few_heads(c_oracle):
    """The same property on the path of long sequences on few heads (2 heads, 2048 tokens: the sequence in segments, a
    block per segment): the kept output is written centred there too."""
    d = _offset_inputs(1, 2048, 2, 20.0, seed=273)
    got, ref = device(d, torch.float32), oracle(c_oracle, d, torch.float32)
    for name in ('y', 'dq', 'dk', 'dv', 'dg'):
        err = seq_ref.rel_err(got[name], ref[name])
        assert err < TOL, (name, err)


@pytest.mark.parametrize('C', [32, 48, 128])
def test_large_mean_other_head_sizes(c_oracle, C):
    """The same property at head sizes other than 64, where attn_ln is the plain WKV7 kernels of that head size followed
    by the epilogue kernels: the scan writes the output centred per block of 16 channels and the epilogue kernels of
    both directions add the centres back in fp32."""
    d = _offset_inputs(2, 128, 3, 20.0, seed=274, C=C)
    got, ref = device(d, torch.float32), oracle(c_oracle, d, torch.float32)
    for name in ('y', 'dq', 'dk', 'dv', 'dg'):
        err = seq_ref.rel_err(got[name], ref[name])
        assert err < TOL, (C, name, err)


def test_moderate_mean_against_oracle(c_oracle):
    """A mean of one and a half spreads, both forward forms, against the fp64 oracle at the usual gate.  (At larger
    offsets the recurrence itself, whose matrix operands are bf16 here as in the reference, is no longer accurate
    to 1e-2 of the SPREAD of its output, whatever the epilogue does: at three spreads da and db reach 1.2e-2.)"""
    for B in (1, 12):
        d = _offset_inputs(B, 128, 12, 1.5, seed=272)
        check(device(d, torch.float32), oracle(c_oracle, d, torch.float32), skip=('ds0',))


def test_attn_ln_parity_cfg2_full(c_oracle):
    """B=8, T=1024, H=12, N=64, bf16: the fused benchmark configuration."""
    d = inputs.attn_ln_inputs(8, 1024, 12, 64, seed=2, dtype=torch.bfloat16)
    errs = check(device(d, torch.float32), oracle(c_oracle, d, torch.float32), skip=('ds0',))
    print('cfg2 errors', {k: f'{v:.2e}' for k, v in errs.items()})
    # ds0 from a zero state is ill-conditioned (see the note above): measured 1.7e-1 here; held to a looser bound so
    # that a regression still shows
    assert errs['ds0'] <= 0.25, errs['ds0']


def test_attn_ln_identity_epilogue_reduces_to_group_norm(c_oracle):
    """ln_w=1, ln_b=0, bonus=0, g=1: the output is the library group_norm of the WKV7 output."""
    from wind_rwkv.rwkv7 import attn_ln, load_attn_ln
    load_attn_ln(64)
    B, T, H, C = 1, 64, 2, 64
    d = inputs.wkv7_inputs(B, T, H, C, seed=9, dtype=torch.bfloat16)
    flat = {n: d[n].view(B, T, H * C).to(DEV) for n in 'qwkvab'}
    g = torch.ones(B, T, H * C, dtype=torch.bfloat16, device=DEV)
    params = torch.stack([torch.ones(H * C), torch.zeros(H * C), torch.zeros(H * C)]).to(DEV)
    out = attn_ln(flat['q'], flat['w'], flat['k'], flat['v'], flat['a'], flat['b'], g, params, C)
    yo, _ = c_oracle.forward(*[d[n] for n in 'qwkvab'], d['s0'])
    ref = torch.nn.functional.group_norm(yo.reshape(B * T, H * C), H, eps=64e-5).view(B, T, H * C)
    assert seq_ref.rel_err(out.float().cpu(), ref) < TOL


def test_dparams_is_deterministic():
    """The parameter gradient is reduced in a fixed order: two runs give identical bits."""
    d = inputs.attn_ln_inputs(2, 128, 2, 64, seed=10, dtype=torch.bfloat16)
    a1 = device(d, torch.float32)['dparams']
    a2 = device(d, torch.float32)['dparams']
    assert torch.equal(a1, a2)


@pytest.mark.parametrize('B,T,H', [(2, 64, 3), (20, 32, 12)])   # epilogue as its own kernel / inside the forward kernel
def test_absent_states_equal_zero_states(B, T, H):
    """An empty s0, no gradient for sT and no request for ds0 (NULL pointers at the C ABI) give bit for bit what
    explicit tensors of zeros give."""
    from wind_rwkv.rwkv7.wkv_attn import no_state
    from wind_rwkv.rwkv7.wkv_attn_ln import WindRWKV7LN
    d = inputs.attn_ln_inputs(B, T, H, 64, seed=78, dtype=torch.bfloat16)
    dy = d['dy'].to(DEV)

    def run(s0, dsT):
        xs = [d[n].to(DEV).requires_grad_() for n in SEQ]
        params = d['params'].to(DEV).requires_grad_()
        y, sT, _ = WindRWKV7LN.apply(*xs, params, s0)
        torch.autograd.backward([y] if dsT is None else [y, sT], [dy] if dsT is None else [dy, dsT])
        return [y.detach(), sT.detach(), params.grad] + [x.grad for x in xs]

    zeros = torch.zeros(B, H, 64, 64, dtype=torch.bfloat16, device=DEV)
    ref = run(zeros.clone().requires_grad_(), torch.zeros_like(zeros))
    got = run(no_state(torch.bfloat16, DEV), None)
    for r, g in zip(ref, got):
        assert torch.equal(r, g)
