"""Single-token decoding and the carried state of the public wrappers, against the fp64 sequential recurrence.

The reference's only decode path is the token loop of ref_attn (time_mixer.py:6-16); the oracle restates that
loop (oracle/seq_ref.py:wkv7_seq, pinned in tests/test_oracle_wkv7.py), so prompt-then-decode on the device is
compared with ONE run of the oracle over prompt + generated tokens.  Gate: normalised L2 error <= 1e-2 for bf16
inputs and outputs (the state is carried in fp32).
"""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
TOL = 1e-2
DEV = 'cuda'


def _f64(d, names):
    return [d[n].double() for n in names]


@pytest.mark.parametrize('C', [64, 16, 48, 96, 128])
@pytest.mark.parametrize('B,H,steps,state_dtype', [(1, 1, 3, torch.float32), (3, 5, 20, torch.float32),
                                                   (2, 12, 8, torch.bfloat16)])
def test_attn_step_chain(B, H, steps, state_dtype, C):
    """`steps` decode calls from a non-zero state equal the sequential recurrence over the same tokens, at head size
    64 and at the other head sizes (their own single-token kernel)."""
    from wind_rwkv.rwkv7 import attn_step
    d = inputs.wkv7_inputs(B, steps, H, C, seed=7 + steps, dtype=torch.bfloat16, s0_scale=0.5)
    s0 = d['s0'].to(state_dtype)
    y_ref, sT_ref = seq_ref.wkv7_seq(*_f64(d, 'qwkvab'), s0.double())
    state = s0.to(DEV).clone()
    ys = []
    for t in range(steps):
        tok = {n: d[n][:, t].reshape(B, H * C).contiguous().to(DEV) for n in 'qwkvab'}
        ys.append(attn_step(tok['q'], tok['w'], tok['k'], tok['v'], tok['a'], tok['b'], state, C))
    y = torch.stack(ys, dim=1).view(B, steps, H, C).float().cpu()
    tol = TOL if state_dtype == torch.float32 else 3e-2   # a bf16 state is re-rounded after every token
    assert seq_ref.rel_err(y, y_ref) <= tol
    assert seq_ref.rel_err(state.float().cpu(), sT_ref) <= tol


@pytest.mark.parametrize('C', [64, 32, 128])
def test_prompt_then_decode_attn(C):
    """attn(..., return_state=True) on a prompt, attn_step on the following tokens == one oracle run."""
    from wind_rwkv.rwkv7 import attn, attn_step
    B, H, Tp, Td = 2, 4, 48, 5
    d = inputs.wkv7_inputs(B, Tp + Td, H, C, seed=31, dtype=torch.bfloat16)
    y_ref, sT_ref = seq_ref.wkv7_seq(*_f64(d, 'qwkvab'))
    flat = {n: d[n].reshape(B, Tp + Td, H * C).to(DEV) for n in 'qwkvab'}
    p = {n: flat[n][:, :Tp].contiguous() for n in flat}
    s0 = torch.zeros(B, H, C, C, device=DEV)   # fp32 carried state
    y_p, state = attn(p['q'], p['w'], p['k'], p['v'], p['a'], p['b'], C, s0=s0, return_state=True)
    ys = [y_p]
    for t in range(Tp, Tp + Td):
        tok = {n: flat[n][:, t].contiguous() for n in flat}
        ys.append(attn_step(tok['q'], tok['w'], tok['k'], tok['v'], tok['a'], tok['b'], state, C)[:, None])
    y = torch.cat(ys, dim=1).view(B, Tp + Td, H, C).float().cpu()
    assert seq_ref.rel_err(y, y_ref) <= TOL
    assert seq_ref.rel_err(y[:, Tp:], y_ref[:, Tp:]) <= TOL
    assert seq_ref.rel_err(state.float().cpu(), sT_ref) <= TOL


@pytest.mark.parametrize('C', [64, 32, 128])
def test_prompt_then_decode_attn_ln(C):
    """The same with the epilogue.  At head sizes other than 64 the prompt runs the plain operator's kernels with the
    epilogue (here with dot_prec='bf16': that head size's matrix-core kernels and the epilogue kernels) and the steps the
    single-token kernel, whose epilogue is its own."""
    from wind_rwkv.rwkv7 import attn_ln, attn_ln_step
    B, H, Tp, Td = 2, 3, 32, 6
    d = inputs.attn_ln_inputs(B, Tp + Td, H, C, 41, dtype=torch.bfloat16)
    out_ref, sT_ref = seq_ref.attn_ln_seq(*_f64(d, 'qwkvab'), d['g'].double(), d['params'].double())
    names = list('qwkvab') + ['g']
    flat = {n: d[n].reshape(B, Tp + Td, H * C).to(DEV) for n in names}
    params = d['params'].to(DEV)
    p = {n: flat[n][:, :Tp].contiguous() for n in names}
    s0 = torch.zeros(B, H, C, C, device=DEV)
    o_p, state = attn_ln(p['q'], p['w'], p['k'], p['v'], p['a'], p['b'], p['g'], params, C, s0=s0, return_state=True,
                         dot_prec='bf16')
    outs = [o_p]
    for t in range(Tp, Tp + Td):
        tok = {n: flat[n][:, t].contiguous() for n in names}
        outs.append(attn_ln_step(tok['q'], tok['w'], tok['k'], tok['v'], tok['a'], tok['b'], tok['g'], params, state,
                                 C)[:, None])
    out = torch.cat(outs, dim=1).view(B, Tp + Td, H, C).float().cpu()
    # skip the first tokens of the prompt: from a zero state the normalised output of token 0 is (k.q) v
    # normalised, whose sign flips where the dot product over the head crosses zero (ill-conditioned in any bf16 path)
    assert seq_ref.rel_err(out[:, 4:], out_ref[:, 4:]) <= TOL
    assert seq_ref.rel_err(out[:, Tp:], out_ref[:, Tp:]) <= TOL
    assert seq_ref.rel_err(state.float().cpu(), sT_ref) <= TOL


def test_any_length_at_another_head_size():
    """Inference on a length that is no multiple of 16 at head size 128: whole chunks through the sequence kernels,
    the remaining tokens through the single-token kernel, one oracle run over all of them."""
    from wind_rwkv.rwkv7 import attn
    B, H, C, T = 2, 3, 128, 75
    d = inputs.wkv7_inputs(B, T, H, C, seed=61, dtype=torch.bfloat16)
    y_ref, sT_ref = seq_ref.wkv7_seq(*_f64(d, 'qwkvab'))
    flat = [d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab']
    with torch.no_grad():
        y, sT = attn(*flat, C, return_state=True)
    assert y.shape == (B, T, H * C)
    assert seq_ref.rel_err(y.view(B, T, H, C).float().cpu(), y_ref) <= TOL
    assert seq_ref.rel_err(sT.float().cpu(), sT_ref) <= TOL


def test_sequence_in_pieces_matches_one_call():
    """Carrying sT -> s0 across two calls reproduces the single call (state carry of the public wrapper)."""
    from wind_rwkv.rwkv7 import attn
    B, H, C, T = 2, 3, 64, 96
    d = inputs.wkv7_inputs(B, T, H, C, seed=51, dtype=torch.bfloat16)
    flat = {n: d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab'}
    args = lambda sl: [flat[n][:, sl].contiguous() for n in 'qwkvab']
    s0 = torch.zeros(B, H, C, C, device=DEV)
    y_all, s_all = attn(*args(slice(0, T)), C, s0=s0, return_state=True)
    y1, s1 = attn(*args(slice(0, 32)), C, s0=s0, return_state=True)
    y2, s2 = attn(*args(slice(32, T)), C, s0=s1, return_state=True)
    y12 = torch.cat([y1, y2], dim=1)
    assert seq_ref.rel_err(y12.float().cpu(), y_all.float().cpu()) <= 2e-3   # same arithmetic up to chunk phase
    assert seq_ref.rel_err(s2.cpu(), s_all.cpu()) <= 2e-3
