"""The matrix-core WKV7 kernels for head sizes other than 64 (bf16 sequences) against the fp64 oracle.

The reference compiles attn.cu per head size (rwkv7_attn.py:46-51) and has rwkv7_attn_triton_bighead.py:31-322 for
large heads; its tests run head size 64 only (tests/test_attn.py:36).  Gate as for head size 64 (tests/utils.py:18,24
of the reference, restated): normalised L2 error <= 1e-2 on the output, the final state and every gradient against
the fp64 sequential recurrence on the same bf16-rounded inputs.
"""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
TOL_BF16 = 1e-2
DEV = 'cuda'


def run_device(d, state_dtype, backward=True, with_state=True):
    from wind_rwkv.rwkv7.wkv_attn import WindRWKV7, no_state
    xs = [d[n].to(DEV).requires_grad_(backward) for n in ('w', 'q', 'k', 'v', 'a', 'b')]
    s0 = d['s0'].to(state_dtype).to(DEV).requires_grad_(backward) if with_state else no_state(state_dtype, DEV)
    y, sT, _ = WindRWKV7.apply(*xs, s0)
    out = {'y': y, 'sT': sT}
    if backward:
        if with_state:
            torch.autograd.backward([y, sT], [d['dy'].to(DEV), d['dsT'].to(state_dtype).to(DEV)])
            out['ds0'] = s0.grad
        else:
            y.backward(d['dy'].to(DEV))
        out.update(dw=xs[0].grad, dq=xs[1].grad, dk=xs[2].grad, dv=xs[3].grad, da=xs[4].grad, db=xs[5].grad)
    torch.cuda.synchronize()
    return {k: v.detach().float().cpu() for k, v in out.items()}


def run_oracle(c_oracle, d, state_dtype, with_state=True):
    s0 = d['s0'].to(state_dtype) if with_state else torch.zeros_like(d['s0'])
    dsT = d['dsT'].to(state_dtype) if with_state else torch.zeros_like(d['dsT'])
    args = [d[n] for n in 'qwkvab']
    y, sT = c_oracle.forward(*args, s0)
    g = c_oracle.backward(*args, s0, d['dy'], dsT)
    out = {'y': y, 'sT': sT, 'dq': g[0], 'dw': g[1], 'dk': g[2], 'dv': g[3], 'da': g[4], 'db': g[5]}
    if with_state:
        out['ds0'] = g[6]
    return out


def check(got, ref, tol=TOL_BF16):
    errs = {k: seq_ref.rel_err(got[k], ref[k]) for k in ref}
    bad = {k: e for k, e in errs.items() if not e <= tol}
    assert not bad, f'over tolerance {tol}: {bad} (all: {errs})'
    return errs


@pytest.mark.parametrize('C', [16, 32, 48, 80, 96, 112, 128])
@pytest.mark.parametrize('state_dtype', [torch.float32, torch.bfloat16])
def test_head_sizes(c_oracle, C, state_dtype):
    """Every multiple of 16 up to 128 except 64, with an initial state and a gradient on the final state."""
    B, T, H = 2, 64, 3
    d = inputs.wkv7_inputs(B, T, H, C, seed=300 + C, dtype=torch.bfloat16, s0_scale=0.1, dsT_scale=0.1)
    print(f'C={C} {state_dtype}', check(run_device(d, state_dtype), run_oracle(c_oracle, d, state_dtype)), flush=True)


@pytest.mark.parametrize('B,T,H,C', [(1, 16, 1, 128), (3, 272, 5, 96), (1, 2048, 2, 128), (20, 32, 7, 32)])
def test_shapes(c_oracle, B, T, H, C):
    """A single chunk, odd batch and head counts, a long sequence, more (batch, head) pairs than a launch round."""
    d = inputs.wkv7_inputs(B, T, H, C, seed=400 + T + C, dtype=torch.bfloat16, s0_scale=0.1, dsT_scale=0.1)
    check(run_device(d, torch.float32), run_oracle(c_oracle, d, torch.float32))


def test_absent_states_equal_zero_states(c_oracle):
    """No initial state and no gradient on the final state (the usual training call) at C = 128."""
    B, T, H, C = 2, 128, 2, 128
    d = inputs.wkv7_inputs(B, T, H, C, seed=7, dtype=torch.bfloat16)
    check(run_device(d, torch.float32, with_state=False), run_oracle(c_oracle, d, torch.float32, with_state=False))


def test_large_head_at_the_headline_length(c_oracle):
    """C = 128 at B = 8, T = 1024, 768 channels (6 heads): the shape of the reference's headline benchmark with
    the head size doubled."""
    B, T, H, C = 8, 1024, 6, 128
    d = inputs.wkv7_inputs(B, T, H, C, seed=11, dtype=torch.bfloat16)
    print(check(run_device(d, torch.float32, with_state=False), run_oracle(c_oracle, d, torch.float32, with_state=False)), flush=True)


def test_reproducible_and_continues_from_a_state():
    """Two calls agree bit for bit; a sequence run in two pieces through the carried fp32 state equals one run to
    bf16 rounding of the state's use."""
    from wind_rwkv.rwkv7 import attn
    B, T, H, C = 2, 96, 2, 128
    d = inputs.wkv7_inputs(B, T, H, C, seed=5, dtype=torch.bfloat16)
    flat = [d[n].reshape(B, T, H * C).to(DEV) for n in 'qwkvab']
    y1, s1 = attn(*flat, C, return_state=True)
    y2, s2 = attn(*flat, C, return_state=True)
    assert y1.dtype == torch.bfloat16
    assert torch.equal(y1, y2) and torch.equal(s1, s2)
    ya, sa = attn(*[x[:, :48].contiguous() for x in flat], C, return_state=True)
    yb, sb = attn(*[x[:, 48:].contiguous() for x in flat], C, s0=sa, return_state=True)
    assert seq_ref.rel_err(torch.cat([ya, yb], 1).float().cpu(), y1.float().cpu()) <= 5e-3
    assert seq_ref.rel_err(sb.float().cpu(), s1.float().cpu()) <= 5e-3


@pytest.mark.parametrize('C,w_max', [(128, 0.5), (128, 1.5), (48, 1.5)])
def test_strong_decay(c_oracle, C, w_max):
    """Decay inputs up to w_max on whole runs of tokens (decay down to 0.011 per token, 1e-31 over a chunk): the
    chunked form divides by cumulative decays inside a chunk, as at head size 64 (tests/test_gpu_wkv7.py)."""
    B, T, H = 2, 128, 3
    d = inputs.wkv7_inputs(B, T, H, C, seed=77, dtype=torch.bfloat16, s0_scale=0.1, dsT_scale=0.1)
    gen = torch.Generator().manual_seed(78)
    w = torch.rand(B, T, H, C, generator=gen) * (w_max + 6) - 6
    w[:, 16:48] = w_max          # two whole chunks at the strongest decay
    w[:, 60:70, 1] = w_max       # and a run across a chunk boundary in one head
    d['w'] = w.bfloat16()
    check(run_device(d, torch.float32), run_oracle(c_oracle, d, torch.float32))


@pytest.mark.parametrize('C,corr,gate', [(128, 0.5, 0.95), (96, 0.2, 1.0)])
def test_strongly_coupled_tokens(c_oracle, C, corr, gate):
    """Neighbouring tokens with nearly the same removal direction and slow decay: every entry of the triangular
    matrix each chunk inverts is near -gate, the hard regime for the inverse (see the head-size-64 test, same
    coupling and gate: da, db 6.7e-3 and 9.9e-3 here as there, everything else within 4e-3)."""
    B, T, H = 2, 96, 3
    d = inputs.wkv7_inputs(B, T, H, C, seed=91, dtype=torch.bfloat16, s0_scale=0.1, dsT_scale=0.1)
    gen = torch.Generator().manual_seed(92)
    u = torch.randn(B, 1, H, C, generator=gen)
    kk = torch.nn.functional.normalize(u + corr * torch.randn(B, T, H, C, generator=gen), dim=-1)
    d['a'] = (-kk).bfloat16()
    d['b'] = (gate * kk).bfloat16()
    d['w'] = (-4.0 - 2.0 * torch.rand(B, T, H, C, generator=gen)).bfloat16()
    print(check(run_device(d, torch.float32), run_oracle(c_oracle, d, torch.float32)), flush=True)
