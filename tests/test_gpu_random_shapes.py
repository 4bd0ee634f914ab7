"""Seeded random shapes through every kernel family, each case against the fp64 oracle at the 1e-2 gate of the
reference's scripts (tests/utils.py:18).  The fixed-shape tests pick their sizes to hit known code paths (segment
counts, helper blocks, tiles per block); these draw B, T, H, C, the LoRA rank, the state dtype and the scale of
the carried state at random, so that a path nobody thought of still gets exercised.  The forward that keeps
nothing for backward is checked on the same cases: bit-identical to the training forward."""
import random

import pytest
import torch

from oracle import inputs, seq_ref

import test_gpu_ddlerp as dd
import test_gpu_expand_loras as el
import test_gpu_wkv7 as wkv

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _wkv_cases(n, seed):
    rng = random.Random(seed)
    for _ in range(n):
        kind = rng.choice(['small', 'small', 'long', 'wide'])
        if kind == 'small':
            B, T, H = rng.randint(1, 5), 16 * rng.randint(1, 30), rng.randint(1, 7)
        elif kind == 'long':       # few (batch, head) pairs: the segmented scan
            B, T, H = 1, 16 * rng.randint(100, 600), rng.randint(1, 3)
        else:                      # many pairs, short sequences
            B, T, H = rng.randint(6, 30), 16 * rng.randint(1, 6), rng.randint(8, 14)
        yield (B, T, H, rng.choice([torch.float32, torch.bfloat16]), rng.choice([0, 0.1, 0.5]), rng.choice([0, 0.1, 0.5]),
               rng.randint(0, 10**6))


@pytest.mark.parametrize('B,T,H,state_dtype,s0s,dsTs,seed', list(_wkv_cases(40, 2024)))
def test_wkv7_random_shape(c_oracle, B, T, H, state_dtype, s0s, dsTs, seed):
    from wind_rwkv.rwkv7 import attn
    d = inputs.wkv7_inputs(B, T, H, 64, seed=seed, dtype=torch.bfloat16, s0_scale=s0s, dsT_scale=dsTs)
    got = wkv.run_device(d, state_dtype)
    wkv.check(got, wkv.run_oracle(c_oracle, d, state_dtype))
    x = [d[n].reshape(B, T, H * 64).to(DEV) for n in ('q', 'w', 'k', 'v', 'a', 'b')]
    with torch.no_grad():
        y, sT = attn(*x, 64, s0=d['s0'].to(state_dtype).to(DEV), return_state=True)
    torch.cuda.synchronize()
    assert torch.equal(y.float().cpu().view(B, T, H, 64), got['y']) and torch.equal(sT.float().cpu(), got['sT'])


def _head_size_cases(n, seed):
    rng = random.Random(seed)
    for _ in range(n):
        C = rng.choice([16, 32, 48, 80, 96, 112, 128])
        kind = rng.choice(['small', 'small', 'long', 'wide'])
        if kind == 'small':
            B, T, H = rng.randint(1, 5), 16 * rng.randint(1, 30), rng.randint(1, 5)
        elif kind == 'long':
            B, T, H = 1, 16 * rng.randint(60, 200), rng.randint(1, 2)
        else:
            B, T, H = rng.randint(6, 20), 16 * rng.randint(1, 4), rng.randint(4, 9)
        yield (B, T, H, C, rng.choice([torch.float32, torch.bfloat16]), rng.choice([0, 0.1, 0.5]), rng.choice([0, 0.1, 0.5]),
               rng.randint(0, 10**6))


@pytest.mark.parametrize('B,T,H,C,state_dtype,s0s,dsTs,seed', list(_head_size_cases(24, 2027)))
def test_wkv7_random_shape_other_head_sizes(c_oracle, B, T, H, C, state_dtype, s0s, dsTs, seed):
    """The matrix-core kernels of the head sizes other than 64, and their forward without autograd."""
    from wind_rwkv.rwkv7 import attn
    d = inputs.wkv7_inputs(B, T, H, C, seed=seed, dtype=torch.bfloat16, s0_scale=s0s, dsT_scale=dsTs)
    got = wkv.run_device(d, state_dtype)
    wkv.check(got, wkv.run_oracle(c_oracle, d, state_dtype))
    x = [d[n].reshape(B, T, H * C).to(DEV) for n in ('q', 'w', 'k', 'v', 'a', 'b')]
    with torch.no_grad():
        y, sT = attn(*x, C, s0=d['s0'].to(state_dtype).to(DEV), return_state=True)
    torch.cuda.synchronize()
    assert torch.equal(y.float().cpu().view(B, T, H, C), got['y']) and torch.equal(sT.float().cpu(), got['sT'])


def _channel_cases(n, seed):
    rng = random.Random(seed)
    for _ in range(n):
        B, T = rng.randint(1, 9), 16 * rng.randint(1, 70)
        C = 64 * rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 24, 32])
        if B * T * C > 6e6:        # keeps the oracle's share of a case under a second
            T = 16 * max(1, int(6e6 / (B * C)) // 16)
        yield B, T, C, rng.choice([16, 32, 64]), rng.randint(0, 10**6), rng.choice([n for n in (16, 32, 64, 64, 128) if C % n == 0])


@pytest.mark.parametrize('B,T,C,D,seed,N', list(_channel_cases(25, 2025)))
def test_ddlerp_and_expand_loras_random_shape(B, T, C, D, seed, N):
    dd.check(*dd.run_both(B, T, C, 64 if D == 64 else 32, seed))   # ddlerp has ranks 32 and 64
    el.check(*el.run_both(B, T, C, D, seed, scale=0.5, head_size=N))


def _attn_ln_cases(n, seed):
    rng = random.Random(seed)
    for _ in range(n):
        if rng.random() < 0.3:     # few pairs, long: the segmented scans under the fused epilogue
            B, T, H = 1, 16 * rng.randint(100, 400), rng.randint(1, 3)
        else:
            B, T, H = rng.randint(1, 6), 16 * rng.randint(1, 24), rng.randint(1, 13)
        yield B, T, H, rng.choice([torch.float32, torch.bfloat16]), rng.choice([0.5, 1.0]), rng.randint(0, 10**6)


@pytest.mark.parametrize('B,T,H,state_dtype,s0s,seed', list(_attn_ln_cases(20, 2026)))
def test_attn_ln_random_shape(c_oracle, B, T, H, state_dtype, s0s, seed):
    """A generic carried state of scale 0.5 or 1 throughout: the gradient of the initial state is dominated by the
    first tokens, whose GroupNorm is ill-conditioned when the state is small against (k.q) v - its error against the
    oracle goes as 1/scale (measured 3e-3 at scale 1, 5e-3 at 0.5, 1.2e-2 to 2e-2 at 0.1, for any T and either state
    dtype; every other tensor is unaffected), which is a property of the bf16 operands, not of the kernels."""
    import test_gpu_attn_ln as ln
    d = inputs.attn_ln_inputs(B, T, H, 64, seed=seed, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(seed + 1)
    d['s0'] = torch.randn(B, H, 64, 64, generator=gen) * s0s
    d['dsT'] = torch.randn(B, H, 64, 64, generator=gen) * 0.1
    ln.check(ln.device(d, state_dtype), ln.oracle(c_oracle, d, state_dtype))


def _block_cases(n, seed):
    rng = random.Random(seed)
    for _ in range(n):
        H = rng.choice([2, 4, 6, 8])
        B = rng.randint(1, 3)
        yield B, 16 * rng.randint(-(-16 // B), 24), 64 * H, H, rng.randint(0, 10**6)     # at least 256 tokens


@pytest.mark.parametrize('B,T,C,H,seed', list(_block_cases(6, 2027)))
def test_time_mixer_random_shape(B, T, C, H, seed):
    """The whole block, output and every gradient, against the oracle that rounds where the bf16 interface rounds,
    at the per-tensor gates of tests/test_gpu_time_mixer.py (1e-2, or 1.2 x the worst measured value where that is
    larger: the two LoRA matrices in front of the normalised key are the worst-conditioned tensors of the block - their
    gradient passes the normalisation's backward, a difference of nearly equal bf16-rounded terms)."""
    import test_gpu_time_mixer as tm
    got, ref = tm.run_block(B, T, seed=seed, C=C, H=H, stage=seq_ref.bf16_boundary)
    errs = {k: seq_ref.rel_err(got[k], ref[k]) for k in ref}
    bad = {k: e for k, e in errs.items() if not e <= tm.gate(k)}
    assert not bad, f'over tolerance: {bad}'


def _f32_cases(n, seed):
    rng = random.Random(seed)
    for _ in range(n):
        C = 16 * rng.randint(1, 8)
        kind = rng.choice(['small', 'small', 'long', 'many'])
        if kind == 'small':
            B, T, H = rng.randint(1, 4), 16 * rng.randint(1, 12), rng.randint(1, 6)
        elif kind == 'long':
            B, T, H = 1, 16 * rng.randint(40, 120), rng.randint(1, 2)
        else:                      # more (batch, head) pairs than a quarter / half of the compute units
            B, T, H = rng.randint(9, 40), 16 * rng.randint(1, 3), rng.randint(4, 8)
        yield B, T, H, C, rng.choice([0, 0.1, 0.5]), rng.choice([0, 0.5]), rng.randint(0, 10**6)


@pytest.mark.parametrize('B,T,H,C,s0s,dsTs,seed', list(_f32_cases(20, 2028)))
def test_wkv7_f32_random_shape(c_oracle, B, T, H, C, s0s, dsTs, seed):
    """The fp32 kernels (float32 tensors) at every head size, at their own gate of 1e-4."""
    from wind_rwkv.rwkv7 import WindRWKV7F32
    d = inputs.wkv7_inputs(B, T, H, C, seed=seed, dtype=torch.float32, s0_scale=s0s, dsT_scale=dsTs)
    args = [d[n] for n in 'qwkvab']
    y_ref, sT_ref = c_oracle.forward(*args, d['s0'])
    ref = dict(zip(['dq', 'dw', 'dk', 'dv', 'da', 'db', 'ds0'], c_oracle.backward(*args, d['s0'], d['dy'], d['dsT'])))
    xs = [d[n].to(DEV).requires_grad_() for n in 'wqkvab']
    s0 = d['s0'].to(DEV).requires_grad_()
    y, sT, _ = WindRWKV7F32.apply(*xs, s0)
    torch.autograd.backward([y, sT], [d['dy'].to(DEV), d['dsT'].to(DEV)])
    torch.cuda.synchronize()
    assert seq_ref.rel_err(y.detach().cpu(), y_ref) <= 1e-4 and seq_ref.rel_err(sT.detach().cpu(), sT_ref) <= 1e-4
    for n, x in zip('wqkvab', xs):
        assert seq_ref.rel_err(x.grad.cpu(), ref['d' + n]) <= 1e-4, n
    assert seq_ref.rel_err(s0.grad.cpu(), ref['ds0']) <= 1e-4
