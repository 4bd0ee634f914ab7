"""Seeded synthetic inputs for the benchmark configurations.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Everything is drawn on the CPU in fp32 from a torch.Generator seeded per
configuration and then cast, so the oracle and the device see identical bits.
Distributions follow the reference's data builders: tests/test_attn.py:24-30
(r,k,v ~ N(0,1); w = -softplus(N(0,1)) - 0.5; unit-norm kk per head), with the
sign convention of tests/test_time_mixer.py:51 (a = -kk, b = kk*sigmoid(N(0,1))).
"""
import torch

F = torch.nn.functional


def wkv7_inputs(B, T, H, C, seed, dtype=torch.float32, with_dy=True, s0_scale=0.0, dsT_scale=0.0):
    """Returns a dict with q,w,k,v,a,b [B,T,H,C] (dtype), optional dy, s0, dsT (fp32)."""
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32)
    q, k, v = rn(B, T, H, C), rn(B, T, H, C), rn(B, T, H, C)
    w = -F.softplus(-rn(B, T, H, C)) - 0.5
    kk = F.normalize(rn(B, T, H, C), dim=-1)
    a = -kk
    b = kk * torch.sigmoid(rn(B, T, H, C))
    out = {n: t.to(dtype).contiguous() for n, t in dict(q=q, w=w, k=k, v=v, a=a, b=b).items()}
    if with_dy:
        out['dy'] = rn(B, T, H, C).to(dtype).contiguous()
    out['s0'] = (rn(B, H, C, C) * s0_scale).contiguous()
    out['dsT'] = (rn(B, H, C, C) * dsT_scale).contiguous()
    return out


def attn_ln_inputs(B, T, H, C, seed, dtype=torch.float32):
    """wkv7_inputs plus the gate g ~ N(0,1) and params = (1+0.1N, 0.1N, 0.1N) fp32 [3,H*C]."""
    d = wkv7_inputs(B, T, H, C, seed, dtype)
    gen = torch.Generator().manual_seed(seed + 1000)
    rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32)
    d['g'] = rn(B, T, H, C).to(dtype).contiguous()
    ln_w = 1 + 0.1 * rn(H * C)
    ln_b = 0.1 * rn(H * C)
    bonus = 0.1 * rn(H * C)
    d['params'] = torch.stack([ln_w, ln_b, bonus]).contiguous()
    return d


def ddlerp_inputs(B, T, C, D, seed, dtype=torch.float32):
    """x ~ N(0,1)/2 and parameters ~ N(0,1)/2 as tests/test_ddlerp.py:25-28."""
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32) / 2
    return dict(x=rn(B, T, C).to(dtype), alpha=rn(C), L=rn(4 * D, C), R=rn(4, C, D), beta=rn(4, 1, 1, C),
                dy=[(2 * rn(B, T, C)).to(dtype) for _ in range(4)])


def expand_loras_inputs(B, T, C, D, seed, dtype=torch.float32):
    """All inputs ~ N(0,1) as tests/test_expand_loras.py:37-45."""
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32)
    names_btc = ['w_in', 'k_in']
    names_btd = ['z_in', 'a_in', 'ma_in', 'mk_in']
    names_cd = ['Wz', 'Wa', 'Wma', 'Wmk']
    names_c = ['w_bias', 'a_bias', 'ma_bias', 'mk_bias']
    d = {}
    for n in names_btc:
        d[n] = rn(B, T, C).to(dtype)
    for n in names_btd:
        d[n] = rn(B, T, D).to(dtype)
    for n in names_cd:
        d[n] = rn(C, D).to(dtype)
    for n in names_c:
        d[n] = rn(C).to(dtype)
    d['dy'] = [rn(B, T, C).to(dtype) for _ in range(4)]
    return d


# The five benchmark configurations (name -> builder).  Sizes are the full ones;
# tests pass smaller B/T where the oracle would take too long.
CONFIGS = {
    'cfg0': dict(kind='wkv7', B=1, T=256, H=4, C=64, seed=0, dtype=torch.float32, backward=False),
    'cfg1': dict(kind='wkv7', B=8, T=1024, H=12, C=64, seed=1, dtype=torch.bfloat16, backward=True),
    'cfg2': dict(kind='attn_ln', B=8, T=1024, H=12, C=64, seed=2, dtype=torch.bfloat16, backward=True),
    'cfg3': dict(kind='wkv7', B=1, T=16384, H=32, C=64, seed=3, dtype=torch.bfloat16, backward=True, s0_scale=0.1),
    'cfg4': dict(kind='time_mixer', B=8, T=1024, H=12, C=64, seed=4, dtype=torch.bfloat16, backward=True),
}
