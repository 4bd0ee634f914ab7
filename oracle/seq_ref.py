"""Sequential (token-by-token) restatements of the reference's spec functions.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Every function here follows one of the reference's own ground-truth functions
(the ones its test scripts compare the kernels against) and runs in whatever
dtype it is handed; the tests hand it fp64.  Gradients come from torch.autograd
on these loops.

Pinning (independent checks live in tests/test_oracle_*.py):
  wkv7_seq          closed forms with a=b=0 (decayed linear attention, and
                    tril(QK^T)V when additionally decay=1), brute-force
                    explicit products at T<=4, sequence-split consistency
                    (pins s0/sT), linearity in v and q, finite-difference
                    gradcheck, and the C oracle's hand-derived reverse pass.
  attn_ln_epilogue  torch.nn.functional.group_norm (library routine) and the
                    special case ln_w=1, ln_b=0, bonus=0, g=1.
  ddlerp_seq        special cases R=0 / L=0 (y_k = x + xx*beta_k), the t=0 row
                    (xx=-x), and an explicit per-token loop.
  expand_loras_seq  unit norm of kk per head, b=-kk*a, zero LoRA inputs give
                    sigmoid(bias), softplus/normalize library routines.
  time_mixer_seq    composition of the above; compared against the module
                    wiring in the package at fp64 on CPU-free parts only.
"""
import math

import torch

F = torch.nn.functional

LN_EPS = 64e-5  # reference: wind_rwkv/rwkv7/time_mixer.py:104, attn_ln.cu:22


def wkv7_seq(q, w, k, v, a, b, s0=None):
    """RWKV-7 state recurrence, one token at a time.

    Follows tests/test_attn.py:6-18 (same loop at time_mixer.py:6-16,
    tests/test_attn_ln.py:6-17, tests/test_time_mixer.py:14-24), extended with
    an initial state and a returned final state as the autograd Function of
    rwkv7_attn.py:20-29 has them.

    q,w,k,v,a,b: [B,T,H,C];  w is the log-log decay (decay = exp(-exp(w))).
    s0: [B,H,C,C] indexed [value i, key j] or None for zeros.
    Returns y [B,T,H,C] and sT [B,H,C,C] in the dtype of the inputs.
    """
    B, T, H, C = q.shape
    decay = torch.exp(-torch.exp(w))
    state = q.new_zeros(B, H, C, C) if s0 is None else s0
    ys = []
    for t in range(T):
        qt, kt, vt, at, bt, dt = (x[:, t] for x in (q, k, v, a, b, decay))
        sa = torch.einsum('bhij,bhj->bhi', state, at)
        state = (state * dt[:, :, None, :]
                 + sa[:, :, :, None] * bt[:, :, None, :]
                 + vt[:, :, :, None] * kt[:, :, None, :])
        ys.append(torch.einsum('bhij,bhj->bhi', state, qt))
    return torch.stack(ys, dim=1), state


def attn_ln_epilogue(y, q, k, v, g, params):
    """Per-head GroupNorm + bonus term + gate on a WKV7 output.

    Follows tests/test_attn_ln.py:18-21 (model statement time_mixer.py:154-157;
    kernel attn_ln.cu:11-37).  y,q,k,v,g: [B,T,H,C]; params: [3,H*C] stacked
    (ln_weight, ln_bias, bonus).  Biased variance, eps = 64e-5.
    """
    B, T, H, C = y.shape
    ln_w, ln_b, bonus = params[0], params[1], params[2]
    mean = y.mean(dim=-1, keepdim=True)
    var = ((y - mean) ** 2).mean(dim=-1, keepdim=True)
    yn = (y - mean) / torch.sqrt(var + LN_EPS)
    yn = yn * ln_w.view(H, C) + ln_b.view(H, C)
    dot = (q * k * bonus.view(H, C)).sum(dim=-1, keepdim=True)
    return (yn + dot * v) * g


def attn_ln_seq(q, w, k, v, a, b, g, params, s0=None, wkv7=None):
    """WKV7 followed by the epilogue; returns (out, sT).  tests/test_attn_ln.py:6-21.
    ``wkv7``: another restatement of the recurrence with wkv7_seq's signature (the C one, for full-size runs)."""
    y, sT = (wkv7 or wkv7_seq)(q, w, k, v, a, b, s0)
    return attn_ln_epilogue(y, q, k, v, g, params), sT


def token_shift(x):
    """x[t-1] with a zero row at t=0  (F.pad(x,(0,0,1,-1)), tests/test_ddlerp.py:9)."""
    return torch.cat([torch.zeros_like(x[:, :1]), x[:, :-1]], dim=1)


def ddlerp_seq(x, alpha, L, R, beta):
    """Data-dependent token-shift lerp.  Follows tests/test_ddlerp.py:5-13.

    x [B,T,C]; alpha [C]; L [4D,C]; R [4,C,D]; beta [4,1,1,C].
    Returns a [4,B,T,C] tensor (the reference returns its four slices).
    """
    B, T, C = x.shape
    D = R.shape[2]
    xx = token_shift(x) - x
    mixed = x + xx * alpha
    mid = torch.tanh(mixed @ L.t()).view(B, T, 4, D)
    c = torch.einsum('btkd,kcd->kbtc', mid, R) + beta
    return x[None] + xx[None] * c


def expand_loras_seq(w_in, k_in, z_in, a_in, ma_in, mk_in, Wz, Wa, Wma, Wmk,
                     w_bias, a_bias, ma_bias, mk_bias, head_size):
    """Second halves of the four rank-D LoRAs and the elementwise tail.

    Follows tests/test_expand_loras.py:6-19 (model statement time_mixer.py:137-147).
    Returns (w_out, k_out, kk_out, b_out), each [B,T,C].
    """
    B, T, C = w_in.shape
    w_out = -F.softplus(-(w_bias + w_in)) - 0.5
    z = k_in + torch.tanh(z_in) @ Wz.t()
    zh = z.view(B, T, C // head_size, head_size)
    kk = (zh / zh.norm(dim=-1, keepdim=True).clamp_min(1e-12)).view(B, T, C)
    a = torch.sigmoid(a_bias + a_in @ Wa.t())
    ma = torch.sigmoid(ma_bias + ma_in @ Wma.t())
    mk = torch.sigmoid(mk_bias + mk_in @ Wmk.t())
    k_mix = k_in * ma + k_in * a * (1 - ma)
    k_out = k_mix * torch.exp(w_out * mk)
    return w_out, k_out, kk, -kk * a


def bf16_ste(t):
    """Round to bfloat16 in the forward pass, identity in the backward pass (straight-through)."""
    return t + (t.to(torch.bfloat16).to(t.dtype) - t).detach()


class _Bf16Boundary(torch.autograd.Function):
    """A bf16 tensor handed from one stage to the next: the value is rounded to bfloat16 on the way
    forward and its gradient is rounded to bfloat16 on the way back, as happens to every activation (not to
    parameters) that crosses a kernel or matmul boundary of the real pipeline."""

    @staticmethod
    def forward(ctx, t):
        return t.to(torch.bfloat16).to(t.dtype)

    @staticmethod
    def backward(ctx, g):
        return g.to(torch.bfloat16).to(g.dtype)


def bf16_boundary(t):
    return _Bf16Boundary.apply(t)


def time_mixer_seq(p, x, n_head, stage=None, weight=None, wkv7=None):
    """Whole RWKV-7 time-mixer block forward.

    Follows RefTimeMixer.forward, tests/test_time_mixer.py:26-55, with the package's sign convention
    (a = kk, b = -kk*a_gate, time_mixer.py:147,150), which gives the same a b^T product as the test's
    (-kk, kk*a_gate).  p: dict of parameters with the reference's names (time_mixer.py:42-104);
    x: [B,T,C].  Returns [B,T,C].

    ``stage`` (default: identity) is applied to every activation that crosses a stage boundary of the real
    pipeline (time_mixer.py:106-167 hands bf16 tensors from each kernel or matmul to the next) and
    ``weight`` to every parameter (cast to bf16 on use; its gradient stays fp32).  Passing
    ``bf16_boundary`` / ``bf16_ste`` gives the block as the bf16 pipeline defines it, exact inside each
    stage, which separates the kernels' own arithmetic error from the rounding the interface imposes.
    """
    st = stage if stage is not None else (lambda t: t)
    wt = weight if weight is not None else (lambda t: t)
    B, T, C = x.shape
    H = n_head
    N = C // H
    W = lambda name: wt(p[name])                      # weights as the stage sees them
    mm = lambda a, w: st(a @ w.t())                   # a bf16 matmul: rounded output
    y4 = st(ddlerp_seq(x, W('time_maa_x'), W('time_maa_w1'), W('time_maa_w2'), W('time_maa')))
    xrg, xwa, xk, xv = y4[0], y4[1], y4[2], y4[3]
    r = mm(xrg, W('Wr'))
    k = mm(xk, W('Wk'))
    v = mm(xv, W('Wv'))
    g = mm(st(torch.tanh(mm(xrg, W('gate_w1')))), W('gate_w2'))
    w2 = mm(st(torch.tanh(mm(xwa, W('time_decay_w1')))), W('time_decay_w2'))
    w, k2, kk, bb = expand_loras_seq(
        w2, k, mm(xk, W('time_kkk_w1')), mm(xwa, W('time_aaa_w1')),
        mm(xwa, W('ma_w1')), mm(xk, W('mk_w1')),
        W('time_kkk_w2'), W('time_aaa_w2'), W('ma_w2'), W('mk_w2'),
        W('time_decay'), W('time_aaaaa'), W('time_misc_a'), W('time_misc_k'), N)
    w, k2, kk, bb = st(w), st(k2), st(kk), st(bb)
    view = lambda t: t.reshape(B, T, H, N)
    params = torch.stack([p['ln_x.weight'], p['ln_x.bias'], p['time_faaaa']])
    out, _ = attn_ln_seq(view(r), view(w), view(k2), view(v), view(kk), view(bb), view(g), params, wkv7=wkv7)
    return mm(st(out).reshape(B, T, C), W('Wo'))


def naive_recurrence_fp32(q, w, k, v, a, b, head_size):
    """The reference's naive PyTorch recurrence, as it would run on a CPU.

    This is the loop of time_mixer.py:6-16 ("ref_attn") restated: fp32, zero
    initial state, [B,T,H*C] in and out.  Used only as the timed CPU baseline.
    """
    B, T, HC = q.shape
    H = HC // head_size
    q, w, k, v, a, b = (x.view(B, T, H, head_size) for x in (q, w, k, v, a, b))
    state = torch.zeros(B, H, head_size, head_size, dtype=q.dtype)
    decay = torch.exp(-torch.exp(w))
    y = torch.empty_like(v)
    for t in range(T):
        state = (state * decay[:, t, :, None, :]
                 + (state @ a[:, t, :, :, None]) * b[:, t, :, None, :]
                 + v[:, t, :, :, None] * k[:, t, :, None, :])
        y[:, t] = (state @ q[:, t, :, :, None]).squeeze(-1)
    return y.view(B, T, HC)


def rel_err(x, ref):
    """||x-ref||_2 / max(||ref||_2, 1e-30)  — the reference's metric, tests/utils.py:24."""
    x = x.double().flatten()
    ref = ref.double().flatten()
    return float((x - ref).norm() / max(float(ref.norm()), 1e-30))
