"""Chunked restatement of WKV7 forward and backward: the executable spec of the device kernels.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The algebra is the chunked form the reference's kernels use
(rwkv7_attn_triton.py:27-69 forward, :72-156 backward; attn.cu:48-101, 177-321),
re-organised into the three phases the device code runs:

  forward   prepare (per chunk, no state)  ->  state scan (sequential, light)  ->  output (per chunk)
  backward  prepare (per chunk, no dstate) ->  dstate scan (reverse)           ->  gradients (per chunk)

With ``rounding='none'`` everything runs in the dtype of the inputs (fp64 in the
tests) and must agree with oracle.seq_ref.wkv7_seq and its autograd gradients to
rounding error; that pins every formula here, including the closed form used for
the decay gradient.  With ``rounding='bf16'`` each matrix-product operand is
rounded to bfloat16 exactly where the device rounds it, which predicts the
device's error against the fp64 oracle.

Notation (per batch b, head h, chunk c; K tokens per chunk, C channels):
  lw   = -exp(w)                 log of the per-step decay            [K,C]
  Lc   = cumsum(lw) (inclusive)  cumulative log decay, kept in full precision
  P    = exp(Lc), Px = exp(Lc-lw), Pi = exp(-Lc), E = exp(Lc[-1]-Lc), fw = exp(Lc[-1])
  wq=q*P  wa=a*Px  kwi=k*Pi  bwi=b*Pi  kf=k*E  bf=b*E
  state S[i,j] (value i, key j)
"""
import torch


def _rounder(rounding):
    if rounding == 'none':
        return lambda x: x
    if rounding == 'bf16':
        return lambda x: x.to(torch.bfloat16).to(x.dtype)
    raise ValueError(rounding)


def _chunks(x, K):
    """[B,T,H,C] -> [B,H,NC,K,C]"""
    B, T, H, C = x.shape
    return x.view(B, T // K, K, H, C).permute(0, 3, 1, 2, 4).contiguous()


def _unchunk(x):
    """[B,H,NC,K,C] -> [B,T,H,C]"""
    B, H, NC, K, C = x.shape
    return x.permute(0, 2, 3, 1, 4).reshape(B, NC * K, H, C)


def _decays(w, K):
    lw = -torch.exp(w)
    Lc = torch.cumsum(lw, dim=-2)
    Ltot = Lc[..., -1:, :]
    return dict(lw=lw, P=torch.exp(Lc), Px=torch.exp(Lc - lw), Pi=torch.exp(-Lc),
                E=torch.exp(Ltot - Lc), fw=torch.exp(Ltot))


def neumann_inverse(X, rnd):
    """inv(I - X) for strictly lower-triangular 16x16 X as (I+X)(I+X^2)(I+X^4)(I+X^8).

    Exact because X^16 = 0.  ``rnd`` is applied to both operands of every product,
    as a matrix unit with rounded inputs would.
    """
    n = X.shape[-1]
    eye = torch.eye(n, dtype=X.dtype, device=X.device).expand_as(X)
    Tm = eye + X
    Xp = X
    steps = 0
    p = 1
    while p * 2 < n:
        Xp = rnd(Xp) @ rnd(Xp)
        Tm = Tm + rnd(Tm) @ rnd(Xp)
        p *= 2
        steps += 1
    return Tm


def _masks(K, like):
    idx = torch.arange(K, device=like.device)
    strict = (idx[:, None] > idx[None, :]).to(like.dtype)
    incl = (idx[:, None] >= idx[None, :]).to(like.dtype)
    return strict, incl


def forward(q, w, k, v, a, b, s0, K=16, rounding='none', inverse='solve'):
    """Returns y [B,T,H,C], sT [B,H,C,C] and a dict of saved intermediates.

    inverse: 'solve' (exact triangular solve) or 'neumann' (the doubling product).
    """
    rnd = _rounder(rounding)
    q, w, k, v, a, b = (_chunks(x, K) for x in (q, w, k, v, a, b))
    B, H, NC, _, C = q.shape
    d = _decays(w, K)
    strict, incl = _masks(K, q)
    mT = lambda x: x.transpose(-1, -2)

    # ---- phase 1: per-chunk prepare (no state) ----
    wa, kwi, bwi = rnd(a * d['Px']), rnd(k * d['Pi']), rnd(b * d['Pi'])
    kf, bf = rnd(k * d['E']), rnd(b * d['E'])
    vr = rnd(v)
    AB = (wa @ mT(bwi)) * strict
    AK = (wa @ mT(kwi)) * strict
    eye = torch.eye(K, dtype=q.dtype).expand_as(AB)
    if inverse == 'solve':
        Tinv = torch.linalg.solve_triangular(eye - AB, eye.clone(), upper=False)
    else:
        Tinv = neumann_inverse(AB, lambda x: x)  # device does this product chain in fp32
    Tinv_r = rnd(Tinv)
    R = rnd(AK) @ vr                      # [K, C(i)]
    Ut = Tinv_r @ rnd(R)                  # state-free part of U
    Wm = rnd(Tinv_r @ wa)                 # [K, C(j)]

    # ---- phase 2: sequential state scan ----
    S = s0.to(q.dtype).clone()            # [B,H,C,C]
    ckpt = []
    Us = []
    for c in range(NC):
        Sb = rnd(S)
        ckpt.append(Sb)
        U = rnd(Ut[:, :, c] + Wm[:, :, c] @ mT(Sb))       # [K, C(i)]
        Us.append(U)
        S = S * d['fw'][:, :, c] + mT(vr[:, :, c]) @ kf[:, :, c] + mT(U) @ bf[:, :, c]
    sT = S
    ckpt = torch.stack(ckpt, dim=2)       # [B,H,NC,C,C]
    U = torch.stack(Us, dim=2)            # [B,H,NC,K,C]

    # ---- phase 3: per-chunk output ----
    wq = rnd(q * d['P'])
    QK = rnd((wq @ mT(kwi)) * incl)
    QB = rnd((wq @ mT(bwi)) * incl)
    Y = QK @ vr + QB @ U + wq @ mT(ckpt)
    saved = dict(ckpt=ckpt, U=U, Tinv=Tinv, Wm=Wm, Ut=Ut, kf=kf, bf=bf)
    return _unchunk(Y), sT, saved


def backward(q, w, k, v, a, b, dy, dsT, saved, K=16, rounding='none', inverse='solve'):
    """Returns dq,dw,dk,dv,da,db [B,T,H,C] and ds0 [B,H,C,C]."""
    rnd = _rounder(rounding)
    q, w, k, v, a, b, dy = (_chunks(x, K) for x in (q, w, k, v, a, b, dy))
    B, H, NC, _, C = q.shape
    d = _decays(w, K)
    strict, incl = _masks(K, q)
    mT = lambda x: x.transpose(-1, -2)
    S0, U = saved['ckpt'], saved['U']

    wq, wa = rnd(q * d['P']), rnd(a * d['Px'])
    kwi, bwi = rnd(k * d['Pi']), rnd(b * d['Pi'])
    kf32, bf32 = k * d['E'], b * d['E']
    kf, bf = rnd(kf32), rnd(bf32)
    vr, dyr = rnd(v), rnd(dy)
    AB = (wa @ mT(bwi)) * strict
    AK = rnd((wa @ mT(kwi)) * strict)
    QK = rnd((wq @ mT(kwi)) * incl)
    QB = rnd((wq @ mT(bwi)) * incl)
    eye = torch.eye(K, dtype=q.dtype).expand_as(AB)
    if inverse == 'solve':
        Tinv = torch.linalg.solve_triangular(eye - AB, eye.clone(), upper=False)
    else:
        Tinv = neumann_inverse(AB, lambda x: x)
    TinvT = rnd(mT(Tinv))

    # ---- phase 1: per-chunk prepare (no dstate) ----
    Ee = rnd(mT(QB) @ dyr)                # QB^T dY            [K, C(i)]
    Dt = TinvT @ Ee                       # state-free part of dab_u
    Bm = rnd(TinvT @ bf)                  # [K, C(j)]

    # ---- phase 2: reverse dstate scan ----
    dS = dsT.to(q.dtype).clone()
    dSs = [None] * NC
    dabus = [None] * NC
    for c in range(NC - 1, -1, -1):
        dSb = rnd(dS)
        dSs[c] = dSb
        dab_u = rnd(Dt[:, :, c] + Bm[:, :, c] @ mT(dSb))            # [K, C(i)]
        dabus[c] = dab_u
        dS = dS * d['fw'][:, :, c] + mT(dyr[:, :, c]) @ wq[:, :, c] + mT(dab_u) @ wa[:, :, c]
    ds0 = dS
    dSc = torch.stack(dSs, dim=2)         # gradient arriving at each chunk's end state
    dab_u = torch.stack(dabus, dim=2)

    # ---- phase 3: per-chunk gradients ----
    dv = mT(QK) @ dyr + kf @ mT(dSc) + mT(AK) @ dab_u
    dab = rnd((dab_u @ mT(U)) * strict)
    dak = rnd((dab_u @ mT(vr)) * strict)
    dqb = rnd((dyr @ mT(U)) * incl)
    dqk = rnd((dyr @ mT(vr)) * incl)
    UdS = U @ dSc                         # [K, C(j)]
    VdS = vr @ dSc
    Ba = dab @ bwi + dak @ kwi + dab_u @ S0
    Bq = dqb @ bwi + dqk @ kwi + dyr @ S0
    Bb = mT(dab) @ wa + mT(dqb) @ wq + d['fw'] * UdS
    Bk = mT(dak) @ wa + mT(dqk) @ wq + d['fw'] * VdS
    da = d['Px'] * Ba
    dq = d['P'] * Bq
    db = d['Pi'] * Bb
    dk = d['Pi'] * Bk
    # decay gradient: dlogw_k = sum_{t>=k}(wq*Bq - kwi*Bk - bwi*Bb) + sum_{t>k} wa*Ba + sum_i S'[i,:]*dS[i,:]
    # with sum_i S'*dS = fw*sum_i S0*dS + sum_t (kf*VdS + bf*UdS); every product uses the same
    # rounded multipliers as the brackets so that the pairs inside [k,K) cancel exactly.
    g_incl = wq * Bq - kwi * Bk - bwi * Bb
    g_strict = wa * Ba
    const = (d['fw'] * (S0 * dSc).sum(dim=-2, keepdim=True)
             + ((kwi * d['fw']) * VdS + (bwi * d['fw']) * UdS).sum(dim=-2, keepdim=True))
    suffix_incl = torch.flip(torch.cumsum(torch.flip(g_incl, [-2]), dim=-2), [-2])
    suffix_strict = torch.flip(torch.cumsum(torch.flip(g_strict, [-2]), dim=-2), [-2]) - g_strict
    dlogw = suffix_incl + suffix_strict + const
    dw = dlogw * d['lw']                  # d decay_log / d w = -exp(w) = lw
    return tuple(_unchunk(x) for x in (dq, dw, dk, dv, da, db)) + (ds0,)
