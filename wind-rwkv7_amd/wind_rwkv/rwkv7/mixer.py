"""RWKV-7 time-mixer block wired onto the HIP kernels.

Mirrors the reference's ``TimeMixer`` (time_mixer.py:18-167): same constructor signature, same parameter
names and shapes (so a state dict moves over unchanged), same forward contract
(``x [B,T,C]`` of any float dtype -> ``[B,T,C]`` bf16).  The projections (:120-131, :167) are bf16 matmuls: the
product and its input gradient go to the BLAS library as in the reference, the weight gradient to this
package's kernel (linear.py); everything else runs in this package's kernels:

    ddlerp -> r, k, v, gate and LoRA first halves (matmuls) -> expand_loras -> attn_ln -> output matmul

The constructor switches keep their names.  ``use_triton_ddlerp`` / ``use_triton_loras`` select the fused
kernels (True, default) or the plain PyTorch expressions of the reference (:113-118, :136-147);
``attn_impl`` is 'cuda' (fused attn_ln kernel, default), 'triton' (WKV7 kernel followed by PyTorch
GroupNorm / bonus / gate, :158-163) or 'ref' (the token-by-token recurrence in PyTorch, :151-157).

Beyond the reference, for inference: ``forward(x, state=..., return_state=True)`` carries (last token, WKV7 state)
from one piece of a sequence to the next, and ``step(x_t, state)`` advances one token per sequence.
"""
import ctypes
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import _native
from .linear import bf16_copies, projection, projection_sets, split_columns
from .loras import expand_loras
from .token_shift import ddlerp
from .wkv_attn import _attn_bf16_head, _bf16_head, attn_triton, load_attn
from .wkv_attn_ln import attn_ln, attn_ln_step, group_norm_heads, load_attn_ln

LORA_RANKS = dict(mix=32, decay=64, aaa=16, kkk=16, gate=128, ma=16, mk=16)  # time_mixer.py:69-94


def ref_attn(q, w, k, v, a, b, HEAD_SIZE):
    """Token-by-token WKV7 in PyTorch (time_mixer.py:6-16): the slow reference path of attn_impl='ref'."""
    B, T, HC = q.shape
    H, C = HC // HEAD_SIZE, HEAD_SIZE
    q, w, k, v, a, b = (t.view(B, T, H, C) for t in (q, w, k, v, a, b))
    state = torch.zeros(B, H, C, C, device=q.device, dtype=q.dtype)
    decay = torch.exp(-torch.exp(w))
    out = []
    for t in range(T):
        sa = state @ a[:, t, :, :, None]
        state = state * decay[:, t, :, None, :] + sa * b[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :]
        out.append((state @ q[:, t, :, :, None]).squeeze(-1))
    return torch.stack(out, dim=1).reshape(B, T, HC)


def _orthogonal(rows, cols, scale, batch=None):
    """Orthogonal init with gain sqrt(rows/cols) when rows > cols, times `scale` (time_mixer.py:57-67)."""
    gain = scale * (math.sqrt(rows / cols) if rows > cols else 1.0)
    shape = (rows, cols) if batch is None else (batch, rows, cols)
    t = torch.zeros(shape)
    for m in (t.unbind(0) if batch is not None else [t]):
        nn.init.orthogonal_(m, gain=gain)
    return t


class TimeMixer(nn.Module):
    def __init__(self, args, layer_id, use_triton_ddlerp=True, use_triton_loras=True, attn_impl='cuda',
                 triton_dot_prec='fp32'):
        super().__init__()
        assert attn_impl in ('cuda', 'ref', 'triton')
        self.args = args
        self.layer_id = layer_id
        self.n_embd = C = args.n_embd
        self.dim_att = C
        self.n_head = H = args.n_head
        assert C % H == 0
        self.head_size = C // H
        self.use_triton_ddlerp = use_triton_ddlerp
        self.use_triton_loras = use_triton_loras
        self.attn_impl = attn_impl
        self.triton_dot_prec = triton_dot_prec
        if attn_impl == 'cuda':
            load_attn_ln(self.head_size)
        elif attn_impl == 'triton':
            load_attn(self.head_size)
        # the LoRA expansion kernels work on blocks of 64 channels and normalise kk over heads of any multiple of
        # 16 channels; anything else takes the PyTorch form of that stage
        self._loras_kernel = use_triton_loras and self.head_size % 16 == 0 and C % 64 == 0

        # depth-dependent closed-form initialisation (time_mixer.py:36-54)
        depth = layer_id / max(args.n_layer - 1, 1)          # 0 at the first layer, 1 at the last
        shallow = 1.0 - layer_id / args.n_layer               # 1 at the first layer, towards 0
        pos = torch.arange(C) / C

        def one_minus_pow(exponent, offset=0.0):
            return 1.0 - (torch.pow(pos, exponent) + offset)

        self.time_maa_x = nn.Parameter(one_minus_pow(0.6 * shallow ** 0.9))
        self.time_maa = nn.Parameter(torch.stack([
            one_minus_pow(0.2 * shallow),                       # r, g
            one_minus_pow(0.9 * shallow),                       # w, a
            one_minus_pow(0.9 * shallow, 0.4 * depth),          # k
            one_minus_pow(0.4 * shallow, 0.6 * depth),          # v
        ])[:, None, None, :])
        ramp = torch.arange(C, dtype=torch.float32) / (C - 1)
        self.time_decay = nn.Parameter(-7.0 + 5.0 * ramp ** (0.85 + depth ** 0.5) + 0.5)   # +0.5: the softplus offset
        self.time_faaaa = nn.Parameter(torch.zeros(C))
        self.time_aaaaa = nn.Parameter(torch.zeros(C))

        R = LORA_RANKS
        self.time_maa_w1 = nn.Parameter(torch.zeros(4 * R['mix'], C))
        self.time_maa_w2 = nn.Parameter(_orthogonal(R['mix'], C, 0.1, batch=4).mT.contiguous())
        self.time_decay_w1 = nn.Parameter(torch.zeros(R['decay'], C))
        self.time_decay_w2 = nn.Parameter(_orthogonal(R['decay'], C, 0.1).mT.contiguous())
        self.time_aaa_w1 = nn.Parameter(torch.zeros(R['aaa'], C))
        self.time_aaa_w2 = nn.Parameter(_orthogonal(R['aaa'], C, 0.1).mT.contiguous())
        self.time_kkk_w1 = nn.Parameter(torch.zeros(R['kkk'], C))
        self.time_kkk_w2 = nn.Parameter(_orthogonal(R['kkk'], C, 0.1).mT.contiguous())
        self.gate_w1 = nn.Parameter(_orthogonal(R['gate'], C, 0.1))
        self.gate_w2 = nn.Parameter(_orthogonal(R['gate'], C, 0.1).mT.contiguous())
        self.ma_w1 = nn.Parameter(torch.zeros(R['ma'], C))
        self.ma_w2 = nn.Parameter(_orthogonal(R['ma'], C, 0.1).mT.contiguous())
        self.time_misc_a = nn.Parameter(torch.zeros(C))
        self.mk_w1 = nn.Parameter(torch.zeros(R['mk'], C))
        self.mk_w2 = nn.Parameter(_orthogonal(R['mk'], C, 0.1).mT.contiguous())
        self.time_misc_k = nn.Parameter(torch.zeros(C))

        def uniform(fan_in, fan_out, scale):
            bound = scale / math.sqrt(fan_in)
            return nn.Parameter(torch.empty(fan_out, fan_in).uniform_(-bound, bound))

        self.Wr = uniform(C, C, 0.5)
        self.Wk = uniform(C, C, 0.05)
        self.Wv = uniform(C, C, 0.5)
        self.Wo = uniform(C, C, 0.0)
        self.ln_x = nn.GroupNorm(H, C, eps=64e-5)

    # ---- the two stages that have a kernel and a plain-PyTorch form ----
    def _mix(self, x, x_prev=None):
        """The four token-shifted streams.  x_prev [B,C]: the token before x[:, 0] (a carried state; zero if None)."""
        if self.use_triton_ddlerp:
            ys = ddlerp(x.bfloat16().contiguous(), self.time_maa_x, self.time_maa_w1, self.time_maa_w2, self.time_maa)
            if x_prev is not None:
                # the kernel shifts in a zero before the first token: redo that one token with the carried one
                first = self._mix_plain(x[:, :1].float(), x_prev.float())
                for y, f in zip(ys, first):
                    y[:, :1] = f.to(y.dtype)
            return ys
        return self._mix_plain(x, x_prev)

    def _mix_plain(self, x, x_prev=None):
        B, T, C = x.shape
        shifted = F.pad(x, (0, 0, 1, -1))
        if x_prev is not None:
            shifted = torch.cat([x_prev.to(x.dtype).view(B, 1, C), x[:, :-1]], dim=1)
        xx = shifted - x
        mid = torch.tanh((x + xx * self.time_maa_x.to(x.dtype)) @ self.time_maa_w1.to(x.dtype).mT)
        mid = mid.view(B * T, 4, -1).transpose(0, 1)
        coeff = (mid @ self.time_maa_w2.to(x.dtype).mT).view(4, B, T, C) + self.time_maa.to(x.dtype)
        return (x + xx * coeff).unbind(dim=0)

    def _expand(self, w2, k, kk1, a1, ma1, mk1):
        N = self.head_size
        if self._loras_kernel:
            return expand_loras(w2, k, kk1, a1, ma1, mk1, self.time_kkk_w2, self.time_aaa_w2, self.ma_w2, self.mk_w2,
                                self.time_decay, self.time_aaaaa, self.time_misc_a, self.time_misc_k, N)
        return self._expand_plain(w2, k, kk1, a1, ma1, mk1)

    def _expand_plain(self, w2, k, kk1, a1, ma1, mk1):
        N = self.head_size
        B, T, C = k.shape
        p = lambda t: t.to(k.dtype)
        w = -F.softplus(-(p(self.time_decay) + w2)) - 0.5
        kk = k + torch.tanh(kk1) @ p(self.time_kkk_w2).mT
        kk = F.normalize(kk.view(B, T, C // N, N), dim=-1, p=2.0).view(B, T, C)
        a = torch.sigmoid(p(self.time_aaaaa) + a1 @ p(self.time_aaa_w2).mT)
        ma = torch.sigmoid(p(self.time_misc_a) + ma1 @ p(self.ma_w2).mT)
        mk = torch.sigmoid(p(self.time_misc_k) + mk1 @ p(self.mk_w2).mT)
        k = (k * ma + k * a * (1 - ma)) * torch.exp(w * mk)
        return w, k, kk, -kk * a

    def _wkv_inputs(self, xrg, xwa, xk, xv, fused, dt):
        """From the four shifted streams [B,T,C] to the operands of the recurrence: (r, w, k, v, kk, b, g) and
        the output projection as a callable."""
        P = lambda t: t.to(dt)
        # y = x W^T: the BLAS library for the product itself, this package's kernel for the weight gradient
        # (fused path, bf16); the all-PyTorch path keeps the reference's plain matmuls
        if fused and xrg.is_cuda:
            # all projection weights to bf16 in one multi-tensor copy; concatenated groups come out adjacent
            groups = [[self.Wr], [self.gate_w1], [self.Wk], [self.time_kkk_w1, self.mk_w1], [self.Wv],
                      [self.time_decay_w1, self.time_aaa_w1, self.ma_w1], [self.gate_w2], [self.time_decay_w2], [self.Wo]]
            bWr, bg1, bWk, bkk, bWv, bw1, bg2, bw2, bWo = bf16_copies(groups)
            # the products of the four streams as one autograd node: its backward has all upstream gradients at
            # hand and computes the six weight gradients in one launch (likewise the two second LoRA factors)
            (r, g1), (k, kkmk), (v,), (w1a1ma1,) = projection_sets(
                [(xrg, [[self.Wr], [self.gate_w1]]), (xk, [[self.Wk], [self.time_kkk_w1, self.mk_w1]]),
                 (xv, [[self.Wv]]), (xwa, [[self.time_decay_w1, self.time_aaa_w1, self.ma_w1]])],
                bf16=[[bWr, bg1], [bWk, bkk], [bWv], [bw1]])
            mm_g2w2 = lambda tg, tw: [o[0] for o in projection_sets(
                [(tg, [[self.gate_w2]]), (tw, [[self.time_decay_w2]])], bf16=[[bg2], [bw2]])]
            mm_o = lambda t: projection(t, self.Wo, bf16=bWo)
        else:
            mm = lambda t, *ws: t @ P(ws[0] if len(ws) == 1 else torch.cat(ws)).mT
            r, g1 = mm(xrg, self.Wr), mm(xrg, self.gate_w1)
            k, kkmk = mm(xk, self.Wk), mm(xk, self.time_kkk_w1, self.mk_w1)
            v = mm(xv, self.Wv)
            w1a1ma1 = mm(xwa, self.time_decay_w1, self.time_aaa_w1, self.ma_w1)
            mm_g2w2 = lambda tg, tw: (mm(tg, self.gate_w2), mm(tw, self.time_decay_w2))
            mm_o = lambda t: mm(t, self.Wo)
        R = LORA_RANKS
        if fused and xrg.is_cuda:
            # the slices of the concatenated products, contiguous, and both tanh in one launch (one more in backward)
            kk1, mk1, tw1, a1, ma1, tg1 = split_columns(
                [kkmk, w1a1ma1, g1], [[(R['kkk'], 0), (R['mk'], 0)], [(R['decay'], 1), (R['aaa'], 0), (R['ma'], 0)],
                                      [(R['gate'], 1)]])
        else:
            kk1, mk1 = kkmk.split([R['kkk'], R['mk']], dim=2)
            w1, a1, ma1 = w1a1ma1.split([R['decay'], R['aaa'], R['ma']], dim=2)
            tw1, tg1 = torch.tanh(w1), torch.tanh(g1)
        g, w2 = mm_g2w2(tg1, tw1)

        w, k, kk, b = self._expand(w2, k, kk1, a1, ma1, mk1)

        return (r, w, k, v, kk, b, g), mm_o

    def forward(self, x, state=None, return_state=False):
        """y = TimeMixer(x), the reference's contract (time_mixer.py:96-167).  Beyond it, for inference:
        `state` = (last token of the preceding segment [B,C], WKV7 state [B,H,N,N]) continues a sequence, and
        `return_state=True` returns (y, state) to continue from - a prompt is run in one or several such calls
        and then token by token with `step`.  Either needs attn_impl='cuda' and no autograd, and lifts the
        reference's restriction of T to multiples of 16 (the tokens after the last full chunk go through `step`)."""
        B, T, C = x.shape
        H, N = self.n_head, self.head_size
        fused = self.use_triton_ddlerp or self.use_triton_loras or self.attn_impl != 'ref'
        dt = torch.bfloat16 if fused else x.dtype          # the all-PyTorch path keeps the caller's precision
        stateful = state is not None or return_state
        if stateful:
            assert self.attn_impl == 'cuda', "a carried state needs attn_impl='cuda'"
            assert not (torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))), \
                'a carried state is for inference: run under torch.no_grad()'
        x_prev, wkv_state = state if state is not None else (None, None)
        if stateful and T % 16:
            return self._forward_any_length(x, state, return_state)
        if stateful and wkv_state is None:   # the state to hand on is kept in fp32
            wkv_state = torch.zeros(B, H, N, N, dtype=torch.float32, device=x.device)
        xrg, xwa, xk, xv = self._mix(x, x_prev)
        xrg, xwa, xk, xv = (t.to(dt) for t in (xrg, xwa, xk, xv))

        (r, w, k, v, kk, b, g), mm_o = self._wkv_inputs(xrg, xwa, xk, xv, fused, dt)

        if self.attn_impl == 'cuda':
            params = torch.stack([self.ln_x.weight, self.ln_x.bias, self.time_faaaa]).float()
            seqs = [t.bfloat16().contiguous() for t in (r, w, k, v, kk, b, g)]
            if stateful:
                y, wkv_state = attn_ln(*seqs, params, N, s0=wkv_state, return_state=True)
            else:
                y = attn_ln(*seqs, params, N)   # (bf16 kernels at every head size; triton_dot_prec belongs to 'triton')
        else:
            if self.attn_impl == 'triton':
                y = attn_triton(*(t.bfloat16().contiguous() for t in (r, w, k, v, kk, b)), N,
                                dot_prec=self.triton_dot_prec).float()   # time_mixer.py:159
            else:
                y = ref_attn(r, w, k, v, kk, b, N)
            y = group_norm_heads(y.reshape(B * T, C), H, self.ln_x.weight.to(y.dtype), self.ln_x.bias.to(y.dtype)).view(B, T, C)
            bonus = (r.view(B, T, H, N) * k.view(B, T, H, N) * self.time_faaaa.view(H, N)).sum(-1, keepdim=True)
            y = y + (bonus * v.view(B, T, H, N)).view(B, T, C).to(y.dtype)
            y = (y * g).to(dt)
        if return_state:
            return mm_o(y), (x[:, -1].clone(), wkv_state)
        return mm_o(y)

    def _forward_any_length(self, x, state, return_state):
        """Inference on a length that is no multiple of 16 (the sequence kernels' chunk): the longest such prefix as
        one piece, the remaining tokens one by one."""
        B, T, C = x.shape
        T0 = T - T % 16
        ys = []
        if T0:
            y, state = self.forward(x[:, :T0].contiguous(), state=state, return_state=True)
            ys.append(y)
        elif state is None:
            state = (torch.zeros(B, C, dtype=x.dtype, device=x.device),
                     torch.zeros(B, self.n_head, self.head_size, self.head_size, dtype=torch.float32, device=x.device))
        else:
            state = (state[0], state[1].clone())     # `step` updates the state tensor in place
        for t in range(T0, T):
            y, state = self.step(x[:, t], state)
            ys.append(y.view(B, 1, C))
        y = torch.cat(ys, dim=1)
        return (y, state) if return_state else y

    def _step_on_kernels(self, x, x_prev, S):
        """`step` on the sequence kernels: the B tokens become rows of one short "sequence" for the row-wise
        stages, so a step rounds where the sequence pass rounds.  The token shift sees (previous token, token) as
        the first two tokens of a 16-token sequence per row; rows are padded to a multiple of 16."""
        B, C = x.shape
        N = self.head_size
        Bp = -(-B // 16) * 16
        pair = torch.zeros(Bp, 16, C, dtype=torch.bfloat16, device=x.device)
        pair[:B, 0] = x_prev
        pair[:B, 1] = x
        streams = [t[:, 1].reshape(1, Bp, C) for t in self._mix(pair)]
        seqs, mm_o = self._wkv_inputs(*streams, True, torch.bfloat16)
        params = torch.stack([self.ln_x.weight, self.ln_x.bias, self.time_faaaa]).float()
        y = attn_ln_step(*(t[0, :B].bfloat16().contiguous() for t in seqs), params, S, N)
        return mm_o(y.view(1, B, C)).view(B, C), (x.clone(), S)

    def _decode_weights(self):
        """bf16 copies of the parameters for the single-token kernels, remade when a parameter has been written to.
        The cache holds tensors only (the argument block of device pointers is built per call), so a module with a
        populated cache still pickles and deep-copies; it is left out of both.  A write through `p.data`
        (`p.data.copy_(...)`, as manual weight loading or an EMA update may do) does not change what the cache is keyed
        on (storage address and version counter): call `invalidate_decode_cache()` after such a write."""
        names = _native.MIXER_WEIGHT_NAMES[:-1]
        ps = [getattr(self, n) for n in names] + [self.ln_x.weight, self.ln_x.bias, self.time_faaaa]
        key = tuple((p.data_ptr(), p._version) for p in ps)
        cache = self.__dict__.get('_decode_cache')
        if cache is None or cache[0] != key:
            copies = [getattr(self, n).detach().to(torch.bfloat16).contiguous() for n in names]
            ln = torch.stack([self.ln_x.weight, self.ln_x.bias, self.time_faaaa]).detach().float().contiguous()
            cache = self.__dict__['_decode_cache'] = (key, copies, ln, {})
        return cache

    def invalidate_decode_cache(self):
        """Drop the bf16 parameter copies `step` keeps; the next step remakes them from the parameters."""
        self.__dict__.pop('_decode_cache', None)

    def __getstate__(self):
        state = dict(self.__dict__)
        state.pop('_decode_cache', None)     # derived data: working copies and per-batch workspaces
        return state

    def _step_fused(self, x, x_prev, S):
        """`step` in five launches (wind_rwkv7_mixer_decode): token shift, all first-half products, LoRA second halves
        with the elementwise tail, the WKV7 step with its epilogue, output projection."""
        B, C = x.shape
        _, copies, ln, workspaces = self._decode_weights()
        weights = _native.MixerWeights(*[c.data_ptr() for c in copies], ln.data_ptr())
        lib = _native.lib()
        ws = workspaces.get((B, x.device))
        if ws is None:
            ws = workspaces[(B, x.device)] = torch.empty(lib.wind_rwkv7_mixer_decode_workspace_bytes(B, C), dtype=torch.uint8,
                                                         device=x.device)
        xb, xp = x.bfloat16().contiguous(), x_prev.bfloat16().contiguous()
        y = torch.empty(B, C, dtype=torch.bfloat16, device=x.device)
        carry = torch.empty(B, C, dtype=torch.bfloat16, device=x.device)   # the token to hand on, copied by the first kernel
        with torch.cuda.device(x.device):
            _native.check(lib.wind_rwkv7_mixer_decode(
                B, C, self.n_head, _native.F32 if S.dtype == torch.float32 else _native.BF16, ctypes.byref(weights),
                xb.data_ptr(), xp.data_ptr(), S.data_ptr(), y.data_ptr(), carry.data_ptr(), ws.data_ptr(), ws.numel(),
                torch.cuda.current_stream(x.device).cuda_stream))
        return y, (carry, S)

    @torch.no_grad()
    def step(self, x, state):
        """One token per sequence (decoding): x [B,C], state as returned by `forward(..., return_state=True)` or by
        a previous step; returns (y [B,C] bf16, new state).  The WKV7 state tensor is updated in place.  With the
        default switches and head size 64 every stage runs on this package's kernels (`_step_on_kernels`).  Otherwise
        the small per-token expressions are the reference's plain PyTorch ones (time_mixer.py:113-147) in fp32, and the
        recurrence with its GroupNorm / bonus / gate epilogue runs in the single-token kernel (head sizes 16 .. 128) or as
        the one-token form of the recurrence (time_mixer.py:6-16)."""
        B, C = x.shape
        H, N = self.n_head, self.head_size
        x_prev, S = state
        if x.is_cuda and self.use_triton_ddlerp and self._loras_kernel and _bf16_head(N) and self.attn_impl == 'cuda':
            if torch.compiler.is_compiling() or not S.is_contiguous() or S.dtype not in (torch.float32, torch.bfloat16):
                return self._step_on_kernels(x, x_prev, S)   # (traceable: every stage is a registered operator)
            return self._step_fused(x, x_prev, S)
        xf = x.float().view(B, 1, C)
        xrg, xwa, xk, xv = self._mix_plain(xf, x_prev.float())
        mm = lambda t, *ws: t @ (ws[0] if len(ws) == 1 else torch.cat(ws)).float().mT
        R = LORA_RANKS
        r, g1 = mm(xrg, self.Wr), mm(xrg, self.gate_w1)
        k, kkmk = mm(xk, self.Wk), mm(xk, self.time_kkk_w1, self.mk_w1)
        v = mm(xv, self.Wv)
        kk1, mk1 = kkmk.split([R['kkk'], R['mk']], dim=2)
        w1, a1, ma1 = mm(xwa, self.time_decay_w1, self.time_aaa_w1, self.ma_w1).split([R['decay'], R['aaa'], R['ma']], dim=2)
        g = mm(torch.tanh(g1), self.gate_w2)
        w2 = mm(torch.tanh(w1), self.time_decay_w2)
        w, k, kk, b = self._expand_plain(w2, k, kk1, a1, ma1, mk1)
        if _bf16_head(N) or (x.is_cuda and _attn_bf16_head(N)):   # the single-token kernels cover head sizes 16 .. 128
            params = torch.stack([self.ln_x.weight, self.ln_x.bias, self.time_faaaa]).float()
            y = attn_ln_step(*(t.view(B, C).bfloat16().contiguous() for t in (r, w, k, v, kk, b, g)), params, S, N)
        else:
            hv = lambda t: t.view(B, H, N).to(S.dtype)
            r_, w_, k_, v_, a_, b_ = (hv(t) for t in (r, w, k, v, kk, b))
            sa = (S * a_[:, :, None, :]).sum(-1, keepdim=True)
            S.mul_(torch.exp(-torch.exp(w_))[:, :, None, :]).add_(sa * b_[:, :, None, :]).add_(v_[:, :, :, None] * k_[:, :, None, :])
            y = (S * r_[:, :, None, :]).sum(-1).float().view(B, C)
            y = group_norm_heads(y, H, self.ln_x.weight.float(), self.ln_x.bias.float())
            bonus = (r.view(B, H, N) * k.view(B, H, N) * self.time_faaaa.view(H, N)).sum(-1, keepdim=True)
            y = (y + (bonus * v.view(B, H, N)).view(B, C)) * g.view(B, C)
        y = (y.float() @ self.Wo.float().mT).bfloat16()
        return y, (x.clone(), S)
