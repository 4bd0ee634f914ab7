"""WKV7 with the fused GroupNorm + bonus + gate epilogue ("attn_ln").

Mirrors the reference's rwkv7_attn_ln.py: ``attn_ln(r,w,k,v,a,b,g,params,HEAD_SIZE)`` (:56-62),
``load_attn_ln(HEAD_SIZE)`` (:49-54) and the Function
``apply(w,q,k,v,a,b,g,params,s0) -> (y,sT,s)`` (:18-47).  ``params`` is the fp32 [3,H*C] stack of
(ln weight, ln bias, bonus).  Its gradient is summed in a fixed order on the device.
"""
import torch

from .. import _native
from .wkv_attn import (_OPS, _any_length, _interval_now, _same_interval, _check_sequences, _check_step, _differentiating, _launch, _no_cpu, _ptr,
                       _sized, _state_code, _stream, _workspace, no_state)

_OPS.define('attn_ln_forward(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor g, Tensor params, '
            'Tensor s0, Tensor(a!) y, Tensor(b!) s, Tensor(c!) sT, Tensor(d!) workspace) -> ()')
_OPS.define('attn_ln_prefill(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor g, Tensor params, '
            'Tensor s0, Tensor(a!) y, Tensor(b!) scratch, Tensor(c!) sT, Tensor(d!) workspace) -> ()')
_OPS.define('attn_ln_backward(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor g, Tensor params, '
            'Tensor dy, Tensor s, Tensor dsT, Tensor(a!) dw, Tensor(b!) dq, Tensor(c!) dk, Tensor(d!) dv, '
            'Tensor(e!) da, Tensor(f!) db, Tensor(g!) dg, Tensor(h!) dparams, Tensor(i!) ds0, '
            'Tensor(j!) workspace) -> ()')


def _fwd_impl(w, q, k, v, a, b, g, params, s0, y, s, sT, workspace, entry='wind_rwkv7_attn_ln_forward'):
    B, T, H, C = w.shape
    workspace = _sized(workspace, _native.lib().wind_rwkv7_attn_ln_fwd_workspace_bytes(B, T, H, C))
    with torch.cuda.device(w.device):
        _native.check(getattr(_native.lib(), entry)(
            B, T, H, C, _native.BF16, _state_code(s0),
            w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(), g.data_ptr(),
            params.data_ptr(), _ptr(s0), y.data_ptr(), s.data_ptr(), sT.data_ptr(),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(w)))


def _prefill_impl(w, q, k, v, a, b, g, params, s0, y, scratch, sT, workspace):
    _fwd_impl(w, q, k, v, a, b, g, params, s0, y, scratch, sT, workspace, 'wind_rwkv7_attn_ln_prefill')


def _bwd_impl(w, q, k, v, a, b, g, params, dy, s, dsT, dw, dq, dk, dv, da, db, dg, dparams, ds0, workspace):
    B, T, H, C = w.shape
    workspace = _sized(workspace, _native.lib().wind_rwkv7_attn_ln_bwd_workspace_bytes(B, T, H, C))
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_ln_backward(
            B, T, H, C, _native.BF16, _state_code(dsT),
            w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(), g.data_ptr(),
            params.data_ptr(), dy.data_ptr(), s.data_ptr(), _ptr(dsT),
            dw.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), da.data_ptr(), db.data_ptr(), dg.data_ptr(),
            dparams.data_ptr(), _ptr(ds0),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(w)))


for _name, _impl in (('attn_ln_forward', _fwd_impl), ('attn_ln_prefill', _prefill_impl), ('attn_ln_backward', _bwd_impl)):
    _OPS.impl(_name, _impl, 'CUDA')
    _OPS.impl(_name, _no_cpu, 'CPU')
    _OPS.impl(_name, lambda *a: None, 'Meta')


@torch.compiler.assume_constant_result
def _sizes(B, T, H, C):
    lib = _native.lib()
    saved = lib.wind_rwkv7_attn_ln_saved_bytes(B, T, H, C)
    if saved == 0:
        if not lib.wind_rwkv7_head_size_supported(C):
            _native.check(3)
        if T % lib.wind_rwkv7_chunk_len():
            _native.check(4)
        _native.check(2)
    return (saved, lib.wind_rwkv7_attn_ln_fwd_workspace_bytes(B, T, H, C),
            lib.wind_rwkv7_attn_ln_bwd_workspace_bytes(B, T, H, C))


@torch.compiler.assume_constant_result
def _saved_unit(C):
    """bf16 elements of the saved tensor per (batch, head, chunk): its size is linear in all three."""
    return _sizes(1, 16, 1, C)[0] // 2


def fw_attn_ln(w, q, k, v, a, b, g, params, s0, save=True):
    """Allocates y, sT and the saved tensor and runs the forward kernels (reference: rwkv7_attn_ln.py:5-11).
    save=False: the forward that stores nothing for a backward pass; the third result is then scratch."""
    B, T, H, C = w.shape
    if not torch.compiler.is_compiling():
        _sizes(B, T, H, C)   # names a bad shape
    y = torch.empty_like(v)
    sT = torch.empty(B, H, C, C, dtype=s0.dtype, device=w.device)   # (s0 may be the empty stand-in for a zero state)
    s = torch.empty(B, H, T // 16, _saved_unit(C), dtype=torch.bfloat16, device=w.device)
    ws = _workspace(lambda: _sizes(B, T, H, C)[1], w.device)
    _launch(*(('attn_ln_forward', _fwd_impl) if save else ('attn_ln_prefill', _prefill_impl)),
            w, q, k, v, a, b, g, params, s0, y, s, sT, ws)
    return y, sT, s


def bw_attn_ln(w, q, k, v, a, b, g, params, s, dy, dsT, want_ds0=True):
    """Allocates the nine gradients and runs the backward kernels (reference: rwkv7_attn_ln.py:13-17).  dsT may be
    the empty stand-in (no gradient reaches the final state); want_ds0=False leaves ds0 empty and unwritten."""
    B, T, H, C = w.shape
    dw, dq, dk, dv, da, db, dg = [torch.empty_like(x) for x in (w, q, k, v, a, b, g)]
    ds0 = torch.empty(B, H, C, C, dtype=dsT.dtype, device=w.device) if want_ds0 else no_state(dsT.dtype, w.device)
    dparams = torch.empty_like(params)
    ws = _workspace(lambda: _sizes(B, T, H, C)[2], w.device)
    _launch('attn_ln_backward', _bwd_impl, w, q, k, v, a, b, g, params, dy, s, dsT,
            dw, dq, dk, dv, da, db, dg, dparams, ds0, ws)
    return dw, dq, dk, dv, da, db, dg, dparams, ds0


def _check_inputs(seqs, params, s0):
    if torch.compiler.is_compiling():
        return
    _check_sequences(seqs, s0)
    B, T, H, C = seqs[0].shape
    assert params.dtype == torch.float32, 'params must be float32'
    assert params.is_contiguous(), 'inputs must be contiguous'
    assert tuple(params.shape) == (3, H * C), 'params must be [3, H*C]'


class WindRWKV7LN(torch.autograd.Function):
    """(w,q,k,v,a,b,g,params,s0) -> (y, sT, s).  Sequences [B,T,H,C] bf16; params [3,H*C] fp32;
    s0 [B,H,C,C] bf16 or fp32."""

    @staticmethod
    def forward(ctx, w, q, k, v, a, b, g, params, s0):
        _check_inputs((w, q, k, v, a, b, g), params, s0)
        y, sT, s = fw_attn_ln(w, q, k, v, a, b, g, params, s0)
        ctx.set_materialize_grads(False)
        ctx.state_dtype = s0.dtype
        ctx.has_s0 = s0.numel() > 0
        ctx.checkpoint_interval = _interval_now()
        ctx.save_for_backward(w, q, k, v, a, b, g, params, s)
        return y, sT, s

    @staticmethod
    def backward(ctx, dy, dsT, ds):
        w, q, k, v, a, b, g, params, s = ctx.saved_tensors
        B, T, H, C = w.shape
        _same_interval(ctx)
        if dsT is None:   # the usual case in training: nothing reads the final state
            dsT = no_state(ctx.state_dtype, w.device)
        if dy is None:
            dy = torch.zeros_like(v)
        if not torch.compiler.is_compiling():
            assert ds is None, 'the saved tensor is not differentiable'
            assert dy.dtype == torch.bfloat16 and dsT.dtype == ctx.state_dtype
        want_ds0 = ctx.has_s0 and ctx.needs_input_grad[8]
        grads = bw_attn_ln(w, q, k, v, a, b, g, params, s, dy.contiguous(), dsT.contiguous(), want_ds0)
        return grads if want_ds0 else grads[:8] + (None,)


@torch.compiler.assume_constant_result
def load_attn_ln(HEAD_SIZE):
    """Reference: JIT-compiles the fused CUDA extension for one head size (rwkv7_attn_ln.py:49-54).
    Here: loads the prebuilt library and checks that some kernel covers the head size."""
    from .wkv_attn import load_attn
    load_attn(HEAD_SIZE)


def group_norm_heads(y, H, weight, bias, eps=64e-5):
    """GroupNorm of y [rows, H*C] over each head's C channels (biased variance), times weight plus bias: what
    `F.group_norm(y, H, weight, bias, eps)` computes (the reference's call, time_mixer.py:154,160), written with
    elementary operations.  The framework's own group_norm is not used on purpose: in this ROCm build its backward
    returns wrong weight and bias gradients for 2-D inputs of 256 rows or more (relative error ~1; the input
    gradient and the forward are right), so every gradient of ln_w / ln_b through it at B*T >= 256 was off."""
    rows, HC = y.shape
    yh = y.view(rows, H, HC // H)
    mean = yh.mean(-1, keepdim=True)
    var = yh.var(-1, unbiased=False, keepdim=True)
    yn = ((yh - mean) * torch.rsqrt(var + eps)).view(rows, HC)
    return yn * weight + bias


_OPS.define('ln_epilogue_forward(Tensor y, Tensor q, Tensor k, Tensor v, Tensor g, Tensor params, int H, '
            'Tensor(a!) out) -> ()')
_OPS.define('ln_epilogue_backward(Tensor y, Tensor q, Tensor k, Tensor v, Tensor g, Tensor params, Tensor dout, int H, '
            'Tensor(a!) dy, Tensor(b!) dq, Tensor(c!) dk, Tensor(d!) dv, Tensor(e!) dg, Tensor(f!) dparams, '
            'Tensor(g!) workspace) -> ()')


def _epilogue_fwd_impl(y, q, k, v, g, params, H, out):
    B, T, HC = y.shape
    with torch.cuda.device(y.device):
        _native.check(_native.lib().wind_rwkv7_ln_epilogue_forward(
            B, T, H, HC // H, y.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), params.data_ptr(),
            out.data_ptr(), _stream(y)))


def _epilogue_bwd_impl(y, q, k, v, g, params, dout, H, dy, dq, dk, dv, dg, dparams, workspace):
    B, T, HC = y.shape
    workspace = _sized(workspace, _native.lib().wind_rwkv7_ln_epilogue_bwd_workspace_bytes(B, T, H, HC // H))
    with torch.cuda.device(y.device):
        _native.check(_native.lib().wind_rwkv7_ln_epilogue_backward(
            B, T, H, HC // H, y.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), params.data_ptr(),
            dout.data_ptr(), dy.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dg.data_ptr(),
            dparams.data_ptr(), workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(y)))


for _name, _impl in (('ln_epilogue_forward', _epilogue_fwd_impl), ('ln_epilogue_backward', _epilogue_bwd_impl)):
    _OPS.impl(_name, _impl, 'CUDA')
    _OPS.impl(_name, _no_cpu, 'CPU')
    _OPS.impl(_name, lambda *a: None, 'Meta')


@torch.compiler.assume_constant_result
def _epilogue_bwd_workspace_bytes(B, T, H, C):
    return _native.lib().wind_rwkv7_ln_epilogue_bwd_workspace_bytes(B, T, H, C)


class LnEpilogue(torch.autograd.Function):
    """The GroupNorm + bonus + gate epilogue of attn_ln as an operator of its own (attn_ln.cu:11-37, :40-104), for the
    head sizes whose WKV7 kernels do not have it inside: y (the WKV7 output), q, k, v, g [B,T,H*C] bf16, params
    [3,H*C] fp32 -> out [B,T,H*C] bf16."""

    @staticmethod
    def forward(ctx, y, q, k, v, g, params, H):
        seqs = [t.contiguous() for t in (y, q, k, v, g)]
        params = params.contiguous()
        if not torch.compiler.is_compiling():
            assert all(t.dtype == torch.bfloat16 and t.shape == seqs[0].shape for t in seqs), 'sequences must be bfloat16'
            assert params.dtype == torch.float32 and tuple(params.shape) == (3, seqs[0].shape[2])
        out = torch.empty_like(seqs[0])
        _launch('ln_epilogue_forward', _epilogue_fwd_impl, *seqs, params, int(H), out)
        ctx.save_for_backward(*seqs, params)
        ctx.H = int(H)
        return out

    @staticmethod
    def backward(ctx, dout):
        *seqs, params = ctx.saved_tensors
        B, T, HC = seqs[0].shape
        grads = [torch.empty_like(seqs[0]) for _ in range(5)]
        dparams = torch.empty_like(params)
        ws = _workspace(lambda: _epilogue_bwd_workspace_bytes(B, T, ctx.H, HC // ctx.H), dout.device)
        _launch('ln_epilogue_backward', _epilogue_bwd_impl, *seqs, params, dout.contiguous(), ctx.H, *grads, dparams, ws)
        dy, dq, dk, dv, dg = grads
        return dy, dq, dk, dv, dg, dparams, None


def attn_ln(r, w, k, v, a, b, g, params, HEAD_SIZE, s0=None, return_state=False, dot_prec=None):
    """out = gate * (group_norm(WKV7(r,w,k,v,a,b)) + bonus term); sequences are [B,T,H*HEAD_SIZE] bf16 (or all
    float32 for the accuracy mode), params [3,H*HEAD_SIZE] fp32 (rwkv7_attn_ln.py:56-62).  As in the reference
    the initial state is zero and only the output is returned; `s0` and `return_state=True` carry the state as
    for `attn`.  The fused bf16 kernels cover HEAD_SIZE 64; other head sizes (multiples of 16 up to 128) run the
    plain WKV7 operator for that head size followed by the epilogue, and return the sequences' dtype.
    On bf16 tensors that is the bf16 matrix-core kernels for that head size followed by the epilogue kernels,
    composed inside the library's attn_ln entry points (`LnEpilogue` offers the epilogue alone), as the reference's attn_ln is its bf16 CUDA kernel at whatever head size it was built for
    (rwkv7_attn_ln.py:11-17).  `dot_prec` (not in the reference's signature; the keyword of `attn_triton_bighead`,
    rwkv7_attn_triton_bighead.py:366) can ask for the accuracy mode instead: 'fp32' runs the fp32 kernels with the
    epilogue in PyTorch in fp32, about seventeen times slower at head size 128; None / 'bf16' / 'tf32' the bf16
    kernels.  float32 tensors always take the fp32 route.  It has no effect at head size 64."""
    from .wkv_attn import attn, _attn_bf16_head, _bf16_head
    B, T, HC = w.shape
    C = HEAD_SIZE
    H = HC // C
    if dot_prec not in (None, 'fp32', 'tf32', 'bf16'):
        raise ValueError(f"dot_prec must be None, 'fp32', 'tf32' or 'bf16', got {dot_prec!r}")
    if w.dtype == torch.float32 or not (_bf16_head(C) or (dot_prec != 'fp32' and _attn_bf16_head(C))):
        # the fp32 WKV7 kernels followed by the epilogue in PyTorch (fp32 arithmetic), as the reference composes its
        # own unfused path (time_mixer.py:158-163); accurate to fp32 rounding, the result cast to the sequences' dtype
        out_dtype = v.dtype
        r, w, k, v, a, b, g = [x.float() for x in (r, w, k, v, a, b, g)]
        y, sT = attn(r, w, k, v, a, b, HEAD_SIZE, s0=s0, return_state=True)
        y = group_norm_heads(y.reshape(B * T, HC), H, params[0], params[1]).view(B, T, HC)
        bonus = (r.view(B, T, H, C) * k.view(B, T, H, C) * params[2].view(H, C)).sum(-1, keepdim=True)
        y = ((y + (bonus * v.view(B, T, H, C)).view(B, T, HC)) * g).to(out_dtype)
        return (y, sT) if return_state else y
    # bf16 tensors from here on: the library's attn_ln entry points (at head size 64 the fused kernels, at the other
    # head sizes that head size's WKV7 kernels and the epilogue kernels, composed inside the library)
    if T % 16 and not _differentiating(r, w, k, v, a, b, g, params):
        # inference on a length that is no multiple of the chunk: whole chunks here, the rest token by token
        y, sT = _any_length(lambda xs, st: attn_ln(*xs, params, C, s0=st, return_state=True),
                            lambda xs, st: attn_ln_step(*xs, params, st, C), (r, w, k, v, a, b, g), s0, H, C)
        return (y, sT) if return_state else y
    r, w, k, v, a, b, g = [x.view(B, T, H, C) for x in (r, w, k, v, a, b, g)]
    if s0 is None:   # the kernels take "no initial state" as such
        s0 = no_state(torch.bfloat16, w.device)
    if _differentiating(w, r, k, v, a, b, g, params, s0):
        y, sT, _ = WindRWKV7LN.apply(w, r, k, v, a, b, g, params, s0)
    else:   # nothing will be differentiated: the forward that keeps nothing for a backward pass
        _check_inputs((w, r, k, v, a, b, g), params, s0)
        y, sT, _ = fw_attn_ln(w, r, k, v, a, b, g, params, s0, save=False)
    y = y.view(B, T, HC)
    return (y, sT) if return_state else y


_OPS.define('attn_ln_decode(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor g, Tensor params, '
            'Tensor(a!) state, Tensor(b!) y) -> ()')


def _attn_ln_decode_impl(w, q, k, v, a, b, g, params, state, y):
    B, H, C = w.shape
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_ln_decode(
            B, H, C, _native.BF16, _state_code(state), w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            a.data_ptr(), b.data_ptr(), g.data_ptr(), params.data_ptr(), state.data_ptr(), y.data_ptr(), _stream(w)))


_OPS.impl('attn_ln_decode', _attn_ln_decode_impl, 'CUDA')
_OPS.impl('attn_ln_decode', _no_cpu, 'CPU')
_OPS.impl('attn_ln_decode', lambda *a: None, 'Meta')


def attn_ln_step(r, w, k, v, a, b, g, params, state, HEAD_SIZE):
    """One token of attn_ln per sequence (decoding): r,w,k,v,a,b,g are [B, H*HEAD_SIZE] bf16, params
    [3, H*HEAD_SIZE] fp32; `state` [B,H,C,C] is updated IN PLACE; returns [B, H*HEAD_SIZE].  Inference only."""
    B, HC = w.shape
    C = int(HEAD_SIZE)
    H = HC // C
    if not torch.compiler.is_compiling():
        _check_step((r, w, k, v, a, b, g), state, B, H, C)
        assert params.dtype == torch.float32 and params.is_contiguous() and tuple(params.shape) == (3, HC)
    y = torch.empty_like(v)
    with torch.no_grad():
        _launch('attn_ln_decode', _attn_ln_decode_impl, *[x.view(B, H, C) for x in (w, r, k, v, a, b, g)], params, state,
                y.view(B, H, C))
    return y
