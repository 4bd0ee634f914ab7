"""WKV7 ("attn"): autograd Function and public wrappers over the HIP kernels.

Mirrors the interface of the reference's rwkv7_attn.py: ``attn(r,w,k,v,a,b,HEAD_SIZE)`` (:53-59),
``load_attn(HEAD_SIZE)`` (:46-51) and the Function ``WindRWKV7.apply(w,q,k,v,a,b,s0) -> (y,sT,s)``
(:18-44).  Differences: the state tensors may be fp32 as well as bf16, the head size is a runtime
argument of a prebuilt library (``load_attn`` only checks it is supported), and the saved tensor ``s``
has a private layout.
"""
import torch

from .. import _native

_OPS = torch.library.Library('wind_rwkv7', 'DEF')
_OPS.define('attn_forward(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor s0, '
            'Tensor(a!) y, Tensor(b!) s, Tensor(c!) sT, Tensor(d!) workspace) -> ()')
_OPS.define('attn_prefill(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor s0, '
            'Tensor(a!) y, Tensor(b!) scratch, Tensor(c!) sT, Tensor(d!) workspace) -> ()')
_OPS.define('attn_backward(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor dy, Tensor s, '
            'Tensor dsT, Tensor(a!) dw, Tensor(b!) dq, Tensor(c!) dk, Tensor(d!) dv, Tensor(e!) da, '
            'Tensor(f!) db, Tensor(g!) ds0, Tensor(h!) workspace) -> ()')


def _state_code(t):
    return _native.F32 if t.dtype == torch.float32 else _native.BF16


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _workspace(nbytes, device):
    """The workspace tensor an operator is given.  Eager: sized here.  Under torch.compile the sizes may be
    symbolic and the library cannot be asked, so an empty tensor goes in and the operator sizes its own when it
    runs (`_sized`)."""
    if torch.compiler.is_compiling():
        return torch.empty(0, dtype=torch.uint8, device=device)
    return torch.empty(nbytes(), dtype=torch.uint8, device=device)


def _ptr(t):
    """Device address of a tensor; an EMPTY tensor stands for "no tensor" and gives the C ABI's NULL (a zero initial
    state, a final state without gradient, an initial-state gradient nobody wants) - no tensor of zeros is made."""
    return t.data_ptr() if t.numel() else 0


def no_state(dtype, device):
    """The empty tensor that stands for an absent state (see _ptr)."""
    return torch.empty(0, dtype=dtype, device=device)


def _sized(workspace, nbytes):
    return workspace if workspace.numel() else torch.empty(max(nbytes, 1), dtype=torch.uint8, device=workspace.device)


def _attn_forward_impl(w, q, k, v, a, b, s0, y, s, sT, workspace, entry='wind_rwkv7_attn_forward'):
    B, T, H, C = w.shape
    workspace = _sized(workspace, _native.lib().wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C))
    with torch.cuda.device(w.device):
        _native.check(getattr(_native.lib(), entry)(
            B, T, H, C, _native.BF16, _state_code(s0),
            w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(), _ptr(s0),
            y.data_ptr(), s.data_ptr(), sT.data_ptr(),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(w)))


def _attn_prefill_impl(w, q, k, v, a, b, s0, y, scratch, sT, workspace):
    _attn_forward_impl(w, q, k, v, a, b, s0, y, scratch, sT, workspace, 'wind_rwkv7_attn_prefill')


def _attn_backward_impl(w, q, k, v, a, b, dy, s, dsT, dw, dq, dk, dv, da, db, ds0, workspace):
    B, T, H, C = w.shape
    workspace = _sized(workspace, _native.lib().wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C))
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_backward(
            B, T, H, C, _native.BF16, _state_code(dsT),
            w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(),
            dy.data_ptr(), s.data_ptr(), _ptr(dsT),
            dw.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), da.data_ptr(), db.data_ptr(), _ptr(ds0),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(w)))


def _numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def _flat_offsets(shapes, dtype):
    """Element offsets of contiguous tensors of the given shapes inside one buffer (each start 256-byte aligned),
    and the buffer's size."""
    step = 256 // dtype.itemsize
    offs, total = [], 0
    for sh in shapes:
        offs.append(total)
        total += (_numel(sh) + step - 1) // step * step
    return offs, total


def _flat_views(shapes, dtype, device):
    """One allocation carved into contiguous tensors of the given shapes (each start 256-byte aligned)."""
    offs, total = _flat_offsets(shapes, dtype)
    flat = torch.empty(total, dtype=dtype, device=device)
    return flat, [flat[o:o + _numel(sh)].view(sh) for sh, o in zip(shapes, offs)]


def _params_as_bf16(params):
    """bf16 contiguous versions of the parameters: the tensors themselves when they already are, otherwise one
    staging buffer filled by a single multi-tensor copy (the reference casts each parameter on its own,
    rwkv7_ddlerp.py:309, rwkv7_expand_loras.py:218)."""
    if all(p.dtype == torch.bfloat16 and p.is_contiguous() for p in params):
        return list(params)
    shapes = [tuple(p.shape) for p in params]
    flat, views = _flat_views(shapes, torch.bfloat16, params[0].device)
    srcs = [p.detach() for p in params]
    if flat.is_cuda and all(p.is_contiguous() and p.dtype in (torch.float32, torch.bfloat16) for p in srcs):
        from .linear import cast_to_bf16   # (linear imports this module)
        cast_to_bf16(srcs, flat, _flat_offsets(shapes, torch.bfloat16)[0])
    else:
        torch._foreach_copy_(views, srcs)
    return views


def _grads_like(flat_f32, views_f32, params_dtype):
    """The fp32 gradient views themselves for fp32 parameters; for bf16 parameters one cast of the whole buffer."""
    if params_dtype == torch.float32:
        return views_f32
    flat = flat_f32.to(params_dtype)
    shapes = [tuple(v.shape) for v in views_f32]
    offs, _ = _flat_offsets(shapes, torch.float32)   # the layout _flat_views gave the fp32 buffer
    return [flat[o:o + _numel(sh)].view(sh) for sh, o in zip(shapes, offs)]


def _launch(name, impl, *args):
    """One operator call.  Under torch.compile it is the `torch.library` operator (what the tracer can record);
    in eager mode the implementation is called directly, which saves the dispatcher's per-call cost (some 10 us
    on each of the ~30 launches of a time-mixer step)."""
    if torch.compiler.is_compiling():
        return getattr(torch.ops.wind_rwkv7, name)(*args)
    for t in args:
        if isinstance(t, (list, tuple)):
            t = next((e for e in t if isinstance(e, torch.Tensor)), None)
        if isinstance(t, torch.Tensor):
            if not t.is_cuda:
                _no_cpu()
            break
    return impl(*args)


def _no_cpu(*args):
    raise RuntimeError('wind_rwkv7 kernels exist for AMD GPUs only (tensors must live on a HIP device); '
                       'there is no CPU implementation')


_OPS.impl('attn_forward', _attn_forward_impl, 'CUDA')
_OPS.impl('attn_prefill', _attn_prefill_impl, 'CUDA')
_OPS.impl('attn_prefill', _no_cpu, 'CPU')
_OPS.impl('attn_prefill', lambda *a: None, 'Meta')
_OPS.impl('attn_backward', _attn_backward_impl, 'CUDA')
_OPS.impl('attn_forward', _no_cpu, 'CPU')
_OPS.impl('attn_backward', _no_cpu, 'CPU')
_OPS.impl('attn_forward', lambda *a: None, 'Meta')
_OPS.impl('attn_backward', lambda *a: None, 'Meta')


@torch.compiler.assume_constant_result
def _sizes(B, T, H, C):
    # (a constant under torch.compile: the tracer does not follow the library calls)
    lib = _native.lib()
    saved = lib.wind_rwkv7_attn_saved_bytes(B, T, H, C)
    if saved == 0:
        # let the entry point name the problem
        if not lib.wind_rwkv7_attn_head_size_supported(C):
            _native.check(3)
        if T % lib.wind_rwkv7_chunk_len():
            _native.check(4)
        _native.check(2)
    return saved, lib.wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C), lib.wind_rwkv7_attn_bwd_workspace_bytes(B, T, H, C)


@torch.compiler.assume_constant_result
def _saved_unit(C):
    """bf16 elements of the saved tensor per (batch, head, chunk): its size is linear in all three."""
    return _sizes(1, 16, 1, C)[0] // 2


def checkpoint_interval():
    """Tokens between the states the training forward keeps for backward: 32 (default) or 16."""
    return _native.lib().wind_rwkv7_checkpoint_interval()


def set_checkpoint_interval(tokens):
    """16: a state checkpoint per 16-token chunk, as in the reference (attn.cu:92-94).  32 (default): two-level
    chunking - 16-token products, a checkpoint only every second chunk, the gradient kernel carries the state across
    the pair itself (512 bytes less per token and head moved in each direction).  Process-wide; set it between whole
    forward + backward passes, never between a forward and its backward."""
    _native.check(_native.lib().wind_rwkv7_set_checkpoint_interval(int(tokens)))


@torch.compiler.assume_constant_result
def _interval_now():
    return _native.lib().wind_rwkv7_checkpoint_interval()


def _same_interval(ctx):
    """The saved tensor's layout follows the checkpoint interval the forward ran under; a backward under another value
    would misread it, so that is an error and not a wrong gradient."""
    if not torch.compiler.is_compiling() and _interval_now() != ctx.checkpoint_interval:
        raise RuntimeError(f'checkpoint interval changed between forward ({ctx.checkpoint_interval}) and backward '
                           f'({_interval_now()}): set it between whole forward + backward passes only')


def _differentiating(*tensors):
    """Whether autograd will ask for a backward pass through an operator on these inputs."""
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def fw_attn(w, q, k, v, a, b, s0, save=True):
    """Allocates y, sT and the saved tensor, then runs the forward kernels (reference: rwkv7_attn.py:5-11).
    save=False: the forward that stores nothing for a backward pass; the third result is then scratch."""
    B, T, H, C = w.shape
    if not torch.compiler.is_compiling():
        _sizes(B, T, H, C)   # names a bad shape
    y = torch.empty_like(v)
    sT = torch.empty(B, H, C, C, dtype=s0.dtype, device=w.device)   # (s0 may be the empty stand-in for a zero state)
    s = torch.empty(B, H, T // 16, _saved_unit(C), dtype=torch.bfloat16, device=w.device)
    ws = _workspace(lambda: _sizes(B, T, H, C)[1], w.device)
    if save:
        _launch('attn_forward', _attn_forward_impl, w, q, k, v, a, b, s0, y, s, sT, ws)
    else:
        _launch('attn_prefill', _attn_prefill_impl, w, q, k, v, a, b, s0, y, s, sT, ws)
    return y, sT, s


def bw_attn(w, q, k, v, a, b, s, dy, dsT, want_ds0=True):
    """Allocates the seven gradients and runs the backward kernels (reference: rwkv7_attn.py:13-16).  dsT may be the
    empty stand-in (no gradient reaches the final state); want_ds0=False leaves ds0 empty and unwritten."""
    B, T, H, C = w.shape
    dw, dq, dk, dv, da, db = [torch.empty_like(x) for x in (w, q, k, v, a, b)]
    ds0 = torch.empty(B, H, C, C, dtype=dsT.dtype, device=w.device) if want_ds0 else no_state(dsT.dtype, w.device)
    ws = _workspace(lambda: _sizes(B, T, H, C)[2], w.device)
    _launch('attn_backward', _attn_backward_impl, w, q, k, v, a, b, dy, s, dsT, dw, dq, dk, dv, da, db, ds0, ws)
    return dw, dq, dk, dv, da, db, ds0


_STATE_DTYPES = (torch.bfloat16, torch.float32)


def _check_sequences(seqs, s0):
    if torch.compiler.is_compiling():
        return
    w = seqs[0]
    B, T, H, C = w.shape
    assert T % 16 == 0, 'sequence length must be a multiple of 16'
    assert all(x.dtype == torch.bfloat16 for x in seqs), 'sequence inputs must be bfloat16'
    assert s0.dtype in _STATE_DTYPES, 's0 must be bfloat16 or float32'
    assert all(x.is_contiguous() for x in tuple(seqs) + (s0,)), 'inputs must be contiguous'
    assert all(x.shape == w.shape for x in seqs), 'sequence inputs must share one shape'
    assert s0.numel() == 0 or tuple(s0.shape) == (B, H, C, C), 's0 must be [B,H,C,C]'


class WindRWKV7(torch.autograd.Function):
    """(w,q,k,v,a,b,s0) -> (y, sT, s).  w..b: [B,T,H,C] bf16; s0: [B,H,C,C] bf16 or fp32."""

    @staticmethod
    def forward(ctx, w, q, k, v, a, b, s0):
        _check_sequences((w, q, k, v, a, b), s0)
        y, sT, s = fw_attn(w, q, k, v, a, b, s0)
        ctx.set_materialize_grads(False)
        ctx.state_dtype = s0.dtype
        ctx.has_s0 = s0.numel() > 0
        ctx.checkpoint_interval = _interval_now()
        ctx.save_for_backward(w, q, k, v, a, b, s)
        return y, sT, s

    @staticmethod
    def backward(ctx, dy, dsT, ds):
        w, q, k, v, a, b, s = ctx.saved_tensors
        B, T, H, C = w.shape
        _same_interval(ctx)
        if dsT is None:   # the usual case in training: nothing reads the final state
            dsT = no_state(ctx.state_dtype, w.device)
        if dy is None:
            dy = torch.zeros_like(v)
        if not torch.compiler.is_compiling():
            assert ds is None, 'the saved tensor is not differentiable'
            assert dy.dtype == torch.bfloat16 and dsT.dtype == ctx.state_dtype
        dy, dsT = dy.contiguous(), dsT.contiguous()
        want_ds0 = ctx.has_s0 and ctx.needs_input_grad[6]
        grads = bw_attn(w, q, k, v, a, b, s, dy, dsT, want_ds0)
        return grads if want_ds0 else grads[:6] + (None,)


# ---- fp32 sequences: the accuracy mode (fp32 state, fp32 arithmetic, no matrix cores) ----
_OPS.define('attn_f32_forward(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor s0, '
            'Tensor(a!) y, Tensor(b!) s, Tensor(c!) sT) -> ()')
_OPS.define('attn_f32_prefill(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor s0, '
            'Tensor(a!) y, Tensor(b!) sT) -> ()')
_OPS.define('attn_f32_backward(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor dy, Tensor s, '
            'Tensor dsT, Tensor(a!) dw, Tensor(b!) dq, Tensor(c!) dk, Tensor(d!) dv, Tensor(e!) da, '
            'Tensor(f!) db, Tensor(g!) ds0) -> ()')


def _attn_f32_forward_impl(w, q, k, v, a, b, s0, y, s, sT):
    B, T, H, C = w.shape
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_f32_forward(
            B, T, H, C, w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(),
            s0.data_ptr(), y.data_ptr(), s.data_ptr(), sT.data_ptr(), _stream(w)))


def _attn_f32_prefill_impl(w, q, k, v, a, b, s0, y, sT):
    B, T, H, C = w.shape
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_f32_prefill(
            B, T, H, C, w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(),
            s0.data_ptr(), y.data_ptr(), sT.data_ptr(), _stream(w)))


def _attn_f32_backward_impl(w, q, k, v, a, b, dy, s, dsT, dw, dq, dk, dv, da, db, ds0):
    B, T, H, C = w.shape
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_f32_backward(
            B, T, H, C, w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), b.data_ptr(),
            dy.data_ptr(), s.data_ptr(), dsT.data_ptr(), dw.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
            da.data_ptr(), db.data_ptr(), ds0.data_ptr(), _stream(w)))


_OPS.impl('attn_f32_forward', _attn_f32_forward_impl, 'CUDA')
_OPS.impl('attn_f32_prefill', _attn_f32_prefill_impl, 'CUDA')
_OPS.impl('attn_f32_prefill', _no_cpu, 'CPU')
_OPS.impl('attn_f32_prefill', lambda *a: None, 'Meta')
_OPS.impl('attn_f32_backward', _attn_f32_backward_impl, 'CUDA')
_OPS.impl('attn_f32_forward', _no_cpu, 'CPU')
_OPS.impl('attn_f32_backward', _no_cpu, 'CPU')
_OPS.impl('attn_f32_forward', lambda *a: None, 'Meta')
_OPS.impl('attn_f32_backward', lambda *a: None, 'Meta')


def _check_f32(w, q, k, v, a, b, s0):
    if torch.compiler.is_compiling():
        return
    B, T, H, C = w.shape
    seqs = (w, q, k, v, a, b)
    assert T % 16 == 0, 'sequence length must be a multiple of 16'
    assert all(x.dtype == torch.float32 for x in seqs + (s0,)), 'w,q,k,v,a,b,s0 must be float32'
    assert all(x.is_contiguous() for x in seqs + (s0,)), 'inputs must be contiguous'
    assert all(x.shape == w.shape for x in seqs) and tuple(s0.shape) == (B, H, C, C)
    _f32_saved_bytes(B, T, H, C)   # names a bad shape


def fw_attn_f32_no_grad(w, q, k, v, a, b, s0):
    """The fp32 forward that saves no states: (y, sT)."""
    _check_f32(w, q, k, v, a, b, s0)
    y, sT = torch.empty_like(v), torch.empty_like(s0)
    _launch('attn_f32_prefill', _attn_f32_prefill_impl, w, q, k, v, a, b, s0, y, sT)
    return y, sT


class WindRWKV7F32(torch.autograd.Function):
    """(w,q,k,v,a,b,s0) -> (y, sT, s) with everything float32: w..b [B,T,H,C], s0 [B,H,C,C].  The counterpart of
    the reference's TritonRWKV7 run with dot_prec='fp32' (rwkv7_attn_triton.py:159-190): slower than the bf16
    kernels, accurate to fp32 rounding."""

    @staticmethod
    def forward(ctx, w, q, k, v, a, b, s0):
        B, T, H, C = w.shape
        _check_f32(w, q, k, v, a, b, s0)
        y, sT = torch.empty_like(v), torch.empty_like(s0)
        s = torch.empty(B * H * (T // 16) * _f32_saved_unit(C), dtype=torch.float32, device=w.device)
        _launch('attn_f32_forward', _attn_f32_forward_impl, w, q, k, v, a, b, s0, y, s, sT)
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(w, q, k, v, a, b, s)
        return y, sT, s

    @staticmethod
    def backward(ctx, dy, dsT, ds):
        w, q, k, v, a, b, s = ctx.saved_tensors
        B, T, H, C = w.shape
        dsT = torch.zeros(B, H, C, C, dtype=torch.float32, device=w.device) if dsT is None else dsT.contiguous()
        dy = torch.zeros_like(v) if dy is None else dy.contiguous()
        dw, dq, dk, dv, da, db, ds0 = [torch.empty_like(x) for x in (w, q, k, v, a, b, dsT)]
        _launch('attn_f32_backward', _attn_f32_backward_impl, w, q, k, v, a, b, dy, s, dsT, dw, dq, dk, dv, da, db, ds0)
        return dw, dq, dk, dv, da, db, ds0


@torch.compiler.assume_constant_result
def _f32_saved_bytes(B, T, H, C):
    saved = _native.lib().wind_rwkv7_attn_f32_saved_bytes(B, T, H, C)
    if saved == 0:   # name the problem
        if not _native.lib().wind_rwkv7_f32_head_size_supported(C):
            _native.check(3)
        if T % 16:
            _native.check(4)
        _native.check(2)
    return saved


@torch.compiler.assume_constant_result
def _f32_saved_unit(C):
    """floats of the saved tensor per (batch, head, 16 tokens)"""
    return _f32_saved_bytes(1, 16, 1, C) // 4


@torch.compiler.assume_constant_result
def _bf16_head(HEAD_SIZE):
    """True where the bf16 matrix-core kernels cover this head size (64)."""
    return bool(_native.lib().wind_rwkv7_head_size_supported(int(HEAD_SIZE)))


@torch.compiler.assume_constant_result
def _attn_bf16_head(HEAD_SIZE):
    """True where the plain WKV7 operator has bf16 matrix-core kernels for this head size (multiples of 16 up to 128)."""
    return bool(_native.lib().wind_rwkv7_attn_head_size_supported(int(HEAD_SIZE)))


@torch.compiler.assume_constant_result
def load_attn(HEAD_SIZE):
    """Reference: JIT-compiles the CUDA extension for one head size (rwkv7_attn.py:46-51).
    Here the library is prebuilt; this loads it and checks that some kernel covers the head size."""
    if not _attn_bf16_head(HEAD_SIZE) and not _native.lib().wind_rwkv7_f32_head_size_supported(int(HEAD_SIZE)):
        _native.check(3)


def _any_length(run_chunks, run_token, seqs, s0, H, C):
    """Inference over T tokens, T no multiple of 16: the longest prefix of whole chunks through the sequence kernels
    (`run_chunks(seqs, state) -> (y, state)`), the remaining tokens through the single-token kernel
    (`run_token(tokens, state) -> y`, state updated in place).  The state is carried in fp32."""
    B, T, HC = seqs[0].shape
    T0 = T - T % 16
    state = torch.zeros(B, H, C, C, dtype=torch.float32, device=seqs[0].device) if s0 is None else s0
    ys = []
    if T0:
        y, state = run_chunks([x[:, :T0].contiguous() for x in seqs], state)
        ys.append(y)
    elif s0 is not None:
        state = s0.clone()       # the caller's tensor stays as it is
    for t in range(T0, T):
        ys.append(run_token([x[:, t].contiguous() for x in seqs], state).view(B, 1, HC))
    return torch.cat(ys, dim=1), state


def attn(r, w, k, v, a, b, HEAD_SIZE, s0=None, return_state=False):
    """y = WKV7(r,w,k,v,a,b); all [B,T,H*HEAD_SIZE] bf16 (rwkv7_attn.py:53-59), or all float32 for the fp32
    kernels (slower; fp32 arithmetic and state throughout, as the reference's Triton variant with dot_prec='fp32').

    As in the reference the initial state is zero and only y is returned.  Beyond it: `s0` ([B,H,C,C], fp32
    or bf16) continues from a carried state and `return_state=True` returns (y, sT), so a long sequence can
    be run in pieces and a prompt's final state handed to `attn_step`.  When nothing is differentiated T need not
    be a multiple of 16 (bf16 tensors): the tokens after the last whole chunk run through `attn_step`.

    Head sizes: multiples of 16 up to 128 (the reference compiles its CUDA kernel per head size,
    rwkv7_attn.py:46-51, and has rwkv7_attn_triton_bighead.py for large ones).  bf16 sequences run matrix-core
    kernels at every one of them: the fused kernels at 64, the three-phase kernels of csrc/wkv7_wide.hip at the
    others."""
    B, T, HC = w.shape
    C = HEAD_SIZE
    H = HC // C
    if T % 16 and w.dtype == torch.bfloat16 and _attn_bf16_head(C) and not _differentiating(r, w, k, v, a, b):
        # inference on a length that is no multiple of the chunk: see _any_length
        y, sT = _any_length(lambda xs, st: attn(*xs, C, s0=st, return_state=True),
                            lambda xs, st: attn_step(*xs, st, C), (r, w, k, v, a, b), s0, H, C)
        return (y, sT) if return_state else y
    r, w, k, v, a, b = [x.view(B, T, H, C) for x in (r, w, k, v, a, b)]
    if w.dtype == torch.float32 or not _attn_bf16_head(C):
        # float32 sequences select the fp32 kernels (float32 state in and out)
        s0 = torch.zeros(B, H, C, C, dtype=torch.float32, device=w.device) if s0 is None else s0.float()
        seqs = [x.float() for x in (w, r, k, v, a, b)]
        if _differentiating(*seqs, s0):
            y, sT, _ = WindRWKV7F32.apply(*seqs, s0)
        else:
            y, sT = fw_attn_f32_no_grad(*[x.contiguous() for x in seqs], s0.contiguous())
        y = y.to(v.dtype)
    else:
        if s0 is None:   # the kernels take "no initial state" as such
            s0 = no_state(torch.bfloat16, w.device)
        if _differentiating(w, r, k, v, a, b, s0):
            y, sT, _ = WindRWKV7.apply(w, r, k, v, a, b, s0)
        else:   # nothing will be differentiated: the forward that keeps nothing for a backward pass
            _check_sequences((w, r, k, v, a, b), s0)
            y, sT, _ = fw_attn(w, r, k, v, a, b, s0, save=False)
    y = y.view(B, T, HC)
    return (y, sT) if return_state else y


_OPS.define('attn_decode(Tensor w, Tensor q, Tensor k, Tensor v, Tensor a, Tensor b, Tensor(a!) state, Tensor(b!) y) -> ()')


def _attn_decode_impl(w, q, k, v, a, b, state, y):
    B, H, C = w.shape
    with torch.cuda.device(w.device):
        _native.check(_native.lib().wind_rwkv7_attn_decode(
            B, H, C, _native.BF16, _state_code(state), w.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            a.data_ptr(), b.data_ptr(), state.data_ptr(), y.data_ptr(), _stream(w)))


_OPS.impl('attn_decode', _attn_decode_impl, 'CUDA')
_OPS.impl('attn_decode', _no_cpu, 'CPU')
_OPS.impl('attn_decode', lambda *a: None, 'Meta')


def _check_step(seqs, state, B, H, C):
    assert all(x.dtype == torch.bfloat16 and x.is_contiguous() and x.numel() == B * H * C for x in seqs), \
        'one-token inputs must be contiguous bfloat16 [B, H*HEAD_SIZE]'
    assert state.dtype in _STATE_DTYPES and state.is_contiguous() and tuple(state.shape) == (B, H, C, C), \
        'state must be a contiguous [B,H,C,C] float32 or bfloat16 tensor'


def attn_step(r, w, k, v, a, b, state, HEAD_SIZE):
    """One token of WKV7 per sequence (decoding): r,w,k,v,a,b are [B, H*HEAD_SIZE] bf16, `state` [B,H,C,C]
    (fp32 or bf16) is updated IN PLACE and y [B, H*HEAD_SIZE] is returned.  Inference only (no autograd).
    The reference offers only the PyTorch token loop for this (ref_attn, time_mixer.py:6-16)."""
    B, HC = w.shape
    C = int(HEAD_SIZE)
    H = HC // C
    if not torch.compiler.is_compiling():
        _check_step((r, w, k, v, a, b), state, B, H, C)
    y = torch.empty_like(v)
    with torch.no_grad():
        _launch('attn_decode', _attn_decode_impl, *[x.view(B, H, C) for x in (w, r, k, v, a, b)], state, y.view(B, H, C))
    return y


def attn_triton(r, w, k, v, a, b, HEAD_SIZE, dot_prec='fp32'):
    """Name kept from the reference's Triton variant (rwkv7_attn_triton.py:192-198).  There is no Triton here.
    `dot_prec` keeps its meaning (:182-190): 'fp32' runs the fp32 kernels (inputs of any float dtype are taken
    to float32 and the result comes back in the inputs' dtype); 'tf32' and 'bf16' run the bf16 matrix-core
    kernels of `attn` (this hardware has no tf32 matrix instruction; bf16 inputs required) where they cover the
    head size, and the fp32 kernels otherwise."""
    if dot_prec not in ('fp32', 'tf32', 'bf16'):
        raise ValueError(f"dot_prec must be 'fp32', 'tf32' or 'bf16', got {dot_prec!r}")
    if dot_prec == 'fp32':
        return attn(*(x.float() for x in (r, w, k, v, a, b)), HEAD_SIZE).to(v.dtype)
    return attn(r, w, k, v, a, b, HEAD_SIZE)


def attn_triton_bighead(r, w, k, v, a, b, HEAD_SIZE, dot_prec='fp32'):
    """The reference's large-head Triton variant (rwkv7_attn_triton_bighead.py:363-372: any head size that is
    a multiple of 16, global scratch instead of shared memory).  Here head sizes 16 .. 128 in steps of 16: with the
    reference's default dot_prec='fp32' the fp32 kernels (at C = 128 the state of a head in the registers of two
    256-thread blocks), with 'bf16' / 'tf32' the bf16 matrix-core kernels for those head sizes (about eight times
    faster at C = 128); larger heads are rejected with WIND_RWKV7_ERR_HEAD_SIZE.  `dot_prec` as in `attn_triton`."""
    load_attn(HEAD_SIZE)
    return attn_triton(r, w, k, v, a, b, HEAD_SIZE, dot_prec)
