"""expand_loras: the four rank-D LoRA expansions of the time mixer and the elementwise tail producing the
WKV7 operands (w, k, kk, b).

Mirrors the reference's rwkv7_expand_loras.py:
``expand_loras(w_in,k_in,z_in,a_in,ma_in,mk_in, Wz,Wa,Wma,Wmk, w_bias,a_bias,ma_bias,mk_bias, HEAD_SIZE)
-> (w, k, kk, b)`` (:214-241).  Weights and biases may be fp32 (cast to bf16 for the kernels as at :218);
their gradients come back in fp32.
"""
import torch

from .. import _native
from .wkv_attn import _OPS, _flat_views, _grads_like, _launch, _no_cpu, _params_as_bf16, _sized, _stream, _workspace

_IN = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias', 'ma_bias', 'mk_bias']
_OUT = ['w_out', 'k_out', 'kk_out', 'b_out']
_GRAD = ['dw_in', 'dk_in', 'dz_in', 'da_in', 'dma_in', 'dmk_in', 'dWz', 'dWa', 'dWma', 'dWmk', 'dw_bias', 'da_bias',
         'dma_bias', 'dmk_bias']
_LET = 'abcdefghijklmnopqrstuvwxyz'
_OPS.define('expand_loras_forward(' + ', '.join(f'Tensor {n}' for n in _IN) + ', int head_size, '
            + ', '.join(f'Tensor({_LET[i]}!) {n}' for i, n in enumerate(_OUT)) + ') -> ()')
_OPS.define('expand_loras_backward(' + ', '.join(f'Tensor {n}' for n in _IN) + ', int head_size, '
            + ', '.join(f'Tensor d{n}' for n in _OUT) + ', '
            + ', '.join(f'Tensor({_LET[i]}!) {n}' for i, n in enumerate(_GRAD + ['workspace'])) + ') -> ()')


def _fwd_impl(*args):
    ins, head_size, outs = args[:14], args[14], args[15:]
    B, T, C = ins[0].shape
    D = ins[2].shape[2]
    with torch.cuda.device(ins[0].device):
        _native.check(_native.lib().wind_rwkv7_expand_loras_forward(
            B, T, C, D, head_size, *[t.data_ptr() for t in ins], *[t.data_ptr() for t in outs], _stream(ins[0])))


def _bwd_impl(*args):
    ins, head_size, dys, grads, ws = args[:14], args[14], args[15:19], args[19:33], args[33]
    B, T, C = ins[0].shape
    D = ins[2].shape[2]
    ws = _sized(ws, _native.lib().wind_rwkv7_expand_loras_bwd_workspace_bytes(B, T, C, D))
    with torch.cuda.device(ins[0].device):
        _native.check(_native.lib().wind_rwkv7_expand_loras_backward(
            B, T, C, D, head_size, *[t.data_ptr() for t in ins], *[t.data_ptr() for t in dys],
            *[t.data_ptr() for t in grads], ws.data_ptr(), ws.numel() * ws.element_size(), _stream(ins[0])))


for _name, _impl in (('expand_loras_forward', _fwd_impl), ('expand_loras_backward', _bwd_impl)):
    _OPS.impl(_name, _impl, 'CUDA')
    _OPS.impl(_name, _no_cpu, 'CPU')
    _OPS.impl(_name, lambda *a: None, 'Meta')


@torch.compiler.assume_constant_result
def _bwd_workspace_bytes(B, T, C, D):
    return _native.lib().wind_rwkv7_expand_loras_bwd_workspace_bytes(B, T, C, D)


class ExpandLoras(torch.autograd.Function):
    @staticmethod
    def forward(ctx, w_in, k_in, z_in, a_in, ma_in, mk_in, Wz, Wa, Wma, Wmk, w_bias, a_bias, ma_bias, mk_bias, HEAD_SIZE):
        acts = [t.contiguous() for t in (z_in, a_in, ma_in, mk_in)]
        ctx.param_dtype = Wz.dtype
        params = _params_as_bf16((Wz, Wa, Wma, Wmk, w_bias, a_bias, ma_bias, mk_bias))
        ins = [w_in, k_in] + acts + params
        B, T, C = w_in.shape
        D = acts[0].shape[2]
        if not torch.compiler.is_compiling():
            assert all(t.dtype == torch.bfloat16 for t in ins), 'activations must be bfloat16'
            assert w_in.is_contiguous() and k_in.is_contiguous(), 'w_in and k_in must be contiguous'
            assert tuple(k_in.shape) == (B, T, C)
            assert all(tuple(t.shape) == (B, T, D) for t in acts)
            assert all(tuple(t.shape) == (C, D) for t in params[:4])
            assert all(tuple(t.shape) == (C,) for t in params[4:])
        outs = [torch.empty_like(w_in) for _ in range(4)]
        _launch('expand_loras_forward', _fwd_impl, *ins, int(HEAD_SIZE), *outs)
        ctx.save_for_backward(*ins)
        ctx.head_size = int(HEAD_SIZE)
        return tuple(outs)

    @staticmethod
    def backward(ctx, dw_out, dk_out, dkk_out, db_out):
        ins = ctx.saved_tensors
        w_in = ins[0]
        B, T, C = w_in.shape
        D = ins[2].shape[2]
        dys = [torch.zeros_like(w_in) if g is None else g.contiguous() for g in (dw_out, dk_out, dkk_out, db_out)]
        if not torch.compiler.is_compiling():
            assert all(g.dtype == torch.bfloat16 for g in dys)
        flat, pgrads = _flat_views([(C, D)] * 4 + [(C,)] * 4, torch.float32, w_in.device)
        grads = [torch.empty_like(w_in) for _ in range(2)] + [torch.empty_like(ins[2]) for _ in range(4)] + pgrads
        ws = _workspace(lambda: _bwd_workspace_bytes(B, T, C, D), w_in.device)
        _launch('expand_loras_backward', _bwd_impl, *ins, ctx.head_size, *dys, *grads, ws)
        # weight and bias gradients leave the kernels in fp32 (as in the reference, rwkv7_expand_loras.py:200-201)
        # and are handed back in the parameters' own dtype so autograd adds no casts
        return (*grads[:6], *_grads_like(flat, pgrads, ctx.param_dtype), None)


expand_loras = ExpandLoras.apply
