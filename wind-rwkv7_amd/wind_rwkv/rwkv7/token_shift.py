"""ddlerp: data-dependent token-shift interpolation (the four mixed input streams of the time mixer).

Mirrors the reference's rwkv7_ddlerp.py: ``ddlerp(x, alpha, L, R, beta) -> (y0, y1, y2, y3)`` (:306-336).
x [B,T,C] bf16; alpha [C]; L [4D,C]; R [4,C,D]; beta [4,1,1,C]; any rank D (the reference reads it from the shapes, :311): the
kernels have ranks 32 and 64, a smaller rank is zero-padded, a larger one runs in pieces (`ddlerp` below).  Parameters may be fp32 (they are cast to
bf16 for the kernels, as the reference does at :309); their gradients come back in fp32.
"""
import torch

from .. import _native
from .wkv_attn import _OPS, _flat_views, _grads_like, _launch, _no_cpu, _params_as_bf16, _sized, _stream, _workspace

_OPS.define('ddlerp_forward(Tensor x, Tensor alpha, Tensor L, Tensor R, Tensor beta, Tensor(a!) bmid, Tensor(b!) bder, Tensor(c!) y) -> ()')
_OPS.define('ddlerp_backward(Tensor x, Tensor alpha, Tensor L, Tensor R, Tensor beta, Tensor bmid, Tensor bder, Tensor dy0, '
            'Tensor dy1, Tensor dy2, Tensor dy3, Tensor(a!) dx, Tensor(b!) dalpha, Tensor(c!) dL, Tensor(d!) dR, '
            'Tensor(e!) dbeta, Tensor(f!) workspace) -> ()')


def _fwd_impl(x, alpha, L, R, beta, bmid, bder, y):
    B, T, C = x.shape
    D = R.shape[2]
    with torch.cuda.device(x.device):
        _native.check(_native.lib().wind_rwkv7_ddlerp_forward(
            B, T, C, D, x.data_ptr(), alpha.data_ptr(), L.data_ptr(), R.data_ptr(), beta.data_ptr(),
            bmid.data_ptr(), bder.data_ptr(), y.data_ptr(), _stream(x)))


def _bwd_impl(x, alpha, L, R, beta, bmid, bder, dy0, dy1, dy2, dy3, dx, dalpha, dL, dR, dbeta, workspace):
    B, T, C = x.shape
    D = R.shape[2]
    workspace = _sized(workspace, _native.lib().wind_rwkv7_ddlerp_bwd_workspace_bytes(B, T, C, D))
    with torch.cuda.device(x.device):
        _native.check(_native.lib().wind_rwkv7_ddlerp_backward(
            B, T, C, D, x.data_ptr(), alpha.data_ptr(), L.data_ptr(), R.data_ptr(), beta.data_ptr(), bmid.data_ptr(),
            bder.data_ptr(), dy0.data_ptr(), dy1.data_ptr(), dy2.data_ptr(), dy3.data_ptr(),
            dx.data_ptr(), dalpha.data_ptr(), dL.data_ptr(), dR.data_ptr(), dbeta.data_ptr(),
            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(x)))


for _name, _impl in (('ddlerp_forward', _fwd_impl), ('ddlerp_backward', _bwd_impl)):
    _OPS.impl(_name, _impl, 'CUDA')
    _OPS.impl(_name, _no_cpu, 'CPU')
    _OPS.impl(_name, lambda *a: None, 'Meta')


@torch.compiler.assume_constant_result
def _bwd_workspace_bytes(B, T, C, D):
    return _native.lib().wind_rwkv7_ddlerp_bwd_workspace_bytes(B, T, C, D)


def _kernel_rank(D):
    """The rank the kernels run a LoRA of rank D at: 32 and 64 as they are, a smaller one zero-padded to the next of the
    two (a zero column of L gives tanh(0) = 0 against a zero row of R: the same result, and its gradients are dropped).
    Above 64 the library reports the rank as unsupported."""
    return 32 if D < 32 else 64 if 32 < D < 64 else D


class DDLerp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, alpha, L, R, beta):
        ctx.param_dtype = alpha.dtype
        alpha, L, R, beta = _params_as_bf16((alpha, L, R, beta))
        B, T, C = x.shape
        D = ctx.rank = R.shape[2]
        if not torch.compiler.is_compiling():
            assert tuple(L.shape) == (4 * D, C), 'L must be [4D,C]'
            assert tuple(R.shape) == (4, C, D), 'R must be [4,C,D]'
        if _kernel_rank(D) != D:
            Dp = _kernel_rank(D)
            L = torch.nn.functional.pad(L.reshape(4, D, C), (0, 0, 0, Dp - D)).view(4 * Dp, C)
            R = torch.nn.functional.pad(R, (0, Dp - D))
            D = Dp
        if not torch.compiler.is_compiling():
            assert x.dtype == torch.bfloat16 and x.is_contiguous(), 'x must be contiguous bfloat16'
            assert tuple(alpha.shape) == (C,), 'alpha must be [C]'
            assert tuple(beta.shape) == (4, 1, 1, C), 'beta must be [4,1,1,C]'
        bmid = torch.empty(B, T, 4 * D, dtype=torch.bfloat16, device=x.device)
        bder = torch.empty_like(bmid)
        y = torch.empty(4, B, T, C, dtype=torch.bfloat16, device=x.device)
        _launch('ddlerp_forward', _fwd_impl, x, alpha, L, R, beta, bmid, bder, y)
        ctx.save_for_backward(x, alpha, L, R, beta, bmid, bder)
        return y.unbind(dim=0)

    @staticmethod
    def backward(ctx, dy0, dy1, dy2, dy3):
        x, alpha, L, R, beta, bmid, bder = ctx.saved_tensors
        B, T, C = x.shape
        D = R.shape[2]
        dys = [torch.zeros_like(x) if g is None else g.contiguous() for g in (dy0, dy1, dy2, dy3)]
        dx = torch.empty_like(x)
        flat, (dalpha, dL, dR, dbeta) = _flat_views([(C,), (4 * D, C), (4, C, D), (4, 1, 1, C)], torch.float32, x.device)
        ws = _workspace(lambda: _bwd_workspace_bytes(B, T, C, D), x.device)
        _launch('ddlerp_backward', _bwd_impl, x, alpha, L, R, beta, bmid, bder, *dys, dx, dalpha, dL, dR, dbeta, ws)
        # parameter gradients leave the kernels in fp32 (the reference: dL fp32, the others bf16,
        # rwkv7_ddlerp.py:265,301); they are handed back in the parameters' own dtype so autograd adds no casts
        dalpha, dL, dR, dbeta = _grads_like(flat, [dalpha, dL, dR, dbeta], ctx.param_dtype)
        if ctx.rank != D:   # a padded rank: the padding's gradients are dropped
            dL = dL.view(4, D, C)[:, :ctx.rank].reshape(4 * ctx.rank, C)
            dR = dR[..., :ctx.rank].contiguous()
        return dx, dalpha, dL, dR, dbeta


def ddlerp(x, alpha, L, R, beta):
    """ddlerp(x, alpha, L, R, beta) -> (y0, y1, y2, y3), rwkv7_ddlerp.py:306-336.  A LoRA rank above 64 runs as pieces of
    at most 64: the interpolation weight is a sum over the rank, c_k = sum_d bmid[k,d] R[k,:,d] + beta_k, so with the
    rank cut in n pieces (beta in the first one only) y_k = sum_i y_k^(i) - (n - 1) x.  The pieces are added in fp32."""
    D = R.shape[2]
    if D <= 64:
        return DDLerp.apply(x, alpha, L, R, beta)
    C = x.shape[-1]
    cuts = list(range(0, D, 64)) + [D]
    L4 = L.reshape(4, D, C)
    acc = None
    for i, (lo, hi) in enumerate(zip(cuts[:-1], cuts[1:])):
        piece = DDLerp.apply(x, alpha, L4[:, lo:hi].reshape(4 * (hi - lo), C), R[..., lo:hi].contiguous(),
                             beta if i == 0 else torch.zeros_like(beta))
        piece = torch.stack(piece).float()
        acc = piece if acc is None else acc + piece
    y = (acc - (len(cuts) - 2) * x.float()).to(x.dtype)
    return y.unbind(dim=0)
