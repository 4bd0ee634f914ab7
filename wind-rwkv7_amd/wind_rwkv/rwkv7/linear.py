"""Bias-free projections of the time-mixer with this package's weight-gradient kernel.

The reference writes its projections as plain matmuls, ``x @ W.mT`` (time_mixer.py:120-131, :167), and leaves
all three products to the BLAS library through autograd.  The forward product and the input gradient are
ordinary GEMMs and stay there; the weight gradient contracts over the tokens, the slow index of both operands,
with a small output (C x C or C x rank), a shape the library handles poorly.  ``projection`` is the same
function with that one product on the package's kernel, which also writes the gradient in the weight's own
dtype (no bf16 detour for fp32 master weights).
"""
import torch

from .. import _native
from .wkv_attn import _OPS, _differentiating, _launch, _no_cpu, _sized, _stream, _workspace


_OPS.define('linear_wgrad(Tensor dy, Tensor x, Tensor(a!) dW, Tensor(b!) workspace) -> ()')
_OPS.define('linear_wgrad_group(Tensor[] dy, Tensor[] x, Tensor(a!)[] dW, Tensor(b!) workspace) -> ()')
_OPS.define('cast_to_bf16(Tensor[] srcs, Tensor(a!) flat, int[]? offsets) -> ()')
_OPS.define('copy_columns(int M, Tensor?[] src, int[] src_ld, int[] src_col0, Tensor(a!)[] dst, int[] dst_ld, '
            'int[] dst_col0, int[] width, int[] op, Tensor?[] aux) -> ()')


def _linear_wgrad_impl(dy2, x2, dW, ws):
    O, I = dW.shape
    ws = _sized(ws, max(_native.lib().wind_rwkv7_linear_wgrad_workspace_bytes(dy2.shape[0], O, I), 256))
    with torch.cuda.device(dy2.device):
        _native.check(_native.lib().wind_rwkv7_linear_wgrad(
            dy2.shape[0], O, I, dy2.data_ptr(), dy2.stride(0), x2.data_ptr(), x2.stride(0), dW.data_ptr(),
            _native.F32 if dW.dtype == torch.float32 else _native.BF16, ws.data_ptr(), ws.numel(), _stream(dy2)))


def _group_arrays(dW):
    import ctypes
    n = len(dW)
    return n, (ctypes.c_int * n)(*[w.shape[0] for w in dW]), (ctypes.c_int * n)(*[w.shape[1] for w in dW])


def _linear_wgrad_group_impl(dy, x, dW, ws):
    import ctypes
    n, O, I = _group_arrays(dW)
    tokens = dy[0].shape[0]
    lib = _native.lib()
    ws = _sized(ws, max(lib.wind_rwkv7_linear_wgrad_group_workspace_bytes(n, tokens, O, I), 256))
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    lds = lambda ts: (ctypes.c_longlong * n)(*[t.stride(0) for t in ts])
    with torch.cuda.device(dy[0].device):
        _native.check(lib.wind_rwkv7_linear_wgrad_group(
            n, tokens, O, I, ptrs(dy), lds(dy), ptrs(x), lds(x), ptrs(dW),
            _native.F32 if dW[0].dtype == torch.float32 else _native.BF16, ws.data_ptr(), ws.numel(), _stream(dy[0])))


def _cast_to_bf16_impl(srcs, flat, offsets):
    import ctypes
    n = len(srcs)
    ptrs = (ctypes.c_void_p * n)(*[w.data_ptr() for w in srcs])
    dtypes = (ctypes.c_int * n)(*[_native.F32 if w.dtype == torch.float32 else _native.BF16 for w in srcs])
    numel = (ctypes.c_longlong * n)(*[w.numel() for w in srcs])
    offs = None if offsets is None else (ctypes.c_longlong * n)(*offsets)
    with torch.cuda.device(flat.device):
        _native.check(_native.lib().wind_rwkv7_cast_to_bf16(n, ptrs, dtypes, numel, offs, flat.data_ptr(), _stream(flat)))


def _copy_columns_impl(M, src, src_ld, src_col0, dst, dst_ld, dst_col0, width, op, aux):
    anchor = dst[0]
    import ctypes
    n = len(dst)
    arr = lambda ctype, vals: (ctype * n)(*vals)
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(anchor.device):
        _native.check(_native.lib().wind_rwkv7_copy_columns(
            M, n, arr(ctypes.c_void_p, [ptr(t) for t in src]), arr(ctypes.c_longlong, src_ld), arr(ctypes.c_int, src_col0),
            arr(ctypes.c_void_p, [ptr(t) for t in dst]), arr(ctypes.c_longlong, dst_ld), arr(ctypes.c_int, dst_col0),
            arr(ctypes.c_int, width), arr(ctypes.c_int, op), arr(ctypes.c_void_p, [ptr(t) for t in aux]), _stream(anchor)))


for _name, _impl in (('linear_wgrad', _linear_wgrad_impl), ('linear_wgrad_group', _linear_wgrad_group_impl),
                     ('cast_to_bf16', _cast_to_bf16_impl),
                     ('copy_columns', _copy_columns_impl)):
    _OPS.impl(_name, _impl, 'CUDA')
    _OPS.impl(_name, _no_cpu, 'CPU')
    _OPS.impl(_name, lambda *a: None, 'Meta')


@torch.compiler.assume_constant_result
def _wgrad_workspace_bytes(tokens, O, I):
    return _native.lib().wind_rwkv7_linear_wgrad_workspace_bytes(tokens, O, I)


def _rows(t):
    """[..., W] -> a 2-D view (or copy) with unit column stride and a row stride that is a multiple of 8 elements.
    (Tensors from the framework's allocator start 16-byte aligned; the library checks.)"""
    t2 = t.reshape(-1, t.shape[-1])
    if t2.stride(1) != 1 or t2.stride(0) % 8:
        t2 = t2.contiguous()
    elif not torch.compiler.is_compiling() and t2.storage_offset() % 8:   # (the tracer cannot read the offset)
        t2 = t2.contiguous()
    return t2


def linear_wgrad(dy, x, out_dtype=torch.float32):
    """dW [O, I] = dy^T x for token-major bf16 dy [..., O] and x [..., I]; fp32 accumulation, fixed order."""
    if dy.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise TypeError('linear_wgrad: dy and x must be bfloat16')
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise TypeError('linear_wgrad: out_dtype must be float32 or bfloat16')
    O, I = dy.shape[-1], x.shape[-1]
    dy2, x2 = _rows(dy), _rows(x)
    if dy2.shape[0] != x2.shape[0]:
        raise ValueError('linear_wgrad: dy and x must have the same number of tokens')
    tokens = dy2.shape[0]
    dW = torch.empty(O, I, device=dy.device, dtype=out_dtype)
    if tokens == 0:
        return dW.zero_()
    ws = _workspace(lambda: max(_wgrad_workspace_bytes(tokens, O, I), 256), dy.device)
    _launch('linear_wgrad', _linear_wgrad_impl, dy2, x2, dW, ws)
    return dW


def _bf16_rows(weights, wb):
    """The bf16 row-wise concatenation of `weights` (or `wb`, the copy that already exists)."""
    if wb is not None:
        return wb
    return weights[0].to(torch.bfloat16) if len(weights) == 1 else torch.cat([w.to(torch.bfloat16) for w in weights])


@torch.compiler.assume_constant_result
def _wgrad_group_workspace_bytes(tokens, Os, Is):
    import ctypes
    n = len(Os)
    return _native.lib().wind_rwkv7_linear_wgrad_group_workspace_bytes(n, tokens, (ctypes.c_int * n)(*Os), (ctypes.c_int * n)(*Is))


GROUP_MAX = 8   # problems per grouped launch (the library's limit)


def linear_wgrad_group(dys, xs, out_dtype=torch.float32):
    """[dW_j = dy_j^T x_j] for up to eight (dy_j [..., O_j], x_j [..., I_j]) bf16 pairs with the same number of
    tokens: one launch for all products and one for the sums of their partial tiles, where separate `linear_wgrad`
    calls take two launches each and (three 768 x 768 products) write three times as many partial tiles.  More
    pairs go in batches of eight; a single pair, or pairs with different token counts, through `linear_wgrad`."""
    n = len(dys)
    assert n == len(xs)
    if n > GROUP_MAX:
        return (linear_wgrad_group(dys[:GROUP_MAX], xs[:GROUP_MAX], out_dtype)
                + linear_wgrad_group(dys[GROUP_MAX:], xs[GROUP_MAX:], out_dtype))
    ok = (2 <= n and out_dtype in (torch.float32, torch.bfloat16)
          and all(t.dtype == torch.bfloat16 for t in tuple(dys) + tuple(xs))
          and all(dy.shape[-1] % 16 == 0 and x.shape[-1] % 16 == 0 for dy, x in zip(dys, xs)))
    dy2, x2 = [_rows(t) for t in dys], [_rows(t) for t in xs]
    tokens = dy2[0].shape[0] if n else 0
    ok = ok and tokens > 0 and all(t.shape[0] == tokens for t in dy2 + x2)
    if not ok:
        return [linear_wgrad(dy, x, out_dtype) for dy, x in zip(dys, xs)]
    dW = [torch.empty(dy.shape[-1], x.shape[-1], device=dy.device, dtype=out_dtype) for dy, x in zip(dy2, x2)]
    Os, Is = tuple(w.shape[0] for w in dW), tuple(w.shape[1] for w in dW)
    ws = _workspace(lambda: max(_wgrad_group_workspace_bytes(tokens, Os, Is), 256), dy2[0].device)
    _launch('linear_wgrad_group', _linear_wgrad_group_impl, dy2, x2, dW, ws)
    return dW


class Projection(torch.autograd.Function):
    """y = x @ cat(weights).mT in bf16; the weights may be fp32 or bf16 and receive gradients of their own dtype."""

    @staticmethod
    def forward(ctx, x, wb, *weights):
        if wb is None:
            wb = weights[0].to(torch.bfloat16) if len(weights) == 1 else torch.cat([w.to(torch.bfloat16) for w in weights])
        ctx.save_for_backward(x, wb)
        ctx.rows = [w.shape[0] for w in weights]
        ctx.dtypes = [w.dtype for w in weights]
        ctx.needs = ctx.needs_input_grad
        return x @ wb.mT

    @staticmethod
    def backward(ctx, dy):
        x, wb = ctx.saved_tensors
        dy = dy.contiguous()
        dx = dy @ wb if ctx.needs[0] else None
        if not any(ctx.needs[2:]):
            return (dx, None) + (None,) * len(ctx.rows)
        same = all(d == ctx.dtypes[0] for d in ctx.dtypes)
        dW = linear_wgrad(dy, x, ctx.dtypes[0] if same and ctx.dtypes[0] in (torch.float32, torch.bfloat16) else torch.float32)
        parts = dW.split(ctx.rows)
        return (dx, None) + tuple(p.to(d) if need else None for p, d, need in zip(parts, ctx.dtypes, ctx.needs[2:]))


def projection(x, *weights, bf16=None):
    """x [..., I] bf16 times the row-wise concatenation of `weights` ([O_k, I] each), transposed: [..., sum O_k].
    `bf16`: an existing bf16 copy of that concatenation ([sum O_k, I], see `bf16_copies`), to skip the casts."""
    if not _differentiating(x, *weights):    # inference: the product alone, no autograd node
        return x @ _bf16_rows(weights, bf16).mT
    return Projection.apply(x, bf16, *weights)


class ProjectionSets(torch.autograd.Function):
    """Several projections of several inputs: y = x_i @ cat(weights of the group).mT for every weight group of every
    input x_i (same number of tokens in all).

    One Function instead of one per product, so that the backward sees all upstream gradients at once: it folds
    the sum of an input's gradients into the matrix products (dx = dy_0 W_0, then dx += dy_g W_g as the
    accumulating form of the product) instead of leaving elementwise adds of [tokens, I] tensors to autograd, and
    it computes the weight gradients of all groups in one grouped launch (`linear_wgrad_group`)."""

    @staticmethod
    def forward(ctx, layout, wbs, *tensors):
        # layout[i] = the group sizes of input i; tensors = the inputs, then all weights in order
        xs, weights = tensors[:len(layout)], tensors[len(layout):]
        groups, i = [], 0
        for sizes in layout:
            for n in sizes:
                groups.append(weights[i:i + n])
                i += n
        if wbs is None:
            wbs = [_bf16_rows(g, None) for g in groups]
        ctx.save_for_backward(*xs, *wbs)
        ctx.layout = layout
        ctx.rows = [w.shape[0] for w in weights]
        ctx.dtypes = [w.dtype for w in weights]
        ctx.needs = ctx.needs_input_grad
        ctx.set_materialize_grads(False)
        owner = [i for i, sizes in enumerate(layout) for _ in sizes]
        return tuple(xs[i] @ wb.mT for i, wb in zip(owner, wbs))

    @staticmethod
    def backward(ctx, *dys):
        nx = len(ctx.layout)
        xs, wbs = ctx.saved_tensors[:nx], ctx.saved_tensors[nx:]
        dxs, pending, grads = [], [], [None] * len(ctx.rows)
        g, w0 = 0, 0     # running indices of the group and of its first weight
        for i, sizes in enumerate(ctx.layout):
            x2, dx = xs[i].reshape(-1, xs[i].shape[-1]), None
            for n in sizes:
                wb, dy = wbs[g], dys[g]
                span = range(w0, w0 + n)
                g, w0 = g + 1, w0 + n
                if dy is None:
                    continue
                dy2 = dy.reshape(-1, dy.shape[-1]).contiguous()
                if ctx.needs[2 + i]:
                    dx = dy2 @ wb if dx is None else dx.addmm_(dy2, wb)   # in place: no copy of dx
                if any(ctx.needs[2 + nx + k] for k in span):
                    dts = [ctx.dtypes[k] for k in span]
                    same = all(d == dts[0] for d in dts) and dts[0] in (torch.float32, torch.bfloat16)
                    pending.append((dy2, x2, dts[0] if same else torch.float32, span))
            if dx is not None:
                dx = dx.view(xs[i].shape)
            elif ctx.needs[2 + i]:
                dx = torch.zeros_like(xs[i])
            dxs.append(dx)
        for dt in (torch.float32, torch.bfloat16):     # one grouped launch per result dtype
            jobs = [j for j in pending if j[2] == dt]
            if not jobs:
                continue
            for (_, _, _, span), dW in zip(jobs, linear_wgrad_group([j[0] for j in jobs], [j[1] for j in jobs], dt)):
                for k, part in zip(span, dW.split([ctx.rows[k] for k in span])):
                    if ctx.needs[2 + nx + k]:
                        grads[k] = part.to(ctx.dtypes[k])
        return (None, None) + tuple(dxs) + tuple(grads)


def projection_sets(inputs, bf16=None):
    """`inputs` = [(x_i, [group, ...]), ...] with x_i [..., I_i] bf16 and each group a list of [O_k, I_i] weights:
    per input a tuple with one output per group, x_i times the row-wise concatenation of the group's weights,
    transposed.  `bf16`: existing bf16 copies of the concatenations, one list per input (see `bf16_copies`).
    Equal to a `projection` per group, with the input gradients of an input's groups accumulated inside the matrix
    products and all weight gradients of the set computed in one grouped launch."""
    layout = tuple(tuple(len(g) for g in groups) for _, groups in inputs)
    xs = [x for x, _ in inputs]
    weights = [w for _, groups in inputs for g in groups for w in g]
    flat_bf16 = None if bf16 is None else [wb for per_input in bf16 for wb in per_input]
    if not _differentiating(*xs, *weights):
        flat = [x @ _bf16_rows(g, None if flat_bf16 is None else flat_bf16[k]).mT
                for k, (x, g) in enumerate((x, g) for x, groups in inputs for g in groups)]
    else:
        flat = ProjectionSets.apply(layout, flat_bf16, *xs, *weights)
    outs, k = [], 0
    for sizes in layout:
        outs.append(tuple(flat[k:k + len(sizes)]))
        k += len(sizes)
    return outs


def projections(x, *groups, bf16=None):
    """One output per group: x [..., I] bf16 times the row-wise concatenation of the group's weights, transposed.
    `projections(x, [Wr], [W1, W2])` equals `(projection(x, Wr), projection(x, W1, W2))` with the input gradients
    of the groups accumulated inside the matrix products and the weight gradients computed in one launch."""
    return projection_sets([(x, list(groups))], bf16=None if bf16 is None else [bf16])[0]


def bf16_copies(groups):
    """bf16 copies of groups of [O_k, I] weights, each group as ONE contiguous [sum O_k, I] tensor, all filled by a
    single multi-tensor copy (the reference casts every weight on its own and concatenates, time_mixer.py:120-131).
    No autograd: the copies are for `projection(..., bf16=)`, which returns gradients for the weights themselves."""
    flat_params = [w for g in groups for w in g]
    if all(w.dtype == torch.bfloat16 for w in flat_params) and all(len(g) == 1 for g in groups):
        return [g[0].detach() for g in groups]
    total = sum(w.numel() for w in flat_params)
    flat = torch.empty(total, dtype=torch.bfloat16, device=flat_params[0].device)
    views, outs, o = [], [], 0
    for g in groups:
        start = o
        for w in g:
            views.append(flat[o:o + w.numel()].view(w.shape))
            o += w.numel()
        outs.append(flat[start:o].view(-1, g[0].shape[-1]))
    srcs = [w.detach() for w in flat_params]
    if flat.is_cuda and all(w.is_contiguous() and w.dtype in (torch.float32, torch.bfloat16) for w in srcs):
        cast_to_bf16(srcs, flat)
    else:
        torch._foreach_copy_(views, srcs)
    return outs


def cast_to_bf16(srcs, flat, offsets=None):
    """Writes bf16 copies of the contiguous float32 / bf16 tensors `srcs` into the bf16 tensor `flat`, at the
    element `offsets` given or else back to back; one kernel launch for up to 32 tensors."""
    if not torch.compiler.is_compiling():
        assert flat.dtype == torch.bfloat16 and flat.is_contiguous()
        assert all(w.is_contiguous() and w.device == flat.device for w in srcs)
        if offsets is None:
            assert flat.numel() == sum(w.numel() for w in srcs)
        else:
            assert len(offsets) == len(srcs) and all(0 <= o and o + w.numel() <= flat.numel() for o, w in zip(offsets, srcs))
    _launch('cast_to_bf16', _cast_to_bf16_impl, list(srcs), flat, None if offsets is None else list(offsets))


def _copy_columns(M, pieces, like):
    """pieces: (src tensor or None, src_ld, src_col0, dst tensor, dst_ld, dst_col0, width, op, aux tensor or None)"""
    _launch(
        'copy_columns', _copy_columns_impl, M, [p[0] for p in pieces], [p[1] for p in pieces], [p[2] for p in pieces], [p[3] for p in pieces],
        [p[4] for p in pieces], [p[5] for p in pieces], [p[6] for p in pieces], [p[7] for p in pieces],
        [p[8] for p in pieces])


class SplitColumns(torch.autograd.Function):
    """Contiguous column slices of several [..., W_s] bf16 tensors in one launch, some of them through tanh; the
    backward pass writes each source's gradient (tanh derivative included, missing pieces as zeros) in one launch."""

    @staticmethod
    def forward(ctx, spec, *srcs):
        # spec: per source a tuple of (width, through_tanh)
        outs, pieces, M = [], [], None
        for src, parts in zip(srcs, spec):
            s2 = _rows(src)
            M = s2.shape[0]
            col = 0
            for width, th in parts:
                out = torch.empty(*src.shape[:-1], width, device=src.device, dtype=torch.bfloat16)
                pieces.append((s2, s2.stride(0), col, out, width, 0, width, 1 if th else 0, None))
                outs.append(out)
                col += width
            assert col == src.shape[-1], 'the pieces must cover the source'
        _copy_columns(M, pieces, srcs[0])
        ctx.spec, ctx.shapes, ctx.device = spec, [tuple(s.shape) for s in srcs], srcs[0].device
        ctx.save_for_backward(*[o for o, (_, th) in zip(outs, [p for parts in spec for p in parts]) if th])
        ctx.set_materialize_grads(False)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *gouts):
        saved = list(ctx.saved_tensors)
        grads, pieces, i, M = [], [], 0, None
        for shape, parts in zip(ctx.shapes, ctx.spec):
            W = shape[-1]
            g = torch.empty(shape, device=ctx.device, dtype=torch.bfloat16) \
                if any(go is not None for go in gouts[i:i + len(parts)]) else None
            col = 0
            for width, th in parts:
                go = gouts[i]
                y = saved.pop(0) if th else None
                if g is not None:
                    go2 = None if go is None else _rows(go)
                    M = g.numel() // W
                    pieces.append((go2, width if go2 is None else go2.stride(0), 0, g, W, col, width,
                                   2 if (th and go2 is not None) else 0, y if (th and go2 is not None) else None))
                i += 1
                col += width
            grads.append(g)
        if pieces:
            _copy_columns(M, pieces, pieces[0][3])
        return (None,) + tuple(grads)


def split_columns(srcs, spec):
    """`srcs`: bf16 tensors [..., W_s]; `spec`: per source a list of (width, through_tanh) covering its columns.
    Returns the slices, contiguous, in order (`tanh(slice)` where asked)."""
    return SplitColumns.apply(tuple(tuple(p) for p in spec), *srcs)
