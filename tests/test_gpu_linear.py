"""Weight gradient of the time-mixer's projections (linear_wgrad / projection) against an fp64 matmul.

The reference computes these products with torch matmuls (time_mixer.py:120-131, :167), so the spec is the
matrix product itself: dW = dy^T x.  Inputs are bf16; the kernel accumulates in fp32, so the fp32 output has
to agree with the fp64 product of the same bf16 inputs to 1e-5 (normalised L2), the bf16 output to 1e-2 (the
gate of every bf16 result here; a single rounding gives 2e-3).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-300)).item()


# (tokens, O, I): every tile shape, both orientations, ragged token counts, sizes that are not tile multiples
CASES = [(31, 16, 16), (32, 16, 48), (1000, 48, 80), (4096, 768, 768), (4100, 768, 128), (2048, 128, 768),
         (2048, 32, 768), (2048, 96, 768), (2048, 768, 64), (3000, 208, 400), (1024, 1024, 1024), (64, 768, 768)]


@pytest.mark.parametrize('tokens,O,I', CASES)
def test_linear_wgrad_matches_fp64_product(tokens, O, I):
    from wind_rwkv.rwkv7 import linear_wgrad
    g = torch.Generator().manual_seed(tokens + O + I)
    dy = torch.randn(tokens, O, generator=g).bfloat16()
    x = torch.randn(tokens, I, generator=g).bfloat16()
    ref = dy.double().T @ x.double()
    got32 = linear_wgrad(dy.to(DEV), x.to(DEV), torch.float32).cpu()
    got16 = linear_wgrad(dy.to(DEV), x.to(DEV), torch.bfloat16).cpu()
    assert got32.shape == (O, I) and got32.dtype == torch.float32 and got16.dtype == torch.bfloat16
    assert _rel(got32, ref) <= 1e-5
    assert _rel(got16, ref) <= 1e-2
    # one-hot rows pin the orientation and the channel order exactly: dW[o][i] = x[t0][i] for dy = e_o at token t0
    dy1 = torch.zeros(tokens, O)
    dy1[tokens // 2, O - 3] = 1.0
    got = linear_wgrad(dy1.bfloat16().to(DEV), x.to(DEV), torch.float32).cpu()
    want = torch.zeros(O, I)
    want[O - 3] = x[tokens // 2].float()
    assert torch.equal(got, want)


def test_linear_wgrad_strided_rows_and_batch_dims():
    """Row strides larger than the width (column slices of a wider tensor) and leading batch dimensions."""
    from wind_rwkv.rwkv7 import linear_wgrad
    g = torch.Generator().manual_seed(5)
    big_dy = torch.randn(4, 96, 256, generator=g).bfloat16().to(DEV)
    big_x = torch.randn(4, 96, 512, generator=g).bfloat16().to(DEV)
    dy, x = big_dy[..., 64:192], big_x[..., 128:384]          # strides 256 / 512, offsets multiples of 8
    ref = dy.double().reshape(-1, 128).T @ x.double().reshape(-1, 256)
    assert _rel(linear_wgrad(dy, x).cpu(), ref.cpu()) <= 1e-5
    dy_odd = big_dy[..., 3:131]                                # misaligned start: the wrapper copies
    ref = dy_odd.double().reshape(-1, 128).T @ x.double().reshape(-1, 256)
    assert _rel(linear_wgrad(dy_odd, x).cpu(), ref.cpu()) <= 1e-5


def test_linear_wgrad_is_reproducible():
    from wind_rwkv.rwkv7 import linear_wgrad
    g = torch.Generator().manual_seed(9)
    dy = torch.randn(8192, 768, generator=g).bfloat16().to(DEV)
    x = torch.randn(8192, 768, generator=g).bfloat16().to(DEV)
    a = linear_wgrad(dy, x)
    b = linear_wgrad(dy, x)
    assert torch.equal(a, b)          # fixed summation order, no atomics


@pytest.mark.parametrize('wdtype', [torch.float32, torch.bfloat16])
def test_projection_forward_backward(wdtype):
    """projection(x, W1, W2) == x @ cat(W1, W2).T with gradients for x and both weights in their own dtype."""
    from wind_rwkv.rwkv7 import projection
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 160, 256, generator=g).bfloat16()
    W1 = (torch.randn(64, 256, generator=g) * 0.05).to(wdtype)
    W2 = (torch.randn(32, 256, generator=g) * 0.05).to(wdtype)
    dy = torch.randn(2, 160, 96, generator=g).bfloat16()
    xd, W1d, W2d = (t.to(DEV).requires_grad_() for t in (x, W1, W2))
    y = projection(xd, W1d, W2d)
    y.backward(dy.to(DEV))
    Wb = torch.cat([W1, W2]).bfloat16().double()
    y_ref = x.double() @ Wb.T
    dx_ref = dy.double() @ Wb
    dW_ref = dy.double().reshape(-1, 96).T @ x.double().reshape(-1, 256)
    assert y.dtype == torch.bfloat16 and _rel(y.cpu(), y_ref) <= 1e-2
    assert _rel(xd.grad.cpu(), dx_ref) <= 1e-2
    assert W1d.grad.dtype == wdtype and W2d.grad.dtype == wdtype
    tol = 1e-5 if wdtype == torch.float32 else 1e-2
    assert _rel(W1d.grad.cpu(), dW_ref[:64]) <= tol
    assert _rel(W2d.grad.cpu(), dW_ref[64:]) <= tol


def test_linear_wgrad_rejects_bad_arguments():
    from wind_rwkv import _native
    from wind_rwkv.rwkv7 import linear_wgrad
    x = torch.zeros(64, 24, device=DEV, dtype=torch.bfloat16)       # 24 is not a multiple of 16
    dy = torch.zeros(64, 32, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(_native.WindRwkv7Error):
        linear_wgrad(dy, x)
    with pytest.raises(TypeError):
        linear_wgrad(dy.float(), x)
    with pytest.raises(ValueError):
        linear_wgrad(dy[:32], torch.zeros(64, 32, device=DEV, dtype=torch.bfloat16))


@pytest.mark.parametrize('stride', [4, 16, 64])
def test_lds_transposed_read_lane_mapping(stride):
    """The hardware fact linear_wgrad is built on: with LDS holding its own element index and lane l of a
    16-lane group pointing at element stride*l, ds_read_b64_tr_b16 hands lane i of the group, in register r,
    element i%4 of the row addressed by lane 4r + i/4."""
    import ctypes
    import os
    from wind_rwkv import _native
    st = ctypes.CDLL(os.path.join(os.path.dirname(_native.LIB_PATH), 'libwind_rwkv7_selftest.so'))
    st.wind_rwkv7_selftest_lds_transpose_read.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    out = torch.zeros(256, dtype=torch.int16, device=DEV)
    assert st.wind_rwkv7_selftest_lds_transpose_read(stride, out.data_ptr(), None) == 0
    torch.cuda.synchronize()
    got = out.cpu().view(64, 4)
    for lane in range(64):
        grp, i = lane // 16, lane % 16
        for r in range(4):
            src_lane = 16 * grp + 4 * r + i // 4
            assert got[lane, r].item() == stride * src_lane + i % 4, (lane, r)


def test_projection_groups_match_separate_projections():
    """projections(x, [W0], [W1, W2]) == (projection(x, W0), projection(x, W1, W2)), gradients included."""
    from wind_rwkv.rwkv7 import projection, projections
    g = torch.Generator().manual_seed(17)
    x = torch.randn(2, 96, 128, generator=g).bfloat16().to(DEV)
    Ws = [(torch.randn(n, 128, generator=g) * 0.05).to(DEV) for n in (128, 16, 32)]
    dys = [torch.randn(2, 96, n, generator=g).bfloat16().to(DEV) for n in (128, 48)]

    def run(fused):
        xs = x.clone().requires_grad_()
        ws = [w.clone().requires_grad_() for w in Ws]
        ys = projections(xs, [ws[0]], [ws[1], ws[2]]) if fused else (projection(xs, ws[0]), projection(xs, ws[1], ws[2]))
        torch.autograd.backward(list(ys), dys)
        return list(ys) + [xs.grad] + [w.grad for w in ws]

    a, b = run(True), run(False)
    for u, v in zip(a[:2], b[:2]):
        assert torch.equal(u, v)
    assert _rel(a[2], b[2]) <= 1e-2                      # dx: one rounding less in the accumulating product
    for u, v in zip(a[3:], b[3:]):
        assert _rel(u, v) <= 1e-5                        # weight gradients: one grouped launch, another split of the tokens
    # a group whose output is unused contributes nothing
    xs = x.clone().requires_grad_()
    y0, _ = projections(xs, [Ws[0].clone().requires_grad_()], [Ws[1], Ws[2]])
    y0.backward(dys[0])
    assert _rel(xs.grad, dys[0].double() @ Ws[0].bfloat16().double()) <= 1e-2


def test_projection_sets_match_separate_projections():
    """Several inputs with their groups as one autograd node == one `projection` per group: outputs bit for bit,
    input gradients to bf16 rounding, weight gradients (fp32 and bf16 weights in one set: two grouped launches) to
    fp32 / bf16 rounding; an unused output and an input that needs no gradient are left out."""
    from wind_rwkv.rwkv7 import projection, projection_sets
    g = torch.Generator().manual_seed(23)
    T = 200
    xa = torch.randn(T, 256, generator=g).bfloat16().to(DEV)
    xb = torch.randn(T, 64, generator=g).bfloat16().to(DEV)
    xc = torch.randn(T, 256, generator=g).bfloat16().to(DEV)
    Ws = [(torch.randn(n, i, generator=g) * 0.05).to(DEV) for n, i in ((256, 256), (32, 256), (16, 256), (256, 64), (160, 256))]
    Ws[3] = Ws[3].bfloat16()
    dys = [torch.randn(T, n, generator=g).bfloat16().to(DEV) for n in (256, 48, 256, 160)]

    def run(fused, skip=None):
        xs = [xa.clone().requires_grad_(), xb.clone().requires_grad_(), xc.clone()]
        ws = [w.clone().requires_grad_() for w in Ws]
        if fused:
            (y0, y1), (y2,), (y3,) = projection_sets([(xs[0], [[ws[0]], [ws[1], ws[2]]]), (xs[1], [[ws[3]]]), (xs[2], [[ws[4]]])])
        else:
            y0, y1 = projection(xs[0], ws[0]), projection(xs[0], ws[1], ws[2])
            y2, y3 = projection(xs[1], ws[3]), projection(xs[2], ws[4])
        ys = [y0, y1, y2, y3]
        keep = [k for k in range(4) if k != skip]
        torch.autograd.backward([ys[k] for k in keep], [dys[k] for k in keep])
        return ys, [xs[0].grad, xs[1].grad], [w.grad for w in ws]

    for skip in (None, 1):
        (ya, dxa, dwa), (yb, dxb, dwb) = run(True, skip), run(False, skip)
        for u, v in zip(ya, yb):
            assert torch.equal(u, v)
        for u, v in zip(dxa, dxb):
            assert _rel(u, v) <= 1e-2
        for k, (u, v) in enumerate(zip(dwa, dwb)):
            if skip == 1 and k in (1, 2):
                assert u is None and v is None
                continue
            assert u.dtype == v.dtype == Ws[k].dtype and u.shape == Ws[k].shape
            assert _rel(u, v) <= (1e-2 if Ws[k].dtype == torch.bfloat16 else 1e-5)
    # against the fp64 products
    _, dx, dw = run(True)
    assert _rel(dw[4], dys[3].double().T @ xc.double()) <= 1e-5
    assert _rel(dx[0], dys[0].double() @ Ws[0].bfloat16().double() + dys[1].double() @ torch.cat(Ws[1:3]).bfloat16().double()) <= 1e-2
    # inference: no autograd node, same numbers
    with torch.no_grad():
        (z0, z1), (z2,), (z3,) = projection_sets([(xa, [[Ws[0]], [Ws[1], Ws[2]]]), (xb, [[Ws[3]]]), (xc, [[Ws[4]]])])
    for u, v in zip((z0, z1, z2, z3), run(False)[0]):
        assert torch.equal(u, v)


def test_cast_to_bf16_matches_torch_bit_for_bit():
    """The one-launch weight cast: same rounding as torch's .to(bfloat16), for aligned tensors (16-byte path),
    odd sizes (which leave the following tensors unaligned), bf16 sources, an empty tensor and more tensors
    than one launch takes."""
    from wind_rwkv.rwkv7.linear import cast_to_bf16, bf16_copies
    gen = torch.Generator().manual_seed(5)
    shapes = [(768, 768), (64, 768), (3,), (0,), (1000,), (2049,), (16, 40)] + [(17,)] * 40
    srcs = [torch.randn(*sh, generator=gen).to(DEV) * 10 ** float(torch.randint(-3, 4, (1,), generator=gen)) for sh in shapes]
    srcs[1] = srcs[1].bfloat16()
    srcs[4][5] = float('inf')
    srcs[4][6] = float('nan')
    flat = torch.full((sum(w.numel() for w in srcs) + 8,), 7.0, dtype=torch.bfloat16, device=DEV)
    cast_to_bf16(srcs, flat[:-8])
    want = torch.cat([w.reshape(-1).bfloat16() for w in srcs])
    got = flat[:-8]
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert (flat[-8:] == 7.0).all()                      # nothing past the end
    # explicit offsets (padded layout); the gaps keep their contents
    flat2 = torch.full((4096,), 7.0, dtype=torch.bfloat16, device=DEV)
    cast_to_bf16([srcs[2], srcs[4]], flat2, offsets=[128, 1024])
    assert torch.equal(flat2[128:131], srcs[2].bfloat16()) and torch.equal(flat2[1024:2024].view(torch.int16), srcs[4].bfloat16().view(torch.int16))
    assert (flat2[:128] == 7.0).all() and (flat2[131:1024] == 7.0).all() and (flat2[2024:] == 7.0).all()
    # through bf16_copies: groups come out as contiguous matrices
    a, b, c = (torch.randn(n, 768, generator=gen).to(DEV) for n in (768, 64, 32))
    ga, gbc = bf16_copies([[a], [b, c]])
    assert torch.equal(ga, a.bfloat16()) and torch.equal(gbc, torch.cat([b, c]).bfloat16())


def test_split_columns_matches_torch():
    """Slices of concatenated products, tanh on some of them, and the gradients of the wide tensors: against
    split / tanh / autograd in PyTorch (the forward bit for bit: same fp32 arithmetic, one rounding)."""
    from wind_rwkv.rwkv7.linear import split_columns
    gen = torch.Generator().manual_seed(11)
    a = torch.randn(2, 48, 32, generator=gen).bfloat16().to(DEV)
    b = torch.randn(2, 48, 96, generator=gen).bfloat16().to(DEV)
    c = torch.randn(2, 48, 128, generator=gen).bfloat16().to(DEV)
    spec = [[(16, 0), (16, 0)], [(64, 1), (16, 0), (16, 0)], [(128, 1)]]
    mine_in = [t.clone().requires_grad_() for t in (a, b, c)]
    ref_in = [t.clone().requires_grad_() for t in (a, b, c)]
    outs = split_columns(mine_in, spec)
    a0, a1 = ref_in[0].split([16, 16], dim=2)
    b0, b1, b2 = ref_in[1].split([64, 16, 16], dim=2)
    refs = [a0, a1, torch.tanh(b0), b1, b2, torch.tanh(ref_in[2])]
    assert all(o.is_contiguous() for o in outs)
    for o, r in zip(outs, refs):
        assert torch.equal(o, r)
    # gradients: the second piece of `a` gets none (zeros in the wide gradient)
    gs = [torch.randn(o.shape, generator=gen).bfloat16().to(DEV) for o in outs]
    use = [0, 2, 3, 4, 5]
    torch.autograd.backward([outs[i] for i in use], [gs[i] for i in use])
    torch.autograd.backward([refs[i] for i in use], [gs[i] for i in use])
    # plain slices are copies.  Through the tanh derivative the kernel computes g (1 - y^2) in fp32 and rounds once;
    # the framework's bf16 tanh-backward rounds after every operation, so it is compared loosely and the fp32
    # formula exactly
    assert torch.equal(mine_in[0].grad, ref_in[0].grad)
    assert torch.equal(mine_in[1].grad[..., 64:], ref_in[1].grad[..., 64:])
    for m, r, g, y in ((mine_in[1].grad[..., :64], ref_in[1].grad[..., :64], gs[2], outs[2]),
                       (mine_in[2].grad, ref_in[2].grad, gs[5], outs[5])):
        exact = (g.float() * (1 - y.detach().float() ** 2)).bfloat16()
        assert torch.equal(m, exact)
        # (its rounding of y^2 to bf16 is an absolute error of 2^-9 in the factor 1 - y^2)
        assert ((m.float() - r.float()).abs() <= 2 ** -7 * g.float().abs() + 1e-30).all()


def test_split_columns_more_pieces_than_one_launch():
    """Twelve slices of one tensor (a launch takes eight pieces): forward copies and the reassembled gradient."""
    from wind_rwkv.rwkv7.linear import split_columns
    gen = torch.Generator().manual_seed(12)
    a = torch.randn(3, 16, 96, generator=gen).bfloat16().to(DEV).requires_grad_()
    outs = split_columns([a], [[(8, 0)] * 12])
    for i, o in enumerate(outs):
        assert o.is_contiguous() and torch.equal(o, a.detach()[..., 8 * i:8 * i + 8])
    gs = [torch.randn(o.shape, generator=gen).bfloat16().to(DEV) for o in outs]
    torch.autograd.backward(list(outs), gs)
    assert torch.equal(a.grad, torch.cat(gs, dim=-1))


@pytest.mark.parametrize('tokens,shapes', [
    (4096, [(768, 768), (768, 768), (768, 768)]),          # the time mixer's r, k, v projections
    (1000, [(896, 768), (160, 1024), (768, 144), (208, 400)]),   # both orientations, ragged sizes and token count
    (64, [(256, 256), (768, 768)]),                        # fewer token steps than compute units per tile
    # the time mixer's two sets: the projections of the four shifted streams, then the second LoRA factors
    (2048, [(768, 768), (128, 768), (768, 768), (64, 768), (768, 768), (160, 768)]),
    (2048, [(768, 128), (768, 64)]),
    (999, [(32, 768), (768, 32), (96, 400), (768, 768), (16, 64), (48, 48), (256, 128), (128, 256), (80, 768)]),  # every tile shape; nine: two batches
])
def test_linear_wgrad_group_matches_fp64_products(tokens, shapes):
    """Several wide problems in one launch: each result against the fp64 product of the same bf16 inputs, and the
    grouped call against the single calls (different split of the token range: equal to fp32 rounding)."""
    from wind_rwkv.rwkv7.linear import linear_wgrad, linear_wgrad_group
    g = torch.Generator().manual_seed(tokens + len(shapes))
    dys = [torch.randn(tokens, O, generator=g).bfloat16().to(DEV) for O, _ in shapes]
    xs = [torch.randn(tokens, I, generator=g).bfloat16().to(DEV) for _, I in shapes]
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        got = linear_wgrad_group(dys, xs, dt)
        assert len(got) == len(shapes)
        for (O, I), dy, x, w in zip(shapes, dys, xs, got):
            assert w.shape == (O, I) and w.dtype == dt
            ref = dy.double().T @ x.double()
            assert _rel(w.cpu(), ref.cpu()) <= tol
            assert _rel(w.cpu(), linear_wgrad(dy, x, dt).cpu()) <= tol
    # one-hot rows pin orientation and channel order of every problem of the group
    dy1 = []
    for O, _ in shapes:
        t = torch.zeros(tokens, O)
        t[tokens // 3, O - 5] = 1.0
        dy1.append(t.bfloat16().to(DEV))
    for (O, I), x, w in zip(shapes, xs, linear_wgrad_group(dy1, xs, torch.float32)):
        want = torch.zeros(O, I)
        want[O - 5] = x[tokens // 3].float().cpu()
        assert torch.equal(w.cpu(), want)


def test_linear_wgrad_group_falls_back_for_different_token_counts():
    from wind_rwkv.rwkv7.linear import linear_wgrad_group
    g = torch.Generator().manual_seed(3)
    dys = [torch.randn(t, 768, generator=g).bfloat16().to(DEV) for t in (256, 512)]
    xs = [torch.randn(t, 768, generator=g).bfloat16().to(DEV) for t in (256, 512)]
    for dy, x, w in zip(dys, xs, linear_wgrad_group(dys, xs)):
        assert _rel(w.cpu(), (dy.double().T @ x.double()).cpu()) <= 1e-5
