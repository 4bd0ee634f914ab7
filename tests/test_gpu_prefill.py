"""The forward that keeps nothing for a backward pass (`wind_rwkv7_attn_prefill`, `wind_rwkv7_attn_ln_prefill`):
what `attn` / `attn_ln` / `TimeMixer` run when autograd will not ask for gradients.  It shares every kernel with the
training forward and differs only in the stores it leaves out, so y and sT must be bit-identical to the training
forward's; parity with the fp64 oracle (1e-2, as tests/utils.py:18 of the reference) is checked on top."""
import pytest
import torch

from oracle import inputs, seq_ref

pytestmark = pytest.mark.gpu
DEV = 'cuda'
SEQ = ('r', 'w', 'k', 'v', 'a', 'b')


def _attn_inputs(B, T, H, seed):
    d = inputs.wkv7_inputs(B, T, H, 64, seed, dtype=torch.bfloat16, s0_scale=0.5)
    return d, [d[n].reshape(B, T, H * 64).to(DEV) for n in ('q', 'w', 'k', 'v', 'a', 'b')]


# the last: a long sequence on few heads, which is scanned in segments
@pytest.mark.parametrize('B,T,H', [(1, 16, 1), (2, 80, 3), (8, 1024, 12), (1, 8192, 2)])
def test_attn_without_grad_matches_training_forward_bit_for_bit(B, T, H):
    from wind_rwkv.rwkv7 import attn
    d, x = _attn_inputs(B, T, H, seed=900 + T)
    s0 = d['s0'].float().to(DEV)
    y_train, sT_train = attn(*[t.clone().requires_grad_() for t in x], 64, s0=s0, return_state=True)
    assert y_train.grad_fn is not None
    with torch.no_grad():
        y, sT = attn(*x, 64, s0=s0, return_state=True)
    y2, sT2 = attn(*x, 64, s0=s0, return_state=True)     # grad mode on, but no input asks for a gradient
    torch.cuda.synchronize()
    assert y.grad_fn is None and y2.grad_fn is None
    for got, got_s in ((y, sT), (y2, sT2)):
        assert torch.equal(got, y_train.detach()) and torch.equal(got_s, sT_train.detach())


def test_attn_prefill_parity_with_oracle():
    from wind_rwkv.rwkv7 import attn
    B, T, H = 2, 256, 3
    d, x = _attn_inputs(B, T, H, seed=17)
    with torch.no_grad():
        y, sT = attn(*x, 64, s0=d['s0'].float().to(DEV), return_state=True)
    yo, sTo = seq_ref.wkv7_seq(*[d[n].double() for n in ('q', 'w', 'k', 'v', 'a', 'b')], d['s0'].double())
    assert seq_ref.rel_err(y.float().cpu().view(B, T, H, 64), yo) <= 1e-2
    assert seq_ref.rel_err(sT.float().cpu(), sTo) <= 1e-2


@pytest.mark.parametrize('B,T,H', [(2, 80, 3), (8, 1024, 12), (1, 8192, 2)])
def test_attn_ln_without_grad_matches_training_forward_bit_for_bit(B, T, H):
    from wind_rwkv.rwkv7 import attn_ln
    d, x = _attn_inputs(B, T, H, seed=950 + T)
    g = torch.randn(B, T, H * 64, generator=torch.Generator().manual_seed(5)).bfloat16().to(DEV)
    params = torch.randn(3, H * 64, generator=torch.Generator().manual_seed(6)).to(DEV)
    y_train, sT_train = attn_ln(*x, g, params.clone().requires_grad_(), 64, return_state=True)
    assert y_train.grad_fn is not None
    with torch.no_grad():
        y, sT = attn_ln(*x, g, params, 64, return_state=True)
    torch.cuda.synchronize()
    assert y.grad_fn is None
    assert torch.equal(y, y_train.detach()) and torch.equal(sT, sT_train.detach())


@pytest.mark.parametrize('C,dtype', [(64, torch.float32), (32, torch.bfloat16), (128, torch.float32), (96, torch.bfloat16)])
def test_fp32_kernels_without_grad_match_their_training_forward_bit_for_bit(C, dtype):
    """float32 sequences and head sizes other than 64 run the fp32 kernels, whose no-autograd forward saves no states."""
    from wind_rwkv.rwkv7 import attn, attn_ln
    B, T, H = 2, 64, 3
    d = inputs.wkv7_inputs(B, T, H, C, 31 + C, dtype=dtype, s0_scale=0.5)
    x = [d[n].reshape(B, T, H * C).to(DEV) for n in ('q', 'w', 'k', 'v', 'a', 'b')]
    s0 = d['s0'].to(DEV)
    y_train, sT_train = attn(*[t.clone().requires_grad_() for t in x], C, s0=s0, return_state=True)
    assert y_train.grad_fn is not None
    with torch.no_grad():
        y, sT = attn(*x, C, s0=s0, return_state=True)
        g = torch.randn(B, T, H * C, generator=torch.Generator().manual_seed(5)).to(dtype).to(DEV)
        params = torch.randn(3, H * C, generator=torch.Generator().manual_seed(6)).to(DEV)
        z = attn_ln(*x, g, params, C, s0=s0)
    z_train = attn_ln(*[t.clone().requires_grad_() for t in x], g, params, C, s0=s0)
    torch.cuda.synchronize()
    assert y.dtype == dtype and torch.equal(y, y_train.detach()) and torch.equal(sT, sT_train.detach())
    assert torch.equal(z, z_train.detach())


def test_prefill_through_the_c_abi_with_a_reused_scratch_buffer():
    """Two calls share one scratch buffer (its contents are undefined between calls) and one workspace."""
    from wind_rwkv import _native
    lib = _native.lib()
    B, T, H, C = 2, 128, 3, 64
    scratch = torch.empty(lib.wind_rwkv7_attn_saved_bytes(B, T, H, C), dtype=torch.uint8, device=DEV)
    ws = torch.empty(max(lib.wind_rwkv7_attn_fwd_workspace_bytes(B, T, H, C), 256), dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    for seed in (1, 2):
        d = inputs.wkv7_inputs(B, T, H, C, seed, dtype=torch.bfloat16)
        x = [d[n].to(DEV).contiguous() for n in ('w', 'q', 'k', 'v', 'a', 'b')]
        s0 = d['s0'].float().to(DEV)
        out = {}
        for entry in ('wind_rwkv7_attn_forward', 'wind_rwkv7_attn_prefill'):
            y, sT = torch.empty_like(x[3]), torch.empty_like(s0)
            s = scratch if entry.endswith('prefill') else torch.empty_like(scratch)
            _native.check(getattr(lib, entry)(B, T, H, C, _native.BF16, _native.F32, *[t.data_ptr() for t in x],
                                              s0.data_ptr(), y.data_ptr(), s.data_ptr(), sT.data_ptr(),
                                              ws.data_ptr(), ws.numel(), stream))
            torch.cuda.synchronize()
            out[entry] = (y, sT)
        (y0, s0T), (y1, s1T) = out.values()
        assert torch.equal(y0, y1) and torch.equal(s0T, s1T)


def test_time_mixer_without_grad_matches_its_training_forward():
    from collections import namedtuple
    from wind_rwkv.rwkv7 import TimeMixer
    gen = torch.Generator().manual_seed(3)
    model = TimeMixer(namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])(4, 4, 256), 1)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    model = model.to(DEV)
    x = torch.randn(2, 64, 256, generator=gen).bfloat16().to(DEV)
    y_train = model(x)
    assert y_train.grad_fn is not None
    with torch.no_grad():
        y = model(x)
    torch.cuda.synchronize()
    assert y.grad_fn is None and torch.equal(y, y_train.detach())


def test_compiled_attn_ln_without_grad():
    from wind_rwkv.rwkv7 import attn_ln
    B, T, H = 2, 64, 2
    d, x = _attn_inputs(B, T, H, seed=23)
    g = torch.randn(B, T, H * 64, generator=torch.Generator().manual_seed(7)).bfloat16().to(DEV)
    params = torch.randn(3, H * 64, generator=torch.Generator().manual_seed(8)).to(DEV)
    fn = torch.compile(lambda *t: attn_ln(*t, 64), fullgraph=True)
    with torch.no_grad():
        want = attn_ln(*x, g, params, 64)
        got = fn(*x, g, params)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_compiled_time_mixer_without_grad():
    from collections import namedtuple
    from wind_rwkv.rwkv7 import TimeMixer
    gen = torch.Generator().manual_seed(9)
    model = TimeMixer(namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])(4, 4, 256), 1)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    model = model.to(DEV)
    x = torch.randn(2, 64, 256, generator=gen).bfloat16().to(DEV)
    compiled = torch.compile(model, fullgraph=True)
    graphed = torch.compile(model, fullgraph=True, mode='reduce-overhead')    # the reference's idiom
    with torch.no_grad():
        want = model(x)
        got = compiled(x)
        replays = [graphed(x).clone() for _ in range(4)]
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert all(torch.equal(r, want) for r in replays)


@pytest.mark.parametrize('T,with_state', [(7, False), (40, True), (100, False)])
def test_any_length_without_grad(T, with_state):
    """T no multiple of 16, nothing differentiated: whole chunks on the sequence kernels, the rest through the
    single-token kernel; against the fp64 oracle over all T tokens."""
    from wind_rwkv.rwkv7 import attn, attn_ln
    B, H = 2, 3
    d = inputs.attn_ln_inputs(B, T, H, 64, 60 + T, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(T)
    s0 = torch.randn(B, H, 64, 64, generator=gen) * 0.5 if with_state else None
    x = [d[n].reshape(B, T, H * 64).to(DEV) for n in ('q', 'w', 'k', 'v', 'a', 'b')]
    g, params = d['g'].reshape(B, T, H * 64).to(DEV), d['params'].to(DEV)
    s0_dev = None if s0 is None else s0.to(DEV)
    with torch.no_grad():
        y, sT = attn(*x, 64, s0=s0_dev, return_state=True)
        z, zT = attn_ln(*x, g, params, 64, s0=s0_dev, return_state=True)
    torch.cuda.synchronize()
    dd = {n: d[n].double() for n in ('q', 'w', 'k', 'v', 'a', 'b', 'g')}
    yo, sTo = seq_ref.wkv7_seq(dd['q'], dd['w'], dd['k'], dd['v'], dd['a'], dd['b'], None if s0 is None else s0.double())
    zo = seq_ref.attn_ln_epilogue(yo, dd['q'], dd['k'], dd['v'], dd['g'], d['params'].double())
    assert y.shape == (B, T, H * 64) and sT.dtype == torch.float32
    if with_state:
        assert torch.equal(s0_dev.cpu(), s0)                     # the caller's state is not written
    assert seq_ref.rel_err(y.float().cpu().view(B, T, H, 64), yo) <= 1e-2
    assert seq_ref.rel_err(sT.cpu(), sTo) <= 1e-2 and seq_ref.rel_err(zT.cpu(), sTo) <= 1e-2
    assert seq_ref.rel_err(z.float().cpu().view(B, T, H, 64), zo.view(B, T, H, 64)) <= 1e-2
    with pytest.raises(Exception):
        attn(*[t.clone().requires_grad_() for t in x], 64)       # training keeps the reference's rule: T % 16 == 0
