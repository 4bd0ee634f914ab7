"""TimeMixer with a carried state (inference): a sequence run in pieces - `forward(..., return_state=True)`,
`forward(..., state=...)`, then `step` token by token - must reproduce the block run over the whole sequence.
The reference's block has no carried state (time_mixer.py:96-167 starts every call from zero); the whole-sequence
result it is compared with is the one tests/test_gpu_time_mixer.py holds against the fp64 oracle.  The pieces round
at different places than the fused kernels (the single-token path evaluates the small expressions in fp32), so the
comparison is at the block's 1e-2 gate, not bit for bit (both sides are bf16 results with their own rounding; the
token-by-token part, which differs most, is held to 1.2 x its worst measured difference, 1.05e-2)."""
from collections import namedtuple

import pytest
import torch

from oracle import seq_ref

pytestmark = pytest.mark.gpu
DEV = 'cuda'
Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])


def _model(C, H, seed, **switches):
    from wind_rwkv.rwkv7 import TimeMixer
    gen = torch.Generator().manual_seed(seed)
    model = TimeMixer(Config(4, H, C), 1, **switches)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    return model.to(DEV), gen


# steps: on the sequence kernels (default switches, head size 64); PyTorch expressions around the single-token
# kernel (head size 64, and head size 32 with that head size's single-token kernel); more rows than one 16-row
# tile; head size 128 with the bf16 matrix-core kernels of that head size behind the sequence calls
@pytest.mark.parametrize('C,H,B,switches', [(256, 4, 2, {}), (256, 4, 2, dict(use_triton_ddlerp=False)), (128, 4, 2, {}),
                                            (256, 4, 19, {}), (512, 4, 2, {})])
def test_pieces_and_steps_reproduce_the_whole_sequence(C, H, B, switches):
    model, gen = _model(C, H, seed=11, **switches)
    T = 64
    x = torch.randn(B, T, C, generator=gen).bfloat16().to(DEV)
    with torch.no_grad():
        whole = model(x)
        y1, state = model(x[:, :32], return_state=True)
        y2, state = model(x[:, 32:48], state=state, return_state=True)
        ys = []
        for t in range(48, T):
            y, state = model.step(x[:, t], state)
            ys.append(y)
    torch.cuda.synchronize()
    pieces = torch.cat([y1, y2, torch.stack(ys, dim=1)], dim=1)
    assert pieces.shape == whole.shape and pieces.dtype == torch.bfloat16
    for lo, hi in ((0, 32), (32, 48), (48, T)):
        err = seq_ref.rel_err(pieces[:, lo:hi].float().cpu(), whole[:, lo:hi].float().cpu())
        assert err <= (1.27e-2 if lo == 48 else 1e-2), (lo, hi, err)
    # the first piece starts from zero like the whole run: the same kernels on fewer rows (the BLAS library may sum
    # a product of another row count in another order, so not bit for bit)
    assert seq_ref.rel_err(pieces[:, :32].float().cpu(), whole[:, :32].float().cpu()) <= 2e-3
    # the state handed on: last token and the WKV7 state
    assert torch.equal(state[0], x[:, -1]) and tuple(state[1].shape) == (B, H, C // H, C // H)


def test_the_carried_token_matters_and_state_needs_no_grad():
    model, gen = _model(256, 4, seed=12)
    x = torch.randn(2, 32, 256, generator=gen).bfloat16().to(DEV)
    with torch.no_grad():
        _, state = model(x[:, :16], return_state=True)
        y = model(x[:, 16:], state=state)
        y_zero_token = model(x[:, 16:], state=(torch.zeros_like(state[0]), state[1]))
    assert not torch.equal(y[:, 0], y_zero_token[:, 0])
    with pytest.raises(AssertionError):
        model(x[:, 16:], state=state)        # parameters require gradients and grad mode is on


def test_stateful_calls_compile():
    """`torch.compile(fullgraph=True)` of a piece with `return_state=True` and of `step`: same results as eager."""
    model, gen = _model(256, 4, seed=13)
    x = torch.randn(2, 32, 256, generator=gen).bfloat16().to(DEV)
    xt = torch.randn(2, 256, generator=gen).bfloat16().to(DEV)
    with torch.no_grad():
        want_y, want_state = model(x, return_state=True)
        y, state = torch.compile(lambda t: model(t, return_state=True), fullgraph=True)(x)
        assert torch.equal(y, want_y) and torch.equal(state[0], want_state[0]) and torch.equal(state[1], want_state[1])
        a = (want_state[0].clone(), want_state[1].clone())
        b = (want_state[0].clone(), want_state[1].clone())
        want_t, _ = model.step(xt, a)
        got_t, _ = torch.compile(model.step, fullgraph=True)(xt, b)
    torch.cuda.synchronize()
    # eager `step` is the five-launch single-token path, the traced one goes through the registered sequence operators:
    # the same roundings between stages, other summation orders inside them
    assert seq_ref.rel_err(got_t.float().cpu(), want_t.float().cpu()) <= 5e-3
    assert seq_ref.rel_err(b[1].float().cpu(), a[1].float().cpu()) <= 5e-3


@pytest.mark.parametrize('C,H,B', [(768, 12, 1), (768, 12, 5), (256, 4, 16), (256, 4, 35), (192, 3, 2)])
def test_single_token_path_against_the_sequence_kernels(C, H, B):
    """`step` in five launches (wind_rwkv7_mixer_decode) against the same step on the sequence kernels (rows padded
    to a tile), two tokens in a row: output, carried token and WKV7 state (fp32 and bf16)."""
    model, gen = _model(C, H, seed=15)
    x = torch.randn(B, 16, C, generator=gen).bfloat16().to(DEV)
    toks = torch.randn(2, B, C, generator=gen).bfloat16().to(DEV)
    for sdt in (torch.float32, torch.bfloat16):
        with torch.no_grad():
            _, st = model(x, return_state=True)
            sa = (st[0].clone(), st[1].to(sdt).clone())
            sb = (st[0].clone(), st[1].to(sdt).clone())
            for t in range(2):
                want, sa = model._step_on_kernels(toks[t], sa[0], sa[1])
                got, sb = model.step(toks[t], sb)
                torch.cuda.synchronize()
                assert got.shape == want.shape and got.dtype == torch.bfloat16
                err = seq_ref.rel_err(got.float().cpu(), want.float().cpu())
                assert err <= 5e-3, (sdt, t, err)
                assert torch.equal(sb[0], toks[t])
            assert seq_ref.rel_err(sb[1].float().cpu(), sa[1].float().cpu()) <= (2e-3 if sdt == torch.float32 else 8e-3)


@pytest.mark.parametrize('T', [5, 16, 37])
def test_any_prompt_length_with_a_carried_state(T):
    """Lengths that are no multiple of 16: prefix on the sequence kernels, the rest token by token; against the
    whole 48-token run of which the prompt is a prefix (the block is causal)."""
    model, gen = _model(256, 4, seed=14)
    x = torch.randn(2, 48, 256, generator=gen).bfloat16().to(DEV)
    with torch.no_grad():
        whole = model(x)
        y, state = model(x[:, :T], return_state=True)
        rest, state = model(x[:, T:], state=state, return_state=True)      # 48 - T tokens: again any length
    torch.cuda.synchronize()
    got = torch.cat([y, rest], dim=1)
    assert got.shape == whole.shape and state[1].dtype == torch.float32
    assert seq_ref.rel_err(got.float().cpu(), whole.float().cpu()) <= 1e-2
    assert torch.equal(state[0], x[:, -1])
