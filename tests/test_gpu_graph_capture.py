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


def test_attn_capture():
    from wind_rwkv.rwkv7.wkv_attn import WindRWKV7
    B, T, H, C = 2, 128, 3, 64

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
