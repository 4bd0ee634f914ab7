#!/usr/bin/env python3
"""Benchmark of the WKV7 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward + backward pass of WKV7 (the `attn` autograd Function) over one synthetic batch at
the shape the headline metric is quoted on: B=8, T=1024, H=12, N=64, bf16 sequences, fp32 carried state,
chunk length 16.  Inputs are resident in HBM before the timed region.  Prints one JSON line with the
tokens/s of the whole job, the roofline figures of the dominant kernel (its duration measured live with
HIP events on the launch stream) and of the whole step, and the naive PyTorch CPU recurrence timed on
this machine's host cores on a bounded sample of the same workload.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, 'wind-rwkv7_amd'))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X published
MFMA_PEAK_BF16 = 2.5e15  # flop/s, MI355X published (dense)
# matrix flops of the chunked algorithm per token per head at N=64, K=16: forward 8N^2 + 16KN, backward 18N^2 + 44KN
FLOPS_PER_TOKEN_HEAD = (8 + 18) * 64 * 64 + (16 + 44) * 16 * 64
# algorithmic bytes per token per head (N=64, bf16 => 128 B per tensor pass):
#   whole fwd+bwd: fwd reads w,q,k,v,a,b writes y (7); bwd reads those + dy (7) writes 6 grads -> 20 passes
#   per kernel: the tensor passes that kernel performs on the caller's tensors.  They sum to 25, not 20: the backward
#   pass is two kernels, and the reverse scan reads w, q, a, b, dy which the gradient kernel reads again (those 5
#   passes are implementation traffic from the whole step's point of view, and `roofline_step` counts 20).
ALGO_PASSES = {
    'step': 20,
    'wkv7_fused_kernel[fwd]': 7,    # reads w,q,k,v,a,b writes y (checkpoints and U are implementation traffic)
    'wkv7_fused_kernel[bwd]': 5,    # reads w,q,a,b,dy
    'bwd_grads_kernel': 13,         # reads w,q,k,v,a,b,dy writes dw,dq,dk,dv,da,db
}
# HBM bytes per launch at the headline workload come from the hardware counters: two `rocprofv3 --pmc` runs of this
# script (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what the same counter reads for the 256 MiB
# device copy of `--workload copy`.  Counters cannot be read from inside a timed run, so the figures are kept in a
# tracked file next to the profile summaries, together with a digest of the kernel sources they were measured on;
# `--record-traffic` writes that file from the two counter runs' CSV output.
TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'wkv7_cfg1_hbm_traffic.json')
KERNEL_SOURCES = ('wkv7_fused.hip', 'wkv7_bwd.hip', 'wkv7_fwd.hip', 'wkv7_common.hpp', 'frag.hpp', 'ln_epilogue.hpp')


def kernel_source_digest():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, 'wind-rwkv7_amd', 'csrc', name), 'rb') as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def load_traffic():
    """{kernel: bytes per launch at cfg1}, and whether the kernel sources changed since they were measured."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
    except OSError:
        return {}, True
    ff, wf = t['fetch_factor'], t['write_factor']
    table = {k: int((v['FETCH_SIZE_KiB'] * ff + v['WRITE_SIZE_KiB'] * wf) * 1024) for k, v in t['kernels'].items()}
    return table, t.get('kernel_source_digest') != kernel_source_digest()


def record_traffic(fetch_csv, write_csv, copy_fetch_csv, copy_write_csv):
    """Writes TRAFFIC_FILE from rocprofv3 `--pmc FETCH_SIZE` / `--pmc WRITE_SIZE` counter_collection CSVs of
    `bench.py --workload wkv7` and of `bench.py --workload copy` (the calibration: a 256 MiB device copy)."""
    import csv
    import re

    def per_kernel(path, counter):
        acc = {}
        with open(path) as f:
            for r in csv.DictReader(f):
                if r['Counter_Name'] == counter:
                    acc.setdefault(r['Kernel_Name'], []).append(float(r['Counter_Value']))
        return {k: sum(v[-5:]) / len(v[-5:]) for k, v in acc.items()}

    def short(n):
        if 'wkv7_fused_kernel' in n:
            fwd = 'ILb1' in n or '<true' in n
            return 'wkv7_fused_kernel[fwd]' if fwd else 'wkv7_fused_kernel[bwd]'
        if 'bwd_grads_kernel' in n:
            return 'bwd_grads_kernel'
        return None

    copied_kib = 256 * 1024
    cf = [v for k, v in per_kernel(copy_fetch_csv, 'FETCH_SIZE').items() if 'copyBuffer' in k or 'copy' in k.lower()]
    cw = [v for k, v in per_kernel(copy_write_csv, 'WRITE_SIZE').items() if 'copyBuffer' in k or 'copy' in k.lower()]
    fetch_factor = copied_kib / max(cf)     # the copy READS 256 MiB
    write_factor = copied_kib / max(cw)     # and WRITES 256 MiB
    kernels = {}
    for path, counter, key in ((fetch_csv, 'FETCH_SIZE', 'FETCH_SIZE_KiB'), (write_csv, 'WRITE_SIZE', 'WRITE_SIZE_KiB')):
        for name, val in per_kernel(path, counter).items():
            k = short(name)
            if k:
                kernels.setdefault(k, {})[key] = val
    out = {'workload': 'cfg1: B=8 T=1024 H=12 N=64', 'unit': 'KiB per dispatch as the counter reads',
           'fetch_factor': round(fetch_factor, 3), 'write_factor': round(write_factor, 3),
           'calibration': {'copy_FETCH_SIZE': max(cf), 'copy_WRITE_SIZE': max(cw), 'copied_KiB': copied_kib},
           'kernel_source_digest': kernel_source_digest(), 'kernels': kernels}
    with open(TRAFFIC_FILE, 'w') as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write('\n')
    print(json.dumps(out))


def measured_peaks():
    """What this machine sustains, next to the published peaks: a 256 MiB device-to-device copy (read + write
    bytes per second) and a dense loop of bf16 matrix instructions with operands in registers."""
    import torch
    from wind_rwkv import _native
    dev = torch.device('cuda:0')
    src = torch.empty(128 << 20, dtype=torch.bfloat16, device=dev).normal_()
    dst = torch.empty_like(src)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    for _ in range(3):
        dst.copy_(src)
    ev[0].record()
    for _ in range(10):
        dst.copy_(src)
    ev[1].record()
    torch.cuda.synchronize()
    copy_gbps = 10 * 2 * src.numel() * 2 / (ev[0].elapsed_time(ev[1]) * 1e-3) / 1e9
    st = ctypes.CDLL(os.path.join(os.path.dirname(_native.LIB_PATH), 'libwind_rwkv7_selftest.so'))
    out = torch.zeros(4, device=dev)
    blocks, iters = 256 * 8, 4096
    stream = torch.cuda.current_stream().cuda_stream
    peaks = {'copy_GBps': copy_gbps}
    # two instruction shapes: this chip sustains the 32x32x16 one much better than the 16x16x32 one
    for key, fn, per_iter in (('mfma_bf16_TFLOPs', st.wind_rwkv7_selftest_mfma_loop, 8 * 16 * 16 * 32 * 2),
                              ('mfma_bf16_32x32x16_TFLOPs', st.wind_rwkv7_selftest_mfma_loop32, 4 * 32 * 32 * 16 * 2)):
        fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        fn(blocks, 64, out.data_ptr(), stream)
        ev[0].record()
        fn(blocks, iters, out.data_ptr(), stream)
        ev[1].record()
        torch.cuda.synchronize()
        peaks[key] = blocks * 4 * iters * per_iter / (ev[0].elapsed_time(ev[1]) * 1e-3) / 1e12
    return peaks


class inputs:
    """Seeded synthetic inputs of the measured workloads, drawn on the CPU in fp32 and then cast.  Distributions as
    the reference's data builders: tests/test_attn.py:24-30 (r,k,v ~ N(0,1); w = -softplus(N(0,1)) - 0.5; unit-norm
    kk per head) with a = -kk, b = kk*sigmoid(N(0,1)) (tests/test_time_mixer.py:51); tests/test_ddlerp.py:25-28;
    tests/test_expand_loras.py:37-45."""

    @staticmethod
    def wkv7_inputs(B, T, H, C, seed, dtype):
        import torch
        F = torch.nn.functional
        gen = torch.Generator().manual_seed(seed)
        rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32)
        q, k, v = rn(B, T, H, C), rn(B, T, H, C), rn(B, T, H, C)
        w = -F.softplus(-rn(B, T, H, C)) - 0.5
        kk = F.normalize(rn(B, T, H, C), dim=-1)
        seqs = dict(q=q, w=w, k=k, v=v, a=-kk, b=kk * torch.sigmoid(rn(B, T, H, C)), dy=rn(B, T, H, C))
        return {n: t.to(dtype).contiguous() for n, t in seqs.items()}

    @staticmethod
    def attn_ln_inputs(B, T, H, C, seed, dtype):
        import torch
        d = inputs.wkv7_inputs(B, T, H, C, seed, dtype)
        gen = torch.Generator().manual_seed(seed + 1000)
        rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32)
        d['g'] = rn(B, T, H, C).to(dtype).contiguous()
        d['params'] = torch.stack([1 + 0.1 * rn(H * C), 0.1 * rn(H * C), 0.1 * rn(H * C)]).contiguous()
        return d

    @staticmethod
    def ddlerp_inputs(B, T, C, D, seed, dtype):
        import torch
        gen = torch.Generator().manual_seed(seed)
        rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32) / 2
        return dict(x=rn(B, T, C).to(dtype), alpha=rn(C), L=rn(4 * D, C), R=rn(4, C, D), beta=rn(4, 1, 1, C),
                    dy=[(2 * rn(B, T, C)).to(dtype) for _ in range(4)])

    @staticmethod
    def expand_loras_inputs(B, T, C, D, seed, dtype):
        import torch
        gen = torch.Generator().manual_seed(seed)
        rn = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float32)
        d = {n: rn(B, T, C).to(dtype) for n in ('w_in', 'k_in')}
        d.update({n: rn(B, T, D).to(dtype) for n in ('z_in', 'a_in', 'ma_in', 'mk_in')})
        d.update({n: rn(C, D).to(dtype) for n in ('Wz', 'Wa', 'Wma', 'Wmk')})
        d.update({n: rn(C).to(dtype) for n in ('w_bias', 'a_bias', 'ma_bias', 'mk_bias')})
        d['dy'] = [rn(B, T, C).to(dtype) for _ in range(4)]
        return d


def cpu_baseline(sample_B=4, reps=3):
    """The reference's naive recurrence (time_mixer.py:6-16 semantics) in fp32 PyTorch, forward + autograd
    backward, on a B=sample_B slice of the benchmark shape."""
    import torch
    from oracle import inputs as oracle_inputs, seq_ref   # this leg times the oracle's CPU port
    T, H, C = 1024, 12, 64
    cores = min(os.cpu_count() or 1, int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    d = oracle_inputs.wkv7_inputs(sample_B, T, H, C, seed=1)
    dy = d['dy'].view(sample_B, T, H * C)

    def one(Tn):
        xs = [d[n].view(sample_B, T, H * C)[:, :Tn].clone().requires_grad_() for n in 'qwkvab']
        y = seq_ref.naive_recurrence_fp32(*xs, C)
        y.backward(dy[:, :Tn])

    one(T)  # warm-up at full length
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        one(T)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {'value': sample_B * T / med, 'unit': 'tokens/s', 'cores': torch.get_num_threads(), 'kind': 'port',
            'sample': f'B={sample_B} of 8, T=1024, H=12, N=64, fp32, fwd+bwd, one warm-up, median of {reps}'}


def other_workload(name, args):
    """Secondary workloads of the same path (not the headline metric): forward+backward of attn_ln (cfg2),
    ddlerp and expand_loras at the block's shape, and the whole TimeMixer block (cfg4).  Prints one JSON line
    with tokens/s and the whole-step algorithmic-bytes roofline fraction; used for the profiles/ summaries."""
    import torch
    from collections import namedtuple
    from wind_rwkv.rwkv7 import TimeMixer, ddlerp, expand_loras
    from wind_rwkv.rwkv7.wkv_attn_ln import WindRWKV7LN, attn_ln
    dev = torch.device('cuda:0')
    B, T, H, C = args.batch, 1024, 12, 64
    if name in ('attn_ln', 'wkv7_f32'):
        T, H = args.seq_len, args.heads
    HC = H * C
    if name in ('expand_loras', 'time_mixer', 'wkv7_f32'):
        H, C = HC // args.head_size, args.head_size
    if name == 'copy':
        # a plain device copy of known size: the calibration run for the FETCH_SIZE / WRITE_SIZE counters
        nbytes = 256 << 20
        src = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({'metric': 'device copy', 'bytes_read': nbytes, 'bytes_written': nbytes,
                          'launches': args.warmup + args.steps}))
        return
    if name == 'linear_wgrad':
        # the C x C weight gradient of one projection of the block (dW = dy^T x over B*T tokens): the one
        # matrix-core-bound kernel of the path, timed through the C ABI with HIP events on the launch stream
        from wind_rwkv import _native
        lib = _native.lib()
        tokens = B * T
        dy = torch.randn(tokens, HC, device=dev).bfloat16()
        x = torch.randn(tokens, HC, device=dev).bfloat16()
        dW = torch.empty(HC, HC, device=dev)
        ws_bytes = lib.wind_rwkv7_linear_wgrad_workspace_bytes(tokens, HC, HC)
        ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
        stream = torch.cuda.current_stream().cuda_stream

        def launch():
            _native.check(lib.wind_rwkv7_linear_wgrad(tokens, HC, HC, dy.data_ptr(), HC, x.data_ptr(), HC, dW.data_ptr(),
                                                      _native.F32, ws.data_ptr(), ws_bytes, stream))
        for _ in range(args.warmup):
            launch()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record()
        for _ in range(args.steps):
            launch()
        ev[1].record()
        torch.cuda.synchronize()
        dt = ev[0].elapsed_time(ev[1]) * 1e-3 / args.steps
        flops = 2.0 * tokens * HC * HC
        print(json.dumps({'metric': 'linear_wgrad TFLOP/s', 'value': flops / dt / 1e12, 'unit': 'TFLOP/s', 'n_gpus': 1,
                          'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': dt * 1e3, 'higher_is_better': True,
                          'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16', 'data': 'synthetic',
                          'config': {'workload': f'linear_wgrad: dW[{HC},{HC}] = dy^T x over {tokens} tokens, fp32 output'},
                          'roofline': {'bound': 'mfma', 'achieved': flops / dt / 1e12, 'peak': 2500.0, 'unit': 'TFLOP/s',
                                       'frac': flops / dt / 2.5e15, 'traffic': None,
                                       'algorithmic_flops_per_launch': flops}}))
        return
    if name == 'bighead':
        # WKV7 at head size 128 (768 channels = 6 heads; the reference: rwkv7_attn_triton_bighead.py): the bf16
        # matrix-core kernels for head sizes other than 64, or with --fp32-kernels the fp32 kernels they replaced
        from wind_rwkv.rwkv7.wkv_attn import WindRWKV7, WindRWKV7F32, no_state
        H, C = HC // 128, 128
        d = inputs.wkv7_inputs(B, T, H, C, 2, dtype=torch.bfloat16)
        cast = (lambda t: t.float()) if args.fp32_kernels else (lambda t: t)
        xs = [cast(d[n]).to(dev).requires_grad_() for n in ('w', 'q', 'k', 'v', 'a', 'b')]
        dy = cast(d['dy']).to(dev)
        s0 = torch.zeros(B, H, C, C, device=dev) if args.fp32_kernels else no_state(torch.bfloat16, dev)
        leaves = xs

        def step():
            y, _, _ = (WindRWKV7F32 if args.fp32_kernels else WindRWKV7).apply(*xs, s0)
            y.backward(dy)
        algo = 20 * B * T * HC * 2
        name = 'bighead (head size 128' + (', fp32 kernels)' if args.fp32_kernels else ')')
    elif name == 'wkv7_f32':
        # the accuracy mode: float32 sequences through the fp32 kernels (the reference: dot_prec='fp32',
        # rwkv7_attn_triton.py:159-190)
        from wind_rwkv.rwkv7.wkv_attn import WindRWKV7F32
        d = inputs.wkv7_inputs(B, T, H, C, 2, dtype=torch.float32)
        xs = [d[n].to(dev).requires_grad_() for n in ('w', 'q', 'k', 'v', 'a', 'b')]
        dy = d['dy'].to(dev)
        s0 = torch.zeros(B, H, C, C, device=dev)
        leaves = xs

        def step():
            y, _, _ = WindRWKV7F32.apply(*xs, s0)
            y.backward(dy)
        algo = 20 * B * T * HC * 4
    elif name == 'attn_ln':
        d = inputs.attn_ln_inputs(B, T, H, C, 2, dtype=torch.bfloat16)
        xs = [d[n].to(dev).requires_grad_() for n in ('w', 'q', 'k', 'v', 'a', 'b', 'g')]
        params = d['params'].to(dev).requires_grad_()
        s0 = torch.zeros(B, H, C, C, device=dev)
        dy = d['dy'].to(dev)
        leaves = xs + [params]

        def step():
            if args.forward_only:
                with torch.no_grad():   # the public wrapper: picks the forward that keeps nothing for backward
                    flat = [t.view(B, T, HC) for t in xs]
                    attn_ln(flat[1], flat[0], *flat[2:], params, C, s0=s0)
                return
            y, _, _ = WindRWKV7LN.apply(*xs, params, s0)
            y.backward(dy)
        algo = (8 if args.forward_only else 23) * B * T * HC * 2
    elif name == 'ddlerp':
        d = inputs.ddlerp_inputs(B, T, HC, args.rank or 32, 4, dtype=torch.bfloat16)
        x = d['x'].to(dev).requires_grad_()
        ps = [d[n].to(dev).requires_grad_() for n in ('alpha', 'L', 'R', 'beta')]
        dys = [g.to(dev) for g in d['dy']]
        leaves = [x] + ps

        def step():
            torch.autograd.backward(list(ddlerp(x, *ps)), dys)
        algo = 22 * HC * B * T
    elif name == 'expand_loras':
        names = ['w_in', 'k_in', 'z_in', 'a_in', 'ma_in', 'mk_in', 'Wz', 'Wa', 'Wma', 'Wmk', 'w_bias', 'a_bias',
                 'ma_bias', 'mk_bias']
        d = inputs.expand_loras_inputs(B, T, HC, args.rank or 16, 4, dtype=torch.bfloat16)
        leaves = [d[n].to(dev).requires_grad_() for n in names]
        dys = [g.to(dev) for g in d['dy']]

        def step():
            torch.autograd.backward(list(expand_loras(*leaves, args.head_size)), dys)
        algo = (28 * HC + 24 * (args.rank or 16)) * B * T
    elif name == 'decode':
        # one token per sequence through attn_ln_step: the state [B,H,64,64] fp32 is read and written once
        from wind_rwkv.rwkv7 import attn_ln_step
        d = inputs.attn_ln_inputs(B, 16, H, C, 5, dtype=torch.bfloat16)
        tok = {n: d[n][:, 0].reshape(B, HC).contiguous().to(dev) for n in ('q', 'w', 'k', 'v', 'a', 'b', 'g')}
        params = d['params'].to(dev)
        state = torch.zeros(B, H, C, C, device=dev)
        leaves = []
        T = 1

        def step():
            attn_ln_step(tok['q'], tok['w'], tok['k'], tok['v'], tok['a'], tok['b'], tok['g'], params, state, C)
        algo = 2 * B * H * C * C * 4 + 8 * B * HC * 2
    elif name == 'decode_block':
        # one token per sequence through the whole block: TimeMixer.step on a carried state
        Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
        torch.manual_seed(4)
        model = TimeMixer(Config(12, H, HC), 6).to(dev)
        with torch.no_grad():
            for p in model.parameters():
                p.normal_(std=0.1)
            _, state = model(torch.randn(B, 16, HC, device=dev).bfloat16(), return_state=True)
        tok = torch.randn(B, HC, device=dev).bfloat16()
        leaves = []
        T = 1

        def step():
            model.step(tok, state)
        algo = None
    else:  # time_mixer
        Config = namedtuple('Config', ['n_layer', 'n_head', 'n_embd'])
        torch.manual_seed(4)
        # (--fp32-kernels: the accuracy mode, fp32 WKV7 kernels with the epilogue in PyTorch)
        model = TimeMixer(Config(12, H, HC), 6, **({'attn_impl': 'triton'} if args.fp32_kernels else {})).to(dev)
        with torch.no_grad():
            for p in model.parameters():
                p.normal_(std=0.1)
        x = torch.randn(B, T, HC, device=dev, requires_grad=True)
        dy = torch.randn(B, T, HC, device=dev).bfloat16()
        leaves = [x] + list(model.parameters())

        def step():
            if args.forward_only:
                with torch.no_grad():
                    model(x)
                return
            model(x).backward(dy)
        algo = None

    def run():
        step()
        for t in leaves:
            t.grad = None

    if args.graph:
        # capture one step in a HIP graph and time replays: the block without host launch overhead
        # (the reference times its block under torch.compile(mode='reduce-overhead'), tests/test_time_mixer.py:90)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                run()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        run = graph.replay

    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    what = 'tokens/s' if name in ('decode', 'decode_block') else ('forward tokens/s' if args.forward_only else 'fwd+bwd tokens/s')
    out = {'metric': f'{name} {what}', 'value': B * T / dt, 'unit': 'tokens/s', 'n_gpus': 1,
           'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': dt * 1e3, 'higher_is_better': True,
           'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32' if name == 'wkv7_f32' else 'bf16', 'data': 'synthetic',
           'config': {'workload': (f'decode: one token for each of B={B} sequences through attn_ln_step, C={HC}, fp32 state'
                                   if name == 'decode' else
                                   f'decode_block: one token for each of B={B} sequences through TimeMixer.step, C={HC}'
                                   if name == 'decode_block' else f'{name}: B={B} T={T} C={HC} ({H} heads of {C}), '
                                   + ('forward only (no autograd)' if args.forward_only else 'forward+backward'))
                                  + (f', rank {args.rank}' if args.rank and name in ('ddlerp', 'expand_loras') else '')
                                  + (', replayed HIP graph' if args.graph else '')}}
    if algo:
        out['roofline_step'] = {'bound': 'hbm', 'algorithmic_bytes': algo, 'achieved': algo / dt / 1e9,
                                'peak': HBM_PEAK / 1e9, 'unit': 'GB/s', 'frac': algo / dt / HBM_PEAK}
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--workload', default='wkv7', choices=['wkv7', 'wkv7_f32', 'attn_ln', 'bighead', 'ddlerp', 'expand_loras', 'linear_wgrad', 'time_mixer', 'decode', 'decode_block', 'copy'],
                    help='wkv7 (default) is the headline benchmark; the others time neighbouring stages of the path')
    ap.add_argument('--eager', action='store_true', help='headline workload: time eager launches instead of graph replays')
    ap.add_argument('--seq-len', type=int, default=1024, help='headline and attn_ln workloads: tokens per sequence (default 1024)')
    ap.add_argument('--heads', type=int, default=12, help='headline and attn_ln workloads: heads of 64 channels (default 12)')
    ap.add_argument('--fp32-kernels', action='store_true', help='bighead and time_mixer workloads: the fp32 kernels instead of the bf16 matrix-core ones')
    ap.add_argument('--rank', type=int, default=0, help='ddlerp (default 32) and expand_loras (default 16) workloads: the LoRA rank')
    ap.add_argument('--head-size', type=int, default=64, help='expand_loras, time_mixer and wkv7_f32 workloads: channels per head (default 64)')
    ap.add_argument('--forward-only', action='store_true', help='attn_ln and time_mixer workloads: the forward pass alone, without autograd (prefill)')
    ap.add_argument('--graph', action='store_true', help='secondary workloads: time replays of a captured HIP graph')
    ap.add_argument('--input-sets', type=int, default=1,
                    help='headline workload: rotate the steps over this many independent sets of tensors, so that '
                         'with enough sets (4 at the default shape: 4 x 101 MB of inputs and 4 x 88 MB of outputs '
                         'against the 256 MB last-level cache) no step finds its inputs cached from the step before')
    ap.add_argument('--batch', type=int, default=8, help='batch size (8 is the shape the headline metric is quoted on)')
    ap.add_argument('--checkpoint-interval', type=int, default=0, choices=[0, 16, 32],
                    help='tokens between the states kept for backward (library default: 32, two-level chunking; 16: a state per chunk)')
    ap.add_argument('--record-traffic', nargs=4, metavar=('FETCH_CSV', 'WRITE_CSV', 'COPY_FETCH_CSV', 'COPY_WRITE_CSV'),
                    help='no GPU work: write profiles/wkv7_cfg1_hbm_traffic.json from rocprofv3 --pmc counter CSVs')
    args = ap.parse_args()
    if args.record_traffic:
        record_traffic(*args.record_traffic)
        return
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        sys.exit('bench.py measures one GPU: this build has no multi-GPU path (every (batch, head) pair is an '
                 'independent recurrence; run one process per GPU on a shard of the batch). Use --gpus 1.')

    import torch
    from wind_rwkv import _native
    from wind_rwkv.rwkv7.wkv_attn import WindRWKV7

    if not torch.cuda.is_available():
        sys.exit('bench.py needs an AMD GPU')
    lib = _native.lib()
    if args.checkpoint_interval:
        _native.check(lib.wind_rwkv7_set_checkpoint_interval(args.checkpoint_interval))
    if args.workload != 'wkv7':
        return other_workload(args.workload, args)
    dev = torch.device('cuda:0')
    B, T, H, C = args.batch, args.seq_len, args.heads, 64   # the headline metric is quoted at the defaults
    d = inputs.wkv7_inputs(B, T, H, C, seed=1, dtype=torch.bfloat16)
    sets = [([d[n].to(dev).clone().requires_grad_() for n in ('w', 'q', 'k', 'v', 'a', 'b')], d['dy'].to(dev).clone())
            for _ in range(max(args.input_sets, 1))]
    s0 = torch.zeros(B, H, C, C, device=dev)

    def step(i=0):
        xs, dy = sets[i % len(sets)]
        y, sT, s = WindRWKV7.apply(*xs, s0)
        torch.autograd.backward([y], [dy])
        for x in xs:
            x.grad = None

    def timed(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    # The three kernels of a step take ~150 us and the Python autograd machinery ~100 us to issue them: an eager
    # loop keeps up only while nothing disturbs the host, so the step is captured once in a HIP graph and the
    # timed region replays it (the reference times its kernels under torch.compile(mode='reduce-overhead'), i.e.
    # graph replay, tests/test_attn_ln.py:52).  The eager figure (same number of steps, after its own warm-up)
    # is reported beside it.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for i in range(max(args.warmup, 10)):
        step(i)
    eager_ms = timed(step, args.steps) / args.steps * 1e3
    if args.eager:
        run = step
    else:
        graphs = []
        for i in range(len(sets)):
            graphs.append(torch.cuda.CUDAGraph())
            with torch.cuda.graph(graphs[-1]):
                step(i)
        run = lambda i: graphs[i % len(graphs)].replay()
    for i in range(args.warmup):
        run(i)
    elapsed = timed(run, args.steps)
    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = B * T * args.steps / elapsed

    # per-kernel durations from HIP events on the launch stream (separate, untimed passes)
    lib.wind_rwkv7_profile_enable(1)
    acc = {}
    n_prof = 10
    buf = (ctypes.c_float * 8)()
    for i in range(n_prof):
        step(i)
        for direction in (0, 1):
            n = lib.wind_rwkv7_profile_read(direction, buf, 8)
            for i in range(max(n, 0)):
                acc.setdefault(lib.wind_rwkv7_profile_kernel_name(direction, i).decode(), []).append(buf[i])
    lib.wind_rwkv7_profile_enable(0)
    kernels_ms = {k: sum(v) / len(v) for k, v in acc.items()}
    dominant = max(kernels_ms, key=kernels_ms.get)
    unit_bytes = C * 2  # one bf16 head-row
    units = B * T * H
    dom_bytes = ALGO_PASSES[dominant] * unit_bytes * units
    dom_ms = kernels_ms[dominant]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    step_bytes = ALGO_PASSES['step'] * unit_bytes * units
    kernel_sum_ms = sum(kernels_ms.values())
    # counter figures are per launch at cfg1; other shapes scale with the token-head count
    traffic, traffic_stale = load_traffic()
    scaled = lambda k: traffic[k] * units // (8 * 1024 * 12) if k in traffic else None

    out = {
        'metric': f'WKV7 fwd+bwd tokens/s at B{B}·T{T}·H{H}·N64 bf16; % of MFMA/HBM roofline',
        'value': tokens_per_s, 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': ms_per_step, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'data': 'synthetic',
        'config': {'workload': f'{"cfg1: " if (B, T, H) == (8, 1024, 12) else ""}WKV7 forward+backward, B={B} T={T} H={H} N=64, bf16 sequences, fp32 state, chunk 16, state checkpoints every {lib.wind_rwkv7_checkpoint_interval()} tokens',
                   'tokens_per_step': B * T, 'launch': 'eager' if args.eager else 'replayed HIP graph of one autograd forward+backward',
                   'eager_ms_per_step': eager_ms, 'input_sets': len(sets)},
        'roofline': {'bound': 'hbm', 'kernel': dominant, 'achieved': achieved, 'peak': HBM_PEAK / 1e9, 'unit': 'GB/s',
                     'frac': achieved / (HBM_PEAK / 1e9), 'traffic': scaled(dominant),
                     'algorithmic_bytes_per_launch': dom_bytes, 'avg_launch_ms': dom_ms},
        'roofline_step': {'bound': 'hbm', 'algorithmic_bytes': step_bytes,
                          'achieved': step_bytes / (ms_per_step * 1e-3) / 1e9, 'peak': HBM_PEAK / 1e9, 'unit': 'GB/s',
                          'frac': step_bytes / (ms_per_step * 1e-3) / HBM_PEAK,
                          'frac_kernels_only': step_bytes / (kernel_sum_ms * 1e-3) / HBM_PEAK},
        'mfma_fraction': FLOPS_PER_TOKEN_HEAD * units / (ms_per_step * 1e-3) / MFMA_PEAK_BF16,
        'kernels_ms': kernels_ms,
        'kernels_traffic_bytes': {k: scaled(k) for k in kernels_ms},
    }
    if traffic_stale:
        out['traffic_note'] = 'kernel sources changed since the counters in profiles/wkv7_cfg1_hbm_traffic.json were read'
    out['measured_peaks'] = measured_peaks()
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline()
    print(json.dumps(out))


if __name__ == '__main__':
    main()
