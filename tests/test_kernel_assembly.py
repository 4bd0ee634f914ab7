"""A guard on the compiled kernels (no GPU needed: hipcc cross-compiles to assembly here).

This compiler release places no wait states between two matrix instructions of DIFFERENT shapes when the second takes
the first one's result as its accumulator (seen with v_mfma_f32_16x16x32_bf16 followed by v_mfma_f32_16x16x16_bf16:
emitted back to back, and the triangular inverse built that way came out wrong by 1e-3 on the GPU).  The sources
therefore never chain shapes through the accumulator; this test scans the assembly of every kernel file that uses
matrix instructions for such a pair, so that a later edit cannot reintroduce one unnoticed.
"""
import os
import re
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, 'wind-rwkv7_amd', 'csrc')
HIPCC = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
MAKEFILE = os.path.join(ROOT, 'wind-rwkv7_amd', 'Makefile')


def makefile_flags():
    """(common flags, {file name: extra flags}) as the package's Makefile sets them, so that the assembly scanned here
    is that of the shipped objects: HIPFLAGS for every file, and the per-target `EXTRA := $(VAR)` lines."""
    text = open(MAKEFILE).read()
    var = dict(re.findall(r'^(\w+)\s*[:?]?=\s*(.*)$', text, flags=re.M))
    expand = lambda v: re.sub(r'\$\((\w+)\)', lambda m: expand(var.get(m.group(1), '')), v)
    common = [f for f in expand(var['HIPFLAGS']).split() if f != '-fPIC']
    extra = {}
    for targets, value in re.findall(r'^((?:build/\w+\.o\s*)+):\s*EXTRA\s*:=\s*(.*)$', text, flags=re.M):
        for t in targets.split():
            extra[os.path.basename(t)[:-2] + '.hip'] = expand(value).split()
    return common, extra


FLAGS, EXTRA = makefile_flags()
FLAGS = FLAGS + ['-S', '--cuda-device-only']
FILES = ['wkv7_fused.hip', 'wkv7_bwd.hip', 'wkv7_fwd.hip', 'wkv7_wide.hip', 'ddlerp.hip', 'expand_loras.hip', 'mixer_decode.hip',
         'linear_wgrad.hip', 'selftest.hip', 'wkv7_f32.hip']
WINDOW = 16   # instructions; a matrix instruction has long finished after that many

MFMA = re.compile(r'(v_mfma_\w+)\s+([av]\[\d+:\d+\]),\s*(?:[av]\[\d+:\d+\]|v\d+),\s*(?:[av]\[\d+:\d+\]|v\d+),\s*([av]\[\d+:\d+\]|0)')


DEST = re.compile(r'v_\w+\s+(v\d+|v\[\d+:\d+\])')


def _regs(operand):
    m = re.match(r'[av]\[(\d+):(\d+)\]', operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    return {int(operand[1:])}


def mixed_pairs(asm):
    ins = [t.strip() for t in asm.split('\n')]
    ins = [t for t in ins if t and not t.startswith((';', '.')) and not t.endswith(':')]
    found = []
    for i, t in enumerate(ins):
        m = MFMA.match(t)
        if not m or m.group(3) == '0':
            continue
        pending = _regs(m.group(3)) if m.group(3)[0] == 'v' else None   # accumulator registers not yet seen rewritten
        for j in range(i - 1, max(i - 1 - WINDOW, -1), -1):
            p = MFMA.match(ins[j])
            if p and p.group(2) == m.group(3):      # the producer of this instruction's accumulator
                if p.group(1) != m.group(1):
                    found.append((ins[j], t))
                break
            # a vector instruction in between that rewrites the whole accumulator range: the matrix instruction before
            # it is not what this one accumulates onto (the registers were merely reused)
            d = DEST.match(ins[j])
            if d and pending is not None and not p:
                pending -= _regs(d.group(1))
                if not pending:
                    break
    return found


def test_flags_are_the_makefiles():
    assert '--offload-arch=gfx950' in FLAGS and '-O3' in FLAGS
    assert EXTRA['wkv7_fused.hip'] == ['-mllvm', '-amdgpu-mfma-vgpr-form'] and 'expand_loras.hip' not in EXTRA


def test_scanner_sees_a_mixed_pair():
    asm = '''
        v_mfma_f32_16x16x32_bf16 v[68:71], v[76:79], v[68:71], v[2:5]
        v_mfma_f32_16x16x16_bf16 v[66:69], v[66:67], v[72:73], v[68:71]
        v_mfma_f32_16x16x16_bf16 v[66:69], v[66:67], v[72:73], v[66:69]
    '''
    assert len(mixed_pairs(asm)) == 1
    reused = '''
        v_mfma_f32_16x16x16_bf16 v[56:59], v[24:25], v[252:253], 0
        v_cvt_pk_bf16_f32 v62, v56, v57
        v_and_b32_e32 v59, 0xffff0000, v43
        v_lshlrev_b32_e32 v58, 16, v43
        v_and_b32_e32 v57, 0xffff0000, v42
        v_lshlrev_b32_e32 v56, 16, v42
        v_mfma_f32_16x16x32_bf16 v[56:59], v[60:63], v[12:15], v[56:59]
    '''
    assert mixed_pairs(reused) == []       # the accumulator registers were rewritten in between
    partly = reused.replace('v_and_b32_e32 v59, 0xffff0000, v43', '')
    assert len(mixed_pairs(partly)) == 1   # one register still holds the first instruction's result


@pytest.mark.skipif(not os.path.exists(HIPCC), reason='hipcc not found')
def test_no_matrix_instructions_of_different_shapes_chained_through_the_accumulator():
    with tempfile.TemporaryDirectory() as tmp:
        def compile_one(name):
            out = os.path.join(tmp, name + '.s')
            extra = EXTRA.get(name, [])
            subprocess.run([HIPCC, *FLAGS, *extra, '-o', out, os.path.join(CSRC, name)], check=True,
                           stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
            with open(out) as f:
                return name, f.read()
        with ThreadPoolExecutor(max_workers=4) as pool:
            results = list(pool.map(compile_one, FILES))
    bad = {name: pairs[:3] for name, asm in results if (pairs := mixed_pairs(asm))}
    assert not bad, bad
    # The WKV7 kernels must not spill to scratch memory.  In the lock-step kernels a spilling wavefront holds up all
    # the others at every barrier; in the gradient kernel every reload of a spilled register makes the compiler wait
    # for ALL outstanding memory operations (scratch accesses count as loads of unknown order), which ends the overlap
    # of the next chunk's prefetch with this chunk's arithmetic.
    spilling = {}
    for name, asm in results:
        # (the fp32 kernels: their backward sits at the register limit of a wavefront, so a change that tips it over shows here)
        if name in ('wkv7_fused.hip', 'wkv7_bwd.hip', 'wkv7_fwd.hip', 'wkv7_f32.hip'):
            for kernel, size in re.findall(r'\.name:\s+(\S+)\n(?:.*\n)*?\s+\.private_segment_fixed_size:\s+(\d+)', asm):
                if int(size):
                    spilling[kernel] = int(size)
    assert not spilling, spilling
