"""ctypes binding of oracle/wkv7_oracle.c.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py)."""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, 'libwkv7_oracle.so')
_lib = None


def build():
    """Compile the C oracle next to its source."""
    subprocess.run(['make', '-C', _HERE, '-B', 'libwkv7_oracle.so'], check=True, capture_output=True)


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        dp = ctypes.POINTER(ctypes.c_double)
        _lib.wkv7_oracle_forward.argtypes = [ctypes.c_int] * 4 + [dp] * 9
        _lib.wkv7_oracle_forward.restype = ctypes.c_int
        _lib.wkv7_oracle_backward.argtypes = [ctypes.c_int] * 4 + [dp] * 16
        _lib.wkv7_oracle_backward.restype = ctypes.c_int
    return _lib


def _np(t):
    return np.ascontiguousarray(t.detach().to(torch.float64).cpu().numpy())


def _p(x):
    return x.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def forward(q, w, k, v, a, b, s0):
    """q..b: [B,T,H,C] tensors (any float dtype), s0 [B,H,C,C].  Returns fp64 (y, sT)."""
    B, T, H, C = q.shape
    arrs = [_np(x) for x in (q, w, k, v, a, b, s0)]
    y = np.empty((B, T, H, C))
    sT = np.empty((B, H, C, C))
    rc = _load().wkv7_oracle_forward(B, T, H, C, *[_p(x) for x in arrs], _p(y), _p(sT))
    assert rc == 0
    return torch.from_numpy(y), torch.from_numpy(sT)


def backward(q, w, k, v, a, b, s0, dy, dsT):
    """Returns fp64 (dq, dw, dk, dv, da, db, ds0)."""
    B, T, H, C = q.shape
    arrs = [_np(x) for x in (q, w, k, v, a, b, s0, dy, dsT)]
    outs = [np.empty((B, T, H, C)) for _ in range(6)] + [np.empty((B, H, C, C))]
    rc = _load().wkv7_oracle_backward(B, T, H, C, *[_p(x) for x in arrs], *[_p(x) for x in outs])
    assert rc == 0
    return tuple(torch.from_numpy(x) for x in outs)


class Wkv7(torch.autograd.Function):
    """The C restatement as a differentiable fp64 operator with zero initial state: lets the block oracle
    (seq_ref.time_mixer_seq) run at the full benchmark size, where autograd's tape over the token loop would not fit.
    (q, w, k, v, a, b) [B,T,H,C] -> y."""

    @staticmethod
    def forward(ctx, q, w, k, v, a, b):
        B, T, H, C = q.shape
        s0 = torch.zeros(B, H, C, C, dtype=torch.float64)
        y, _ = forward(q, w, k, v, a, b, s0)
        ctx.save_for_backward(q, w, k, v, a, b)
        return y.to(q.dtype)

    @staticmethod
    def backward(ctx, dy):
        q, w, k, v, a, b = ctx.saved_tensors
        B, T, H, C = q.shape
        z = torch.zeros(B, H, C, C, dtype=torch.float64)
        dq, dw, dk, dv, da, db, _ = backward(q, w, k, v, a, b, z, dy, z)
        return tuple(g.to(q.dtype) for g in (dq, dw, dk, dv, da, db))


def wkv7(q, w, k, v, a, b, s0=None):
    """Drop-in for seq_ref.wkv7_seq with s0 = None; returns (y, None)."""
    assert s0 is None
    return Wkv7.apply(q, w, k, v, a, b), None
