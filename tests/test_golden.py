"""The committed golden vectors (tests/golden/*.npz) against today's oracle.

The vectors were written once by tests/golden/make_fixtures.py.  Recomputing them here means that an edit of
oracle/ which changes any result fails, and the C restatement of the WKV7 recurrence is held to the same
numbers as the autograd one.  (The reference itself ships no fixtures: tests/test_attn.py:34-48 draws unseeded
data.)
"""
import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
_spec = importlib.util.spec_from_file_location('make_fixtures', os.path.join(HERE, 'make_fixtures.py'))
make_fixtures = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_fixtures)


def _close(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64))) <= 1e-6 * max(float(np.linalg.norm(b.astype(np.float64))), 1e-30)


@pytest.mark.parametrize('name', sorted(make_fixtures.CASES))
def test_oracle_reproduces_the_golden_vectors(name):
    stored = np.load(os.path.join(HERE, name))
    fresh = make_fixtures.CASES[name]()
    assert sorted(stored.files) == sorted(fresh)
    for key in stored.files:
        if key.startswith('in_') and stored[key].dtype == np.uint16:
            assert np.array_equal(stored[key], fresh[key]), key       # the seeded inputs, bit for bit
        else:
            assert _close(fresh[key], stored[key]), key


def test_c_oracle_matches_the_wkv7_golden_vectors(c_oracle):
    z = np.load(os.path.join(HERE, 'wkv7_b1_t32_h2.npz'))
    bf = lambda k: torch.from_numpy(z[k].view(np.int16).copy()).view(torch.bfloat16)
    args = [bf('in_' + n) for n in 'qwkvab']
    s0, dsT = torch.from_numpy(z['in_s0']), torch.from_numpy(z['in_dsT'])
    y, sT = c_oracle.forward(*args, s0)
    g = c_oracle.backward(*args, s0, bf('in_dy'), dsT)            # dq, dw, dk, dv, da, db, ds0
    assert _close(y.numpy(), z['y']) and _close(sT.numpy(), z['sT'])
    for name, got in zip(['dq', 'dw', 'dk', 'dv', 'da', 'db', 'ds0'], g):
        assert _close(got.numpy(), z[name]), name
