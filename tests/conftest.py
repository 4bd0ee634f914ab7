"""Shared test plumbing: import paths, the `gpu` marker, the oracle and the package."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_ROOT = os.path.join(ROOT, 'wind-rwkv7_amd')
for p in (ROOT, PKG_ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs an AMD GPU (MI355X); run with -m gpu on the GPU box')


def pytest_collection_modifyitems(config, items):
    """Tests marked gpu are skipped (not failed) when no device is visible, so that a plain
    `pytest tests` still works on a CPU-only machine."""
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason='no GPU visible')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope='session')
def c_oracle():
    from oracle import c_oracle as mod
    mod._load()
    return mod
