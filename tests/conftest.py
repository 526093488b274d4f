import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, 'oracle')):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu on the GPU box)')


@pytest.fixture(scope='session')
def dev():
    """GPU device for parity tests.  Fails (does not skip) without a GPU so a
    silent CPU pass can never be mistaken for a GPU pass."""
    import torch
    assert torch.cuda.is_available(), 'GPU tests need a GPU'
    from var_q_amd import _lib
    _lib.load()
    return torch.device('cuda:0')
