import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu on the GPU box)')


@pytest.fixture(scope='session', autouse=True)
def _seed():
    import numpy as np
    import torch

    np.random.seed(42)
    torch.manual_seed(42)


@pytest.fixture(scope='session')
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip('no GPU')
    return torch.device('cuda:0')


@pytest.fixture
def acc64():
    """The oracle's contractions in float64 (its quantizers stay fp32) for the duration of a test."""
    from oracle import hgq_ref

    hgq_ref.ACC64 = True
    yield
    hgq_ref.ACC64 = False
