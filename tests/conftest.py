import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def nonzero_randn(shape, *, dtype=torch.float32, seed=0, floor=0.2):
    """Seeded normal samples pushed away from zero so signs are unambiguous."""

    generator = torch.Generator().manual_seed(seed)
    values = torch.randn(shape, dtype=torch.float64, generator=generator)
    signs = torch.where(values >= 0, 1.0, -1.0)
    return (signs * (values.abs() + floor)).to(dtype)


@pytest.fixture(scope="session")
def c_oracle():
    from oracle import c_oracle as module

    module.load()
    return module
