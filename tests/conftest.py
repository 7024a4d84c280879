import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    from __graft_entry__ import load_package
    return load_package()


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def T(dev):
    import torch

    class Helper:
        def t(self, x):
            return torch.from_numpy(np.ascontiguousarray(x)).to(dev)

        def f1(self, v):
            return torch.tensor([v], dtype=torch.float32, device=dev)

        def n(self, x):
            torch.cuda.synchronize()
            return x.cpu().numpy()
    return Helper()


def rel_fro(got, want64):
    return np.linalg.norm(got.astype(np.float64) - want64) / max(np.linalg.norm(want64), 1e-300)
