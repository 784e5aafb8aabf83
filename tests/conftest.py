import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def bf16_round(x):
    """Round a float array to bf16-representable float32 values (round-to-nearest-even)."""
    import numpy as np
    import torch

    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.bfloat16).float().numpy()


@pytest.fixture
def rng():
    import numpy as np

    return np.random.default_rng(20250)
