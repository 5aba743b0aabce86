import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


@pytest.fixture(scope="session")
def golden():
    """Vectors produced by the reference itself (tests/golden/make_golden.py)."""
    return np.load(os.path.join(ROOT, "tests", "golden", "golden_v1.npz"))


@pytest.fixture(scope="session")
def tri_widths():
    """TriAttention at coefficient widths 8 / 16 and post-RoPE scoring, produced by the reference itself
    (tests/golden/make_golden_tri_widths.py)."""
    return np.load(os.path.join(ROOT, "tests", "golden", "golden_tri_widths.npz"))


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def tq25():
    """HybridTurboQuant in mode tq25 (sign vectors, codebooks, encode / decode), produced by the reference
    itself (tests/golden/make_golden_tq25.py)."""
    return np.load(os.path.join(ROOT, "tests", "golden", "golden_tq25.npz"))
