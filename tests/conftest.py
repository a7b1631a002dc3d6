import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def golden(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


@pytest.fixture(scope="session")
def oracle():
    from oracle import exl3_oracle

    exl3_oracle.lib()
    return exl3_oracle


@pytest.fixture(scope="session")
def cuda():
    """GPU tests were asked for explicitly (-m gpu): a missing GPU or a missing
    HIP library is a failure, never a skip."""
    import torch

    assert torch.cuda.is_available(), "GPU test selected but no HIP device is visible"
    from ponyexl3_amd import _lib

    _lib.load()
    return torch.device("cuda:0")


def rel_l2(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30))
