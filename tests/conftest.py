import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: exhaustive CPU check, opt in with -m slow")


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "dequant_golden.npz")
    return np.load(path, allow_pickle=False)


TUNING_KEYS = ("rows8_shape", "gemv_shape", "gemm_ksplit", "dense_tile", "dense_mfma16", "dense_pf")


@pytest.fixture
def tuning():
    """Forces launch shapes through cuthip_set_tuning for the duration of one test; every key is restored afterwards."""
    from cut_amd import lib

    yield lib.set_tuning
    for key in TUNING_KEYS:
        lib.set_tuning(key, None)
