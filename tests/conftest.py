import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# Switches of the environment that keep one kernel for every shape (for comparing kernels: same results, other
# launches).  Assertions about WHICH kernel a shape takes hold for the library's own choice only.
KERNEL_SWITCHES = ("PIMDL_CCS_EXACT", "PIMDL_CCS_F32", "PIMDL_GATHER_ROWS", "PIMDL_GATHER_DENSE")


def kernel_switches():
    return [e for e in KERNEL_SWITCHES if os.environ.get(e) == "1"]


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_index():
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "index_calc_golden.npz")
    return np.load(path, allow_pickle=False)
