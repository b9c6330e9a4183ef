import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "sage_attention: SageAttention forward path (the reference's own marker, pytest.ini:6)")


@pytest.fixture(scope="session")
def sage_lib():
    from baselinebenchmark_amd import _cabi
    return _cabi.lib()


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "quant_golden.npz"))
