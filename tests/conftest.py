import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real GPU (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "codec_vectors.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def oracle_codec():
    from oracle import codec
    return codec.oracle()


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    from packkv_amd import _lib
    _lib.load()   # the HIP library must be there: no fallback
    return torch.device("cuda:0")
