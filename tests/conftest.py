import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def capi():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from dynamiq_sigcomm_artifact_amd import capi as C
    C.lib()
    return C


@pytest.fixture(scope="session")
def eden_utils():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import dynamiq_sigcomm_artifact_amd as pkg
    return pkg.load_eden_utils()
