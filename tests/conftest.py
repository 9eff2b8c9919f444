import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure); built on demand with gcc."""
    from oracle import oracle as mod

    mod.lib()
    return mod


@pytest.fixture(scope="session")
def ocn():
    """The product package; needs the built HIP library (build it if nothing is built)."""
    import opencnn_amd

    if not os.path.exists(opencnn_amd.LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()
    opencnn_amd.load_library()
    return opencnn_amd


@pytest.fixture(scope="session")
def torch_gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests need a real MI355X")
    return torch
