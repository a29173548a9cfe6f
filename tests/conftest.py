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
    """The CPU parity oracle: the reference's own translation unit when it has
    been built (oracle/_ref), else this repository's C restatement."""
    from oracle import build as obuild
    from oracle import qref

    if not os.path.isfile(qref.QREF_SO):
        obuild.build_qref()
    kind = "reference" if qref.reference_built() else "port"
    return qref.Oracle(kind)


@pytest.fixture(scope="session")
def port_oracle():
    from oracle import build as obuild
    from oracle import qref

    if not os.path.isfile(qref.QREF_SO):
        obuild.build_qref()
    return qref.Oracle("port")


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("test is marked gpu but no GPU is visible")
    from mlx_amd import _lib

    _lib.load()  # no CPU fallback: fail loudly if the HIP library is missing
    return torch.device("cuda:0")
