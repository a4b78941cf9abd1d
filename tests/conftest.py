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
    from oracle.ftnn_oracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    from oracle.ftnn_oracle import Reference
    if not Reference.available():
        pytest.skip("compiled reference (oracle/_ref) not present")
    return Reference()


@pytest.fixture(scope="session")
def reference_baseline():
    from oracle.ftnn_oracle import ReferenceBaseline
    if not ReferenceBaseline.available():
        pytest.skip("compiled reference baseline (oracle/_ref) not present")
    return ReferenceBaseline()


@pytest.fixture(scope="session")
def hip():
    """The HIP library binding; fails (does not skip) when the library is missing."""
    import torch
    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    import fastertnn_amd.lib as lib
    return lib
