import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import ix_oracle

    ix_oracle.build()
    return ix_oracle


@pytest.fixture
def force_decoder():
    """Force one of the library's decoders for the duration of a test (``ixh_set_option``), then give the choice
    back to the library."""
    from ixrun_amd import _lib

    def force(name: str) -> None:
        _lib.set_option("decode_kernel", name)

    yield force
    _lib.set_option("decode_kernel", "auto")
