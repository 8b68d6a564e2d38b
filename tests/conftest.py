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


@pytest.fixture
def gemv_option():
    """Set a kernel-selection switch of ixh_gemv or ixh_gemm for the duration of a test (``ixh_set_option``)."""
    from ixrun_amd import _lib

    defaults = {"gemv_strips": 0, "gemv_shared_x": 8, "gemv_tiles": 0, "gemv_tile_rows": 0, "gemv_tile_cus": 0, "gemv_tile_split": 0, "gemv_dense_tiles": 0, "gemv_slots": 0, "gemv_slot_waves": 0, "gemm_tiles": 0}
    touched = []

    def set_(name: str, value: int) -> None:
        touched.append(name)
        _lib.set_option(name, value)

    yield set_
    for name in touched:
        _lib.set_option(name, defaults[name])
