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
    from oracle.binding import Oracle

    return Oracle()


@pytest.fixture
def blend_form():
    """Returns a function that forces one form of the blend kernels (1 or 4 pixels per lane) for the
    rest of the test; the library's own choice by image size is restored afterwards."""
    from ds_splat_amd import _native
    lib = _native.load()

    def force(pixels_per_lane):
        _native.check(lib.dsx_set_blend_pixels_per_lane(int(pixels_per_lane)))

    yield force
    _native.check(lib.dsx_set_blend_pixels_per_lane(0))


@pytest.fixture
def list_bin():
    """Returns a function that sets the bin size of the tile lists (1, 2, 4 or 8 tiles a side; 0: the
    library's choice) that this package's callers ask for by default, for the rest of the test; the
    library's own choice is restored afterwards.  (The native library has no such setting: the Python
    callers pass the value with every call.)"""
    from ds_splat_amd import _native

    def force(tiles_per_side):
        _native.set_default_list_bin(int(tiles_per_side))

    yield force
    _native.set_default_list_bin(0)
