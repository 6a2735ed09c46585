import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    """The loaded C-ABI library; built first only if no built library is present."""
    from flash_muon_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from flash_muon_amd import build
        build.build(verbose=False)
    return _lib.load()


KNOBS = {"FLASHMUON_GRID": 0, "FLASHMUON_KSPLIT": 1, "FLASHMUON_FAST_MIN_UNITS": 2, "FLASHMUON_NO_MID": 3,
         "FLASHMUON_NO_SUB64": 4, "FLASHMUON_HALF": 5, "FLASHMUON_DIAG_LAST": 6, "FLASHMUON_NO_TICKETS": 7}


@pytest.fixture
def knobs(lib):
    """set(name, value) turns a tuning knob of the library (fm_set_knob) for the length of one test;
    afterwards every knob is back on automatic."""
    def set(name, value):
        assert lib.fm_set_knob(KNOBS[name], int(value)) == 0
    yield set
    for k in KNOBS.values():
        lib.fm_set_knob(k, -1)
