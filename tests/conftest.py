import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "flash-3-way-attention_amd")
for p in (ROOT, PKG_DIR):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def tune():
    """tune(knob, value): sets a tuning knob of the library (tritt_set_tuning) for the rest of the test; every
    knob the test touched goes back to its previous value afterwards."""
    from flash_trittention import _lib

    first = {}

    def set_knob(knob, value):
        previous = _lib.set_tuning(knob, value)
        first.setdefault(knob, previous)

    yield set_knob
    for knob, previous in first.items():
        _lib.set_tuning(knob, previous)
