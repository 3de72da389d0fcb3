import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run through the C-ABI of the HIP library)")
    config.addinivalue_line("markers", "ref: needs the compiled reference under oracle/_ref (built by oracle/Makefile)")


def pytest_collection_modifyitems(config, items):
    from oracle import ref
    if ref.available():
        return
    skip = pytest.mark.skip(reason="oracle/_ref/libexcalibur_ref.so not built (needs the reference sources)")
    for item in items:
        if "ref" in item.keywords:
            item.add_marker(skip)
