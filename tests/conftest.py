"""Shared test configuration: the ``gpu`` marker and the dimension lists of the reference's suites
(tests/conftest.py:40-66 of the reference)."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HAS_GPU = torch.cuda.is_available()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if HAS_GPU:
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def tb_option():
    """Set tuning / test hooks of the library for one test (tb_debug_option); they go back to their
    defaults afterwards.  The hooks' environment variables are read only once per process."""
    from tritonblas_amd import _lib
    changed = []

    def set_option(name, value):
        _lib.debug_option(name, value)
        changed.append(name)

    yield set_option
    for name in changed:
        _lib.debug_option(name, -1 if name == "panel" else 0)


STANDARD_DIMS = [(128, 256, 512), (256, 256, 256), (512, 1024, 768), (768, 1024, 512), (2048, 1024, 512), (1024, 2048, 512)]
EDGE_CASE_DIMS = [(32, 32, 32), (64, 16, 128), (16, 64, 128), (128, 8, 256), (8, 128, 256), (12, 12, 512), (15, 17, 512),
                  (19, 13, 512), (128, 64, 12)]
SKINNY_DIMS = [(16, 16, 4096), (32, 32, 8192)]
DTYPES = [torch.bfloat16, torch.float16]
