import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # the tests load the library that is built in-tree; only a tree without one builds it first
    from universal_attention_triton_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from universal_attention_triton_amd import build
        build.build()


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")
