import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip_lib():
    """The C-ABI library; built on demand only when no built copy exists."""
    from latentq_llm_amd import _C
    if not os.path.exists(_C.LIB_PATH):
        from latentq_llm_amd.build import build_library
        build_library()
    return _C.load()
