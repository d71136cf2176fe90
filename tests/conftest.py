import os
import sys

import pytest

TESTS = os.path.dirname(os.path.realpath(__file__))
ROOT = os.path.dirname(TESTS)
for path in (TESTS, ROOT):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def _built_libraries():
    """Load what is built; compile only what is missing (the GPU box has no reference checkout and does not need
    one: the prebuilt oracle/_ref travels with the tree)."""
    import oracle
    from vesin_amd import _build

    if not os.path.exists(_build.LIB_PATH):
        _build.build()
    if not os.path.exists(_build.TORCH_LIB_PATH):
        _build.build_torch()
    if not os.path.exists(oracle.ORACLE_LIB):
        oracle.build()
