import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    import oracle
    return oracle.Oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own compiled code; present only where oracle/_ref has been built."""
    import oracle
    if not oracle.Reference.available():
        pytest.skip("oracle/_ref/libggml_ref.so not built (needs the reference tree)")
    return oracle.Reference()
