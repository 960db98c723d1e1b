import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# The Q6_K matrix-core GEMV is only chosen for very large matrices (an output head); the parity tests run it on
# ordinary shapes as well.  The library reads the variable once, at its first multi-token Q6_K call.
os.environ.setdefault("CHIP_MMV_Q6K", "1")
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
