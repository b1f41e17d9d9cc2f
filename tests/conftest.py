import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

REF_SO = os.path.join(ROOT, "oracle", "_ref", "libnart_ref.so")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ref_ws():
    """A workspace of the reference CPU `quant` module, compiled from the reference's own sources by
    oracle/Makefile.  Absent wherever the reference tree was never mounted: those tests skip and the
    committed golden outputs (tests/golden) stand in."""
    if not os.path.exists(REF_SO):
        pytest.skip("oracle/_ref not built (reference sources not available here)")
    from nart_amd import art
    rt = art.Runtime(REF_SO)
    return rt.workspace("quant")
