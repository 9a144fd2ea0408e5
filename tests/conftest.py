import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from tests import oracle_lib
    return oracle_lib.oracle()


@pytest.fixture(scope="session")
def ref():
    from tests import oracle_lib
    handle = oracle_lib.reference()
    if handle is None:
        pytest.skip("oracle/_ref/libmf_ref.so not built (needs the reference tree at build time)")
    return handle


@pytest.fixture(scope="session")
def lib():
    from memfabric_hybrid_amd import native
    return native.lib()
